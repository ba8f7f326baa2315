// CHipMathEngine: the interface members beyond the inference and training path of the benchmark networks (what losses,
// ONNX-style operators, embeddings and NeoML's automatic differentiation call). Like the rest of the engine every method
// resolves its handles and calls entry points of the C ABI; semantics are the reference CPU engine's.
#include "HipMathEngine.h"

namespace NeoML {

#define NH_CALL( expr ) check( ( expr ), #expr, __LINE__ )

void CHipMathEngine::VectorFillBernoulli( const CFloatHandle& result, float p, int vectorSize, float value, int seed )
{
	NH_CALL( nhVectorFillBernoulli( stream, raw( result ), p, vectorSize, value, seed ) );
}

void CHipMathEngine::FilterSmallValues( const CFloatHandle& data, int dataSize, float threshold )
{
	NH_CALL( nhFilterSmallValues( stream, raw( data ), dataSize, threshold ) );
}

void CHipMathEngine::VectorSumAdd( const CConstFloatHandle& firstHandle, int vectorSize, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorSumAdd( stream, raw( firstHandle ), vectorSize, raw( resultHandle ) ) );
}

void CHipMathEngine::VectorSumAlongDimension( const CConstFloatHandle& firstHandle, int precedingDimension, int dimension,
	int followingDimension, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorSumAlongDimension( stream, raw( firstHandle ), precedingDimension, dimension, followingDimension, raw( resultHandle ) ) );
}

void CHipMathEngine::VectorCumSumAlongDimension( const CConstFloatHandle& firstHandle, int precedingDimension, int dimension,
	int followingDimension, const CFloatHandle& resultHandle, bool reverse )
{
	NH_CALL( nhVectorCumSumAlongDimension( stream, raw( firstHandle ), precedingDimension, dimension, followingDimension,
		raw( resultHandle ), reverse ? 1 : 0 ) );
}

void CHipMathEngine::VectorCumSumAlongDimension( const CConstIntHandle& firstHandle, int precedingDimension, int dimension,
	int followingDimension, const CIntHandle& resultHandle, bool reverse )
{
	NH_CALL( nhVectorCumSumAlongDimensionInt( stream, raw( firstHandle ), precedingDimension, dimension, followingDimension,
		raw( resultHandle ), reverse ? 1 : 0 ) );
}

void CHipMathEngine::VectorSumAlongDimensionDiag( const CConstFloatHandle& firstHandle, int precedingDimension, int dimension,
	int followingDimension, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorSumAlongDimensionDiag( stream, raw( firstHandle ), precedingDimension, dimension, followingDimension,
		raw( resultHandle ), 0 ) );
}

void CHipMathEngine::VectorCumSumAlongDimensionDiag( const CConstFloatHandle& firstHandle, int precedingDimension, int dimension,
	int followingDimension, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorSumAlongDimensionDiag( stream, raw( firstHandle ), precedingDimension, dimension, followingDimension,
		raw( resultHandle ), 1 ) );
}

void CHipMathEngine::VectorEqual( const CConstIntHandle& firstHandle, const CConstIntHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEqualInt( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEqualValue( const CConstIntHandle& firstHandle, const CFloatHandle& resultHandle, int vectorSize,
	const CConstIntHandle& valueHandle )
{
	NH_CALL( nhVectorEqualValueInt( stream, raw( firstHandle ), raw( resultHandle ), vectorSize, raw( valueHandle ) ) );
}

void CHipMathEngine::VectorMax( const CConstFloatHandle& firstHandle, float secondValue, const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorMax( stream, raw( firstHandle ), secondValue, raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorMaxDiff( const CConstFloatHandle& firstHandle, float secondValue, const CFloatHandle& gradHandle,
	int gradHeight, int gradWidth )
{
	NH_CALL( nhVectorMaxDiff( stream, raw( firstHandle ), secondValue, raw( gradHandle ), gradHeight, gradWidth ) );
}

void CHipMathEngine::VectorAbsDiff( const CConstFloatHandle& sourceGradHandle, int gradHeight, int gradWidth,
	const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorAbsDiffRows( stream, raw( sourceGradHandle ), gradHeight, gradWidth, raw( firstHandle ), raw( resultHandle ) ) );
}

void CHipMathEngine::VectorLogDiff( const CConstFloatHandle& sourceGradHandle, int sourceGradHeight, int sourceGradWidth,
	const CConstFloatHandle& valueHandle, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorLogDiff( stream, raw( sourceGradHandle ), sourceGradHeight, sourceGradWidth, raw( valueHandle ), raw( resultHandle ) ) );
}

void CHipMathEngine::VectorBernulliKLDerivative( const CConstFloatHandle& estimationHandle, const CFloatHandle& resultHandle,
	int vectorSize, const CConstFloatHandle& target )
{
	NH_CALL( nhVectorBernulliKLDerivative( stream, raw( estimationHandle ), raw( resultHandle ), vectorSize, raw( target ) ) );
}

void CHipMathEngine::VectorEltwiseDivide( const CConstIntHandle& firstHandle, const CConstIntHandle& secondHandle,
	const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseDivideInt( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwisePower( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwisePower( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorMinMaxDiff( const CConstFloatHandle& sourceGradHandle, int gradHeight, int gradWidth,
	const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle, const CConstFloatHandle& minHandle,
	const CConstFloatHandle& maxHandle )
{
	NH_CALL( nhVectorMinMaxDiff( stream, raw( sourceGradHandle ), gradHeight, gradWidth, raw( firstHandle ), raw( resultHandle ),
		raw( minHandle ), raw( maxHandle ) ) );
}

void CHipMathEngine::VectorPower( float exponent, const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorPower( stream, exponent, raw( firstHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorPowerDiff( float exponent, const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorPowerDiff( stream, exponent, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorPowerDiffOp( float exponent, const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorPowerDiffOp( stream, exponent, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseNot( const CConstIntHandle& firstHandle, const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseNotInt( stream, raw( firstHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseNotNegative( const CConstIntHandle& firstHanle, const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseNotNegative( stream, raw( firstHanle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseLess( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseLess( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseLess( const CConstFloatHandle& firstHandle, float second, const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseLessValue( stream, raw( firstHandle ), second, raw( resultHandle ), vectorSize, 0 ) );
}

void CHipMathEngine::VectorEltwiseLess( float firstHandle, const CConstFloatHandle& secondHandle, const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseLessValue( stream, raw( secondHandle ), firstHandle, raw( resultHandle ), vectorSize, 1 ) );
}

void CHipMathEngine::VectorEltwiseLess( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseLessToInt( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseLess( const CConstIntHandle& firstHandle, const CConstIntHandle& secondHandle,
	const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseLessInt( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseEqual( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseEqualToInt( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseEqual( const CConstIntHandle& firstHandle, const CConstIntHandle& secondHandle,
	const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseEqualInt( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseWhere( const CConstIntHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CConstFloatHandle& thirdHandle, const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseWhere( stream, raw( firstHandle ), raw( secondHandle ), raw( thirdHandle ), raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorEltwiseWhere( const CConstIntHandle& firstHandle, const CConstIntHandle& secondHandle,
	const CConstIntHandle& thirdHandle, const CIntHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhVectorEltwiseWhere( stream, raw( firstHandle ), raw( secondHandle ), raw( thirdHandle ), raw( resultHandle ), vectorSize ) );
}

// the reference folds the set with its element-wise maximum ( src/CPU/CpuMathEngineVectorMath.cpp:286-301 )
void CHipMathEngine::VectorFindMaxValueInSet( const CConstFloatHandle* vectors, int vectorCount, const CFloatHandle& resultHandle, int vectorSize )
{
	ASSERT_EXPR( vectorCount > 0 );
	if( vectorCount == 1 ) {
		VectorCopy( resultHandle, vectors[0], vectorSize );
		return;
	}
	VectorEltwiseMax( vectors[0], vectors[1], resultHandle, vectorSize );
	for( int i = 2; i < vectorCount; ++i ) {
		VectorEltwiseMax( vectors[i], resultHandle, resultHandle, vectorSize );
	}
}

void CHipMathEngine::VectorFindMaxValueInSet( const CConstFloatHandle* vectors, int vectorCount, const CFloatHandle& resultHandle,
	const CIntHandle& indexHandle, int vectorSize )
{
	ASSERT_EXPR( vectorCount > 0 );
	VectorFill( indexHandle, 0, vectorSize );
	VectorCopy( resultHandle, vectors[0], vectorSize );
	for( int j = 1; j < vectorCount; ++j ) {
		NH_CALL( nhVectorMaxWithIndex( stream, raw( vectors[j] ), raw( resultHandle ), raw( indexHandle ), j, vectorSize ) );
	}
}

void CHipMathEngine::VectorSpreadValues( const CConstFloatHandle& sourceHandle, CFloatHandle* vectors, int vectorCount,
	const CConstIntHandle& indexHandle, int vectorSize )
{
	for( int j = 0; j < vectorCount; ++j ) {
		NH_CALL( nhVectorSpreadValuesTo( stream, raw( sourceHandle ), raw( vectors[j] ), raw( indexHandle ), j, vectorSize ) );
	}
}

} // namespace NeoML
