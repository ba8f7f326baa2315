// CHipMathEngine: the interface members beyond the inference and training path of the benchmark networks (what losses,
// ONNX-style operators, embeddings and NeoML's automatic differentiation call). Like the rest of the engine every method
// resolves its handles and calls entry points of the C ABI; semantics are the reference CPU engine's.
#include "HipMathEngine.h"

#include <algorithm>
#include <memory>

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

// ---- indexed additions ( one entry point, the mode names the member ) ----------------------------------------

void CHipMathEngine::AddMatrixElementsToVector( const CConstFloatHandle& matrix, int height, int width, const CConstIntHandle& indices,
	const CFloatHandle& result, int vectorSize )
{
	ASSERT_EXPR( vectorSize >= height );
	NH_CALL( nhIndexedAdd( stream, 0, raw( matrix ), raw( result ), height, width, raw( indices ), nullptr ) );
}

void CHipMathEngine::AddMatrixElementsToMatrix( const CConstFloatHandle& matrix, int height, int width, const CFloatHandle& result,
	const CConstIntHandle& indices )
{
	NH_CALL( nhIndexedAdd( stream, 1, raw( matrix ), raw( result ), height, width, raw( indices ), nullptr ) );
}

void CHipMathEngine::AddMatrixElementsToVector( const CConstFloatHandle& matrix, int height, int width, const CConstIntHandle& rowIndices,
	const CConstIntHandle& columnIndices, const CFloatHandle& result, int vectorSize )
{
	NH_CALL( nhIndexedAdd( stream, 2, raw( matrix ), raw( result ), vectorSize, width, raw( rowIndices ), raw( columnIndices ) ) );
}

void CHipMathEngine::AddVectorToMatrixElements( const CFloatHandle& matrix, int height, int width, const CConstIntHandle& indices,
	const CConstFloatHandle& vector )
{
	NH_CALL( nhIndexedAdd( stream, 3, raw( vector ), raw( matrix ), height, width, raw( indices ), nullptr ) );
}

void CHipMathEngine::AddVectorToMatrixElements( const CFloatHandle& matrix, int height, int width, const CConstIntHandle& rowIndices,
	const CConstIntHandle& columnIndices, const CConstFloatHandle& vector, int vectorSize )
{
	NH_CALL( nhIndexedAdd( stream, 4, raw( vector ), raw( matrix ), vectorSize, width, raw( rowIndices ), raw( columnIndices ) ) );
}

// ---- matrices -------------------------------------------------------------------------------------------------

void CHipMathEngine::AddDiagMatrixToMatrix( const CConstFloatHandle& diagMatrix, const CConstFloatHandle& matrix, int height, int width,
	const CFloatHandle& result )
{
	NH_CALL( nhAddDiagMatrixToMatrix( stream, raw( diagMatrix ), raw( matrix ), height, width, raw( result ) ) );
}

void CHipMathEngine::AddVectorToMatrixColumns( const CConstIntHandle& matrixHandle, const CIntHandle& resultHandle, int matrixHeight,
	int matrixWidth, const CConstIntHandle& vectorHandle )
{
	NH_CALL( nhAddVectorToMatrixColumnsInt( stream, raw( matrixHandle ), raw( resultHandle ), matrixHeight, matrixWidth, raw( vectorHandle ) ) );
}

void CHipMathEngine::SumMatrixRows( int batchSize, const CIntHandle& resultHandle, const CConstIntHandle& matrixHandle, int matrixHeight,
	int matrixWidth )
{
	NH_CALL( nhSumMatrixRowsInt( stream, batchSize, raw( resultHandle ), raw( matrixHandle ), matrixHeight, matrixWidth ) );
}

void CHipMathEngine::MatrixColumnsEltwiseDivide( const CConstFloatHandle& matrix, int matrixHeight, int matrixWidth,
	const CConstFloatHandle& vector, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMatrixColumnsEltwiseDivide( stream, raw( matrix ), matrixHeight, matrixWidth, raw( vector ), raw( resultHandle ) ) );
}

void CHipMathEngine::MatrixSoftmaxByColumns( const CConstFloatHandle& matrix, int height, int width, const CFloatHandle& result )
{
	NH_CALL( nhMatrixSoftmaxByColumns( stream, raw( matrix ), height, width, raw( result ) ) );
}

void CHipMathEngine::MatrixSoftmaxDiffOpByColumns( const CConstFloatHandle& first, const CConstFloatHandle& second, int height, int width,
	const CFloatHandle& result )
{
	NH_CALL( nhMatrixSoftmaxDiffOpByColumns( stream, raw( first ), raw( second ), height, width, raw( result ) ) );
}

void CHipMathEngine::FindMinValueInColumns( const CConstFloatHandle& matrixHandle, int matrixHeight, int matrixWidth,
	const CFloatHandle& resultHandle, const CIntHandle& columnIndices )
{
	NH_CALL( nhFindMinValueInColumns( stream, raw( matrixHandle ), matrixHeight, matrixWidth, raw( resultHandle ), raw( columnIndices ) ) );
}

void CHipMathEngine::Multiply1DiagMatrixByMatrix( int batchSize, const CConstFloatHandle& firstHandle, int firstSize,
	const CConstFloatHandle& secondHandle, int secondWidth, const CFloatHandle& resultHandle, int )
{
	NH_CALL( nhMultiply1DiagMatrixByMatrix( stream, batchSize, raw( firstHandle ), firstSize, raw( secondHandle ), secondWidth, raw( resultHandle ) ) );
}

void CHipMathEngine::MatrixRowsToVectorSquaredL2Distance( const CConstFloatHandle& matrixHandle, const int matrixHeight, const int matrixWidth,
	const CConstFloatHandle& vectorHandle, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMatrixRowsToVectorSquaredL2Distance( stream, raw( matrixHandle ), matrixHeight, matrixWidth, raw( vectorHandle ), raw( resultHandle ) ) );
}

void CHipMathEngine::MatrixSpreadRows( const CConstFloatHandle& sourceHandle, int height, int width, const CFloatHandle& resultHandle,
	int resultHeight, const CConstIntHandle& indexHandle, const CConstFloatHandle& fillValue )
{
	NH_CALL( nhMatrixSpreadRows( stream, raw( sourceHandle ), height, width, raw( resultHandle ), resultHeight, raw( indexHandle ),
		fillValue.IsNull() ? nullptr : raw( fillValue ) ) );
}

void CHipMathEngine::MatrixSpreadRows( const CConstIntHandle& sourceHandle, int height, int width, const CIntHandle& resultHandle,
	int resultHeight, const CConstIntHandle& indexHandle, const CConstIntHandle& fillValue )
{
	NH_CALL( nhMatrixSpreadRows( stream, raw( sourceHandle ), height, width, raw( resultHandle ), resultHeight, raw( indexHandle ),
		fillValue.IsNull() ? nullptr : raw( fillValue ) ) );
}

void CHipMathEngine::MatrixSpreadRowsAdd( const CConstFloatHandle& sourceHandle, int height, int width, const CFloatHandle& resultHandle,
	int, const CConstIntHandle& indexHandle )
{
	NH_CALL( nhMatrixSpreadRowsAdd( stream, raw( sourceHandle ), height, width, raw( resultHandle ), raw( indexHandle ) ) );
}

void CHipMathEngine::BuildIntegerHist( const CConstIntHandle& numbersHandle, int numbersCount, const CIntHandle& resultHandle, int maxNumber )
{
	NH_CALL( nhBuildIntegerHist( stream, raw( numbersHandle ), numbersCount, raw( resultHandle ), maxNumber ) );
}

void CHipMathEngine::EnumBinarization( int batchSize, const CConstFloatHandle& inputHandle, int enumSize, const CFloatHandle& resultHandle )
{
	NH_CALL( nhEnumBinarization( stream, batchSize, raw( inputHandle ), 1, enumSize, raw( resultHandle ) ) );
}

void CHipMathEngine::EnumBinarization( int batchSize, const CConstIntHandle& inputHandle, int enumSize, const CFloatHandle& resultHandle )
{
	NH_CALL( nhEnumBinarization( stream, batchSize, raw( inputHandle ), 0, enumSize, raw( resultHandle ) ) );
}

void CHipMathEngine::BitSetBinarization( int batchSize, int bitSetSize, const CConstIntHandle& inputHandle, int outputVectorSize,
	const CFloatHandle& resultHandle )
{
	NH_CALL( nhBitSetBinarization( stream, batchSize, bitSetSize, raw( inputHandle ), outputVectorSize, raw( resultHandle ) ) );
}

// ---- lookups: one launch per table, as the tables are separate blobs ( src/CPU/CpuMathEngineBlas.cpp:432-571 ) ----------

void CHipMathEngine::VectorMultichannelLookupAndCopy( int batchSize, int channelCount, const CConstFloatHandle& inputHandle,
	const CConstFloatHandle* lookupHandles, const CLookupDimension* lookupDimensions, int lookupCount, const CFloatHandle& outputHandle,
	int outputChannels )
{
	int offset = 0;
	for( int j = 0; j < lookupCount; ++j ) {
		NH_CALL( nhLookupAndCopy( stream, batchSize, channelCount, raw( inputHandle ), 1, j, raw( lookupHandles[j] ),
			lookupDimensions[j].VectorCount, lookupDimensions[j].VectorSize, raw( outputHandle ), outputChannels, offset ) );
		offset += lookupDimensions[j].VectorSize;
	}
	if( channelCount > lookupCount ) {
		NH_CALL( nhCopyColumns( stream, batchSize, raw( inputHandle ), channelCount, lookupCount, raw( outputHandle ), outputChannels, offset,
			channelCount - lookupCount ) );
	}
}

void CHipMathEngine::VectorMultichannelLookupAndCopy( int batchSize, int channelCount, const CConstIntHandle& inputHandle,
	const CConstFloatHandle* lookupHandles, const CLookupDimension* lookupDimensions, int lookupCount, const CFloatHandle& outputHandle,
	int outputChannels )
{
	int offset = 0;
	for( int j = 0; j < lookupCount && j < channelCount; ++j ) {
		NH_CALL( nhLookupAndCopy( stream, batchSize, channelCount, raw( inputHandle ), 0, j, raw( lookupHandles[j] ),
			lookupDimensions[j].VectorCount, lookupDimensions[j].VectorSize, raw( outputHandle ), outputChannels, offset ) );
		offset += lookupDimensions[j].VectorSize;
	}
}

void CHipMathEngine::VectorMultichannelLookupAndCopy( int batchSize, int channelCount, const CConstIntHandle& inputHandle,
	const CConstIntHandle* lookupHandles, const CLookupDimension* lookupDimensions, int lookupCount, const CIntHandle& outputHandle,
	int outputChannels )
{
	int offset = 0;
	for( int j = 0; j < lookupCount; ++j ) {
		NH_CALL( nhLookupAndCopy( stream, batchSize, channelCount, raw( inputHandle ), 0, j, raw( lookupHandles[j] ),
			lookupDimensions[j].VectorCount, lookupDimensions[j].VectorSize, raw( outputHandle ), outputChannels, offset ) );
		offset += lookupDimensions[j].VectorSize;
	}
	if( channelCount > lookupCount ) {
		NH_CALL( nhCopyColumns( stream, batchSize, raw( inputHandle ), channelCount, lookupCount, raw( outputHandle ), outputChannels, offset,
			channelCount - lookupCount ) );
	}
}

// the gradient matrix has a row per input row: the tables' vectors side by side, then the unmapped channels
static int lookupMatrixWidth( const CLookupDimension* lookupDimensions, int lookupCount, int channelCount )
{
	int width = 0;
	for( int j = 0; j < lookupCount && j < channelCount; ++j ) {
		width += lookupDimensions[j].VectorSize;
	}
	return width + ( channelCount > lookupCount ? channelCount - lookupCount : 0 );
}

void CHipMathEngine::VectorMultichannelLookupAndAddToTable( int batchSize, int channelCount, const CConstFloatHandle& inputHandle,
	const CFloatHandle* lookupHandles, const CLookupDimension* lookupDimensions, int lookupCount, const CConstFloatHandle& multHandle,
	const CConstFloatHandle& matrixHandle, int )
{
	const int matrixWidth = lookupMatrixWidth( lookupDimensions, lookupCount, channelCount );
	int offset = 0;
	for( int j = 0; j < lookupCount && j < channelCount; ++j ) {
		NH_CALL( nhLookupAndAddToTable( stream, batchSize, channelCount, raw( inputHandle ), 1, j, raw( lookupHandles[j] ),
			lookupDimensions[j].VectorCount, lookupDimensions[j].VectorSize, raw( multHandle ), raw( matrixHandle ), matrixWidth, offset ) );
		offset += lookupDimensions[j].VectorSize;
	}
}

void CHipMathEngine::VectorMultichannelLookupAndAddToTable( int batchSize, int channelCount, const CConstIntHandle& inputHandle,
	const CFloatHandle* lookupHandles, const CLookupDimension* lookupDimensions, int lookupCount, const CConstFloatHandle& multHandle,
	const CConstFloatHandle& matrixHandle, int )
{
	const int matrixWidth = lookupMatrixWidth( lookupDimensions, lookupCount, channelCount );
	int offset = 0;
	for( int j = 0; j < lookupCount && j < channelCount; ++j ) {
		NH_CALL( nhLookupAndAddToTable( stream, batchSize, channelCount, raw( inputHandle ), 0, j, raw( lookupHandles[j] ),
			lookupDimensions[j].VectorCount, lookupDimensions[j].VectorSize, raw( multHandle ), raw( matrixHandle ), matrixWidth, offset ) );
		offset += lookupDimensions[j].VectorSize;
	}
}

void CHipMathEngine::LookupAndSum( const CConstIntHandle& indicesHandle, int batchSize, int indexCount, const CConstFloatHandle& tableHandle,
	int vectorSize, const CFloatHandle& result )
{
	NH_CALL( nhLookupAndSum( stream, raw( indicesHandle ), batchSize, indexCount, raw( tableHandle ), vectorSize, raw( result ) ) );
}

void CHipMathEngine::LookupAndAddToTable( const CConstIntHandle& indicesHandle, int batchSize, int indexCount,
	const CConstFloatHandle& additionsHandle, int vectorSize, const CFloatHandle& tableHandle, int vectorCount )
{
	NH_CALL( nhLookupAndAddToWholeTable( stream, raw( indicesHandle ), batchSize, indexCount, raw( additionsHandle ), vectorSize,
		raw( tableHandle ), vectorCount ) );
}

void CHipMathEngine::MultiplyLookupMatrixByLookupVector( int batchSize, const CLookupMatrix& matrix, const CLookupVector& vector,
	const CFloatHandle& result, int )
{
	ASSERT_EXPR( matrix.Width() == vector.VectorSize() );
	NH_CALL( nhMultiplyLookupMatrixByLookupVector( stream, batchSize, raw( matrix.Table ), raw( matrix.Rows ), matrix.RowCount, matrix.Width(),
		raw( vector.Table ), raw( vector.Vector ), raw( result ) ) );
}

void CHipMathEngine::MultiplyTransposedLookupMatrixByVector( int batchSize, const CLookupMatrix& matrix, const CConstFloatHandle& vectorHandle,
	const CFloatHandle& resultHandle, int )
{
	NH_CALL( nhMultiplyTransposedLookupMatrixByVector( stream, batchSize, raw( matrix.Table ), raw( matrix.Rows ), matrix.RowCount, matrix.Width(),
		raw( vectorHandle ), raw( resultHandle ), 0 ) );
}

void CHipMathEngine::MultiplyTransposedLookupMatrixByVectorAndAdd( int batchSize, const CLookupMatrix& matrix,
	const CConstFloatHandle& vectorHandle, const CFloatHandle& resultHandle, int )
{
	NH_CALL( nhMultiplyTransposedLookupMatrixByVector( stream, batchSize, raw( matrix.Table ), raw( matrix.Rows ), matrix.RowCount, matrix.Width(),
		raw( vectorHandle ), raw( resultHandle ), 1 ) );
}

void CHipMathEngine::MultiplyVectorByTransposedLookupVectorAndAddToTable( int batchSize, const CFloatHandle& tableHandle, int, int vectorSize,
	const CConstIntHandle& indices, const CConstFloatHandle& firstHandle, int firstSize, const CLookupVector& secondVector )
{
	ASSERT_EXPR( vectorSize == secondVector.VectorSize() );
	NH_CALL( nhMultiplyVectorByTransposedLookupVectorAndAddToTable( stream, batchSize, raw( tableHandle ), vectorSize, raw( indices ),
		raw( firstHandle ), firstSize, raw( secondVector.Table ), raw( secondVector.Vector ) ) );
}

// ---- blobs ------------------------------------------------------------------------------------------------------

void CHipMathEngine::AddWidthIndex( const CBlobDesc& source, const CConstFloatHandle& sourceData, bool isForward, const CFloatHandle& result )
{
	NH_CALL( nhAddDimIndex( stream, raw( sourceData ), raw( result ), 1, source.ObjectCount() * source.Height(), source.Width(),
		source.Depth() * source.Channels(), isForward ? 1 : 0 ) );
}

void CHipMathEngine::AddWidthIndex( const CBlobDesc& source, const CConstIntHandle& sourceData, bool isForward, const CIntHandle& result )
{
	NH_CALL( nhAddDimIndex( stream, raw( sourceData ), raw( result ), 0, source.ObjectCount() * source.Height(), source.Width(),
		source.Depth() * source.Channels(), isForward ? 1 : 0 ) );
}

void CHipMathEngine::AddHeightIndex( const CBlobDesc& source, const CConstFloatHandle& sourceData, bool isForward, const CFloatHandle& result )
{
	NH_CALL( nhAddDimIndex( stream, raw( sourceData ), raw( result ), 1, source.ObjectCount(), source.Height(),
		source.Width() * source.Depth() * source.Channels(), isForward ? 1 : 0 ) );
}

void CHipMathEngine::AddHeightIndex( const CBlobDesc& source, const CConstIntHandle& sourceData, bool isForward, const CIntHandle& result )
{
	NH_CALL( nhAddDimIndex( stream, raw( sourceData ), raw( result ), 0, source.ObjectCount(), source.Height(),
		source.Width() * source.Depth() * source.Channels(), isForward ? 1 : 0 ) );
}

void CHipMathEngine::BlobGetSubSequence( const CBlobDesc& from, const CFloatHandle& fromData, const CIntHandle& indexHandle,
	const CBlobDesc& to, const CFloatHandle& toData, int startPos, bool isRev )
{
	ASSERT_EXPR( from.BatchWidth() == to.BatchWidth() && from.ObjectSize() == to.ObjectSize() && from.ListSize() == to.ListSize() );
	NH_CALL( nhBlobGetSubSequence( stream, raw( fromData ), from.BatchLength(), from.BatchWidth(), from.ObjectSize() * from.ListSize(),
		indexHandle.IsNull() ? nullptr : raw( indexHandle ), raw( toData ), to.BatchLength(), startPos, isRev ? 1 : 0 ) );
}

void CHipMathEngine::Upsampling2DForward( const CBlobDesc& input, const CConstIntHandle& inputData, int heightCopyCount, int widthCopyCount,
	const CBlobDesc& result, const CIntHandle& resultData )
{
	ASSERT_EXPR( result.Height() == input.Height() * heightCopyCount && result.Width() == input.Width() * widthCopyCount );
	NH_CALL( nhUpsampling2DForward( stream, input.ObjectCount(), input.Height(), input.Width(), input.Depth() * input.Channels(),
		raw( inputData ), heightCopyCount, widthCopyCount, raw( resultData ) ) );
}

void CHipMathEngine::Upsampling2DForward( const CBlobDesc& input, const CConstFloatHandle& inputData, int heightCopyCount, int widthCopyCount,
	const CBlobDesc& result, const CFloatHandle& resultData )
{
	ASSERT_EXPR( result.Height() == input.Height() * heightCopyCount && result.Width() == input.Width() * widthCopyCount );
	NH_CALL( nhUpsampling2DForward( stream, input.ObjectCount(), input.Height(), input.Width(), input.Depth() * input.Channels(),
		raw( inputData ), heightCopyCount, widthCopyCount, raw( resultData ) ) );
}

void CHipMathEngine::Upsampling2DBackward( const CBlobDesc& input, const CConstFloatHandle& inputData, int heightCopyCount, int widthCopyCount,
	const CBlobDesc& result, const CFloatHandle& resultData )
{
	ASSERT_EXPR( input.Height() == result.Height() * heightCopyCount && input.Width() == result.Width() * widthCopyCount );
	NH_CALL( nhUpsampling2DBackward( stream, input.ObjectCount(), result.Height(), result.Width(), input.Depth() * input.Channels(),
		raw( inputData ), heightCopyCount, widthCopyCount, raw( resultData ) ) );
}

void CHipMathEngine::Reorg( const CBlobDesc& source, const CFloatHandle& sourceData, int stride, bool isForward, const CBlobDesc& result,
	const CFloatHandle& resultData )
{
	const CBlobDesc& dims = isForward ? source : result;
	NH_CALL( nhReorg( stream, raw( sourceData ), stride, isForward ? 1 : 0, source.ObjectCount(), dims.Channels(), dims.Height(), dims.Width(),
		raw( resultData ) ) );
}

void CHipMathEngine::Reorg( const CBlobDesc& source, const CIntHandle& sourceData, int stride, bool isForward, const CBlobDesc& result,
	const CIntHandle& resultData )
{
	const CBlobDesc& dims = isForward ? source : result;
	NH_CALL( nhReorg( stream, raw( sourceData ), stride, isForward ? 1 : 0, source.ObjectCount(), dims.Channels(), dims.Height(), dims.Width(),
		raw( resultData ) ) );
}

void CHipMathEngine::SpaceToDepth( const CBlobDesc& source, const CConstFloatHandle& sourceData, int blockSize, const CBlobDesc& result,
	const CFloatHandle& resultData )
{
	NH_CALL( nhSpaceToDepth( stream, raw( sourceData ), source.ObjectCount() * result.Height(), result.Width(), source.Channels(), blockSize, 1,
		raw( resultData ) ) );
}

void CHipMathEngine::SpaceToDepth( const CBlobDesc& source, const CConstIntHandle& sourceData, int blockSize, const CBlobDesc& result,
	const CIntHandle& resultData )
{
	NH_CALL( nhSpaceToDepth( stream, raw( sourceData ), source.ObjectCount() * result.Height(), result.Width(), source.Channels(), blockSize, 1,
		raw( resultData ) ) );
}

void CHipMathEngine::DepthToSpace( const CBlobDesc& source, const CConstFloatHandle& sourceData, int blockSize, const CBlobDesc& result,
	const CFloatHandle& resultData )
{
	NH_CALL( nhSpaceToDepth( stream, raw( sourceData ), source.ObjectCount() * source.Height(), source.Width(), result.Channels(), blockSize, 0,
		raw( resultData ) ) );
}

void CHipMathEngine::DepthToSpace( const CBlobDesc& source, const CConstIntHandle& sourceData, int blockSize, const CBlobDesc& result,
	const CIntHandle& resultData )
{
	NH_CALL( nhSpaceToDepth( stream, raw( sourceData ), source.ObjectCount() * source.Height(), source.Width(), result.Channels(), blockSize, 0,
		raw( resultData ) ) );
}

// ---- convolution over time: the 2-D convolution with the sequence axis as the height and the batch width as the width
// ---- ( src/CPU/CpuMathEngineDnnTimeConv.cpp:27-208 ); the padding at the back is implied by the result's length ----

struct CHipTimeConvolutionDesc : public CTimeConvolutionDesc {
	nhConvDesc D;
};

CTimeConvolutionDesc* CHipMathEngine::InitTimeConvolution( const CBlobDesc& source, int stride, int paddingFront, int paddingBack,
	int dilation, const CBlobDesc& filter, const CBlobDesc& result )
{
	ASSERT_EXPR( stride > 0 && paddingFront >= 0 && paddingBack >= 0 && dilation > 0 );
	ASSERT_EXPR( filter.BatchLength() == 1 && filter.Width() == 1 && filter.Depth() == 1 );
	ASSERT_EXPR( filter.Channels() == source.ObjectSize() );
	const int span = ( filter.Height() - 1 ) * dilation + 1;
	ASSERT_EXPR( source.BatchLength() + paddingFront + paddingBack >= span );
	ASSERT_EXPR( result.BatchLength() == ( source.BatchLength() - span + paddingFront + paddingBack ) / stride + 1 );
	ASSERT_EXPR( result.BatchWidth() == source.BatchWidth() && result.ListSize() == 1 && source.ListSize() == 1 );
	ASSERT_EXPR( result.Width() == 1 && result.Height() == 1 && result.Depth() == 1 && result.Channels() == filter.BatchWidth() );
	ASSERT_EXPR( paddingFront < span && paddingBack < span );
	std::unique_ptr<CHipTimeConvolutionDesc> desc( new CHipTimeConvolutionDesc() );
	nhConvDesc& d = desc->D;
	d.batch = 1;
	d.height = source.BatchLength();
	d.width = source.BatchWidth();
	d.channels = source.ObjectSize();
	d.filterCount = filter.BatchWidth();
	d.filterHeight = filter.Height();
	d.filterWidth = 1;
	d.paddingHeight = paddingFront;
	d.paddingWidth = 0;
	d.strideHeight = stride;
	d.strideWidth = 1;
	d.dilationHeight = dilation;
	d.dilationWidth = 1;
	d.resultHeight = result.BatchLength();
	d.resultWidth = source.BatchWidth();
	return desc.release();
}

void CHipMathEngine::BlobTimeConvolution( const CTimeConvolutionDesc& desc, const CConstFloatHandle& source, const CConstFloatHandle& filter,
	const CConstFloatHandle& freeTerm, const CFloatHandle& result )
{
	const CHipTimeConvolutionDesc& d = static_cast<const CHipTimeConvolutionDesc&>( desc );
	NH_CALL( nhBlobConvolution( stream, &d.D, raw( source ), raw( filter ), raw( freeTerm ), raw( result ) ) );
}

// ( the free term does not enter the input's gradient, :117-166 )
void CHipMathEngine::BlobTimeConvolutionBackward( const CTimeConvolutionDesc& desc, const CConstFloatHandle& outputDiff,
	const CConstFloatHandle& filter, const CConstFloatHandle&, const CFloatHandle& inputDiff )
{
	const CHipTimeConvolutionDesc& d = static_cast<const CHipTimeConvolutionDesc&>( desc );
	size_t workspaceSize = 0;
	NH_CALL( nhBlobConvolutionBackwardWorkspaceSize( &d.D, &workspaceSize ) );
	const CMemoryHandle workspace = StackAlloc( std::max<size_t>( workspaceSize, 16 ) );
	NH_CALL( nhBlobConvolutionBackward( stream, &d.D, raw( outputDiff ), raw( filter ), nullptr, raw( inputDiff ), rawBytes( workspace ),
		workspaceSize ) );
	StackFree( workspace );
}

void CHipMathEngine::BlobTimeConvolutionLearnAdd( const CTimeConvolutionDesc& desc, const CConstFloatHandle& input,
	const CConstFloatHandle& outputDiff, const CFloatHandle& filterDiff, const CFloatHandle& freeTermDiff )
{
	const CHipTimeConvolutionDesc& d = static_cast<const CHipTimeConvolutionDesc&>( desc );
	NH_CALL( nhBlobConvolutionLearnAdd( stream, &d.D, raw( input ), raw( outputDiff ), raw( filterDiff ) ) );
	SumMatrixRowsAdd( 1, freeTermDiff, outputDiff, d.D.resultHeight * d.D.resultWidth, d.D.filterCount );
}

// ---- poolings over an object and over time ---------------------------------------------------------------------

struct CHipGlobalMaxPoolingDesc : public CGlobalMaxPoolingDesc {
	int Objects, PoolSize, Channels, MaxCount;
};

CGlobalMaxPoolingDesc* CHipMathEngine::InitGlobalMaxPooling( const CBlobDesc& source, const CBlobDesc& maxIndices, const CBlobDesc& result )
{
	ASSERT_EXPR( result.ObjectCount() == source.ObjectCount() && result.Channels() == source.Channels() );
	ASSERT_EXPR( maxIndices.BlobSize() == result.BlobSize() );
	std::unique_ptr<CHipGlobalMaxPoolingDesc> desc( new CHipGlobalMaxPoolingDesc() );
	desc->Objects = source.ObjectCount();
	desc->PoolSize = source.Height() * source.Width() * source.Depth();
	desc->Channels = source.Channels();
	desc->MaxCount = result.Height() * result.Width() * result.Depth();
	return desc.release();
}

void CHipMathEngine::BlobGlobalMaxPooling( const CGlobalMaxPoolingDesc& desc, const CConstFloatHandle& source, const CIntHandle& maxIndices,
	const CFloatHandle& result )
{
	const CHipGlobalMaxPoolingDesc& d = static_cast<const CHipGlobalMaxPoolingDesc&>( desc );
	NH_CALL( nhBlobGlobalMaxPooling( stream, d.Objects, d.PoolSize, d.Channels, d.MaxCount, raw( source ), raw( maxIndices ), raw( result ) ) );
}

void CHipMathEngine::BlobGlobalMaxPoolingBackward( const CGlobalMaxPoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CConstIntHandle& maxIndices, const CFloatHandle& sourceDiff )
{
	const CHipGlobalMaxPoolingDesc& d = static_cast<const CHipGlobalMaxPoolingDesc&>( desc );
	NH_CALL( nhBlobGlobalMaxPoolingBackward( stream, d.Objects, d.PoolSize, d.Channels, d.MaxCount, raw( resultDiff ), raw( maxIndices ),
		raw( sourceDiff ) ) );
}

struct CHipMaxOverTimePoolingDesc : public CMaxOverTimePoolingDesc {
	int SourceLength, ResultLength, SeqElemSize, FilterLen, StrideLen;
};

CMaxOverTimePoolingDesc* CHipMathEngine::InitMaxOverTimePooling( const CBlobDesc& source, int filterLen, int strideLen, const CBlobDesc& result )
{
	ASSERT_EXPR( filterLen > 0 && strideLen > 0 && source.BatchLength() >= filterLen );
	ASSERT_EXPR( result.BatchLength() == ( source.BatchLength() - filterLen ) / strideLen + 1 );
	ASSERT_EXPR( result.BatchWidth() == source.BatchWidth() && result.ObjectSize() == source.ObjectSize() );
	std::unique_ptr<CHipMaxOverTimePoolingDesc> desc( new CHipMaxOverTimePoolingDesc() );
	desc->SourceLength = source.BatchLength();
	desc->ResultLength = result.BatchLength();
	desc->SeqElemSize = source.BlobSize() / source.BatchLength();
	desc->FilterLen = filterLen;
	desc->StrideLen = strideLen;
	return desc.release();
}

void CHipMathEngine::BlobMaxOverTimePooling( const CMaxOverTimePoolingDesc& desc, const CConstFloatHandle& source, const CIntHandle* maxIndices,
	const CFloatHandle& result )
{
	const CHipMaxOverTimePoolingDesc& d = static_cast<const CHipMaxOverTimePoolingDesc&>( desc );
	NH_CALL( nhBlobMaxOverTimePooling( stream, d.SourceLength, d.SeqElemSize, d.FilterLen, d.StrideLen, raw( source ),
		maxIndices != nullptr ? raw( *maxIndices ) : nullptr, raw( result ) ) );
}

void CHipMathEngine::BlobMaxOverTimePoolingBackward( const CMaxOverTimePoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CConstIntHandle& maxIndices, const CFloatHandle& sourceDiff )
{
	const CHipMaxOverTimePoolingDesc& d = static_cast<const CHipMaxOverTimePoolingDesc&>( desc );
	NH_CALL( nhBlobOverTimePoolingBackward( stream, d.SourceLength, d.ResultLength, d.SeqElemSize, raw( resultDiff ), raw( maxIndices ),
		raw( sourceDiff ), 0 ) );
}

struct CHipGlobalMaxOverTimePoolingDesc : public CGlobalMaxOverTimePoolingDesc {
	int SourceLength, SeqElemSize;
};

CGlobalMaxOverTimePoolingDesc* CHipMathEngine::InitGlobalMaxOverTimePooling( const CBlobDesc& source, const CBlobDesc& result )
{
	ASSERT_EXPR( result.BatchLength() == 1 && result.BatchWidth() == source.BatchWidth() && result.ObjectSize() == source.ObjectSize() );
	std::unique_ptr<CHipGlobalMaxOverTimePoolingDesc> desc( new CHipGlobalMaxOverTimePoolingDesc() );
	desc->SourceLength = source.BatchLength();
	desc->SeqElemSize = source.BatchWidth() * source.ObjectSize();
	return desc.release();
}

// the maximum of every column of [length][batch width x object size], the first of equal maxima keeps its step
// ( src/CPU/CpuMathEngineDnnPooling.cpp:274-298 )
void CHipMathEngine::BlobGlobalMaxOverTimePooling( const CGlobalMaxOverTimePoolingDesc& desc, const CConstFloatHandle& source,
	const CIntHandle* maxIndices, const CFloatHandle& result )
{
	const CHipGlobalMaxOverTimePoolingDesc& d = static_cast<const CHipGlobalMaxOverTimePoolingDesc&>( desc );
	NH_CALL( nhBlobMaxOverTimePooling( stream, d.SourceLength, d.SeqElemSize, d.SourceLength, 1, raw( source ),
		maxIndices != nullptr ? raw( *maxIndices ) : nullptr, raw( result ) ) );
}

void CHipMathEngine::BlobGlobalMaxOverTimePoolingBackward( const CGlobalMaxOverTimePoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CConstIntHandle& maxIndices, const CFloatHandle& sourceDiff )
{
	const CHipGlobalMaxOverTimePoolingDesc& d = static_cast<const CHipGlobalMaxOverTimePoolingDesc&>( desc );
	NH_CALL( nhBlobOverTimePoolingBackward( stream, d.SourceLength, 1, d.SeqElemSize, raw( resultDiff ), raw( maxIndices ), raw( sourceDiff ), 1 ) );
}

void CHipMathEngine::LinearInterpolation( const CConstFloatHandle& dataHandle, const CFloatHandle& resultHandle, TInterpolationCoords coords,
	TInterpolationRound round, int objectCount, int scaledAxis, int objectSize, float scale )
{
	NH_CALL( nhLinearInterpolation( stream, raw( dataHandle ), raw( resultHandle ), static_cast<int>( coords ), static_cast<int>( round ),
		objectCount, scaledAxis, objectSize, scale ) );
}

void CHipMathEngine::ScatterND( const CConstIntHandle& indicesHandle, const CConstFloatHandle& updatesHandle, const CFloatHandle& dataHandle,
	const CBlobDesc& dataDesc, int updateCount, int indexDims )
{
	nhBlobDesc desc;
	for( int i = 0; i < 7; ++i ) {
		desc.dims[i] = dataDesc.DimSize( i );
	}
	NH_CALL( nhScatterND( stream, raw( indicesHandle ), raw( updatesHandle ), raw( dataHandle ), &desc, updateCount, indexDims ) );
}

void CHipMathEngine::ScatterND( const CConstIntHandle& indicesHandle, const CConstIntHandle& updatesHandle, const CIntHandle& dataHandle,
	const CBlobDesc& dataDesc, int updateCount, int indexDims )
{
	nhBlobDesc desc;
	for( int i = 0; i < 7; ++i ) {
		desc.dims[i] = dataDesc.DimSize( i );
	}
	NH_CALL( nhScatterND( stream, raw( indicesHandle ), raw( updatesHandle ), raw( dataHandle ), &desc, updateCount, indexDims ) );
}

} // namespace NeoML
