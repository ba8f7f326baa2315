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

} // namespace NeoML
