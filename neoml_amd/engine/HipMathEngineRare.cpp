// CHipMathEngine: the interface members that no network of the benchmark configurations calls (the recurrent parts of
// QRNN and IndRNN, BERT's light-weight convolution, local response normalization, products with a sparse matrix, top-k,
// 3-D convolution and pooling, convolution over run-length encoded images). Every method resolves its handles and calls
// entry points of the C ABI; semantics are the reference CPU engine's.
#include "HipMathEngine.h"

#include <memory>

namespace NeoML {

#define NH_CALL( expr ) check( ( expr ), #expr, __LINE__ )

// an optional handle as a pointer
#define OPTIONAL( handle ) ( ( handle ).IsNull() ? nullptr : raw( handle ) )

void CHipMathEngine::QrnnFPooling( bool reverse, int sequenceLength, int objectSize, const CConstFloatHandle& update,
	const CConstFloatHandle& forget, const CConstFloatHandle& initialState, const CFloatHandle& result )
{
	NH_CALL( nhQrnnFPooling( stream, reverse ? 1 : 0, sequenceLength, objectSize, raw( update ), raw( forget ), OPTIONAL( initialState ),
		raw( result ) ) );
}

void CHipMathEngine::QrnnFPoolingBackward( bool reverse, int sequenceLength, int objectSize, const CConstFloatHandle& update,
	const CConstFloatHandle& forget, const CConstFloatHandle& initialState, const CConstFloatHandle& result, const CFloatHandle& resultDiff,
	const CFloatHandle& updateDiff, const CFloatHandle& forgetDiff )
{
	NH_CALL( nhQrnnFPoolingBackward( stream, reverse ? 1 : 0, sequenceLength, objectSize, raw( update ), raw( forget ),
		OPTIONAL( initialState ), raw( result ), raw( resultDiff ), raw( updateDiff ), raw( forgetDiff ) ) );
}

void CHipMathEngine::QrnnIfPooling( bool reverse, int sequenceLength, int objectSize, const CConstFloatHandle& update,
	const CConstFloatHandle& forget, const CConstFloatHandle& input, const CConstFloatHandle& initialState, const CFloatHandle& result )
{
	NH_CALL( nhQrnnIfPooling( stream, reverse ? 1 : 0, sequenceLength, objectSize, raw( update ), raw( forget ), raw( input ),
		OPTIONAL( initialState ), raw( result ) ) );
}

void CHipMathEngine::QrnnIfPoolingBackward( bool reverse, int sequenceLength, int objectSize, const CConstFloatHandle& update,
	const CConstFloatHandle& forget, const CConstFloatHandle& input, const CConstFloatHandle& initialState, const CConstFloatHandle& result,
	const CFloatHandle& resultDiff, const CFloatHandle& updateDiff, const CFloatHandle& forgetDiff, const CFloatHandle& inputDiff )
{
	NH_CALL( nhQrnnIfPoolingBackward( stream, reverse ? 1 : 0, sequenceLength, objectSize, raw( update ), raw( forget ), raw( input ),
		OPTIONAL( initialState ), raw( result ), raw( resultDiff ), raw( updateDiff ), raw( forgetDiff ), raw( inputDiff ) ) );
}

static int indRnnActivation( TActivationFunction activation )
{
	ASSERT_EXPR( activation == AF_Sigmoid || activation == AF_ReLU );
	return activation == AF_ReLU ? NH_INDRNN_RELU : NH_INDRNN_SIGMOID;
}

void CHipMathEngine::IndRnnRecurrent( bool reverse, int sequenceLength, int batchSize, int objectSize, TActivationFunction activation,
	const CConstFloatHandle& wx, const CConstFloatHandle& mask, const CConstFloatHandle& u, const CFloatHandle& h )
{
	NH_CALL( nhIndRnnRecurrent( stream, reverse ? 1 : 0, sequenceLength, batchSize, objectSize, indRnnActivation( activation ), raw( wx ),
		OPTIONAL( mask ), raw( u ), raw( h ) ) );
}

void CHipMathEngine::IndRnnRecurrentBackward( bool reverse, int sequenceLength, int batchSize, int objectSize,
	TActivationFunction activation, const CConstFloatHandle& mask, const CConstFloatHandle& u, const CConstFloatHandle& h,
	const CConstFloatHandle& hDiff, const CFloatHandle& wxDiff )
{
	NH_CALL( nhIndRnnRecurrentBackward( stream, reverse ? 1 : 0, sequenceLength, batchSize, objectSize, indRnnActivation( activation ),
		OPTIONAL( mask ), raw( u ), raw( h ), raw( hDiff ), raw( wxDiff ) ) );
}

void CHipMathEngine::IndRnnRecurrentLearn( bool reverse, int sequenceLength, int batchSize, int objectSize,
	TActivationFunction activation, const CConstFloatHandle& mask, const CConstFloatHandle& u, const CConstFloatHandle& h,
	const CConstFloatHandle& hDiff, const CFloatHandle& uDiff )
{
	NH_CALL( nhIndRnnRecurrentLearn( stream, reverse ? 1 : 0, sequenceLength, batchSize, objectSize, indRnnActivation( activation ),
		OPTIONAL( mask ), raw( u ), raw( h ), raw( hDiff ), raw( uDiff ) ) );
}

void CHipMathEngine::BertConv( const CConstFloatHandle& dataHandle, const CConstFloatHandle& kernelHandle, int seqLen, int batchSize,
	int numHeads, int headSize, int kernelSize, const CFloatHandle& outputHandle )
{
	NH_CALL( nhBertConv( stream, raw( dataHandle ), raw( kernelHandle ), seqLen, batchSize, numHeads, headSize, kernelSize,
		raw( outputHandle ) ) );
}

void CHipMathEngine::BertConvBackward( const CConstFloatHandle& dataHandle, const CConstFloatHandle& kernelHandle,
	const CConstFloatHandle& outDiffHandle, int seqLen, int batchSize, int numHeads, int headSize, int kernelSize,
	const CFloatHandle& dataDiffHandle, const CFloatHandle& kernelDiffHandle )
{
	NH_CALL( nhBertConvBackward( stream, raw( dataHandle ), raw( kernelHandle ), raw( outDiffHandle ), seqLen, batchSize, numHeads, headSize,
		kernelSize, raw( dataDiffHandle ), raw( kernelDiffHandle ) ) );
}

struct CHipLrnDesc : public CLrnDesc {
	int VectorCount, VectorSize, WindowSize;
	float Bias, Alpha, Beta;
};

CLrnDesc* CHipMathEngine::InitLrn( const CBlobDesc& source, int windowSize, float bias, float alpha, float beta )
{
	ASSERT_EXPR( windowSize > 0 );
	std::unique_ptr<CHipLrnDesc> desc( new CHipLrnDesc() );
	desc->VectorCount = source.ObjectCount() * source.GeometricalSize();
	desc->VectorSize = source.Channels();
	desc->WindowSize = windowSize;
	desc->Bias = bias;
	desc->Alpha = alpha;
	desc->Beta = beta;
	return desc.release();
}

void CHipMathEngine::Lrn( const CLrnDesc& desc, const CConstFloatHandle& input, const CFloatHandle& invSum, const CFloatHandle& invSumBeta,
	const CFloatHandle& outputHandle )
{
	const CHipLrnDesc& d = static_cast<const CHipLrnDesc&>( desc );
	NH_CALL( nhLrn( stream, raw( input ), d.VectorCount, d.VectorSize, d.WindowSize, d.Bias, d.Alpha, d.Beta, OPTIONAL( invSum ),
		OPTIONAL( invSumBeta ), raw( outputHandle ) ) );
}

void CHipMathEngine::LrnBackward( const CLrnDesc& desc, const CConstFloatHandle& input, const CConstFloatHandle& output,
	const CConstFloatHandle& outputDiff, const CConstFloatHandle& invSum, const CConstFloatHandle& invSumBeta, const CFloatHandle& inputDiff )
{
	const CHipLrnDesc& d = static_cast<const CHipLrnDesc&>( desc );
	NH_CALL( nhLrnBackward( stream, raw( input ), raw( output ), raw( outputDiff ), raw( invSum ), raw( invSumBeta ), d.VectorCount,
		d.VectorSize, d.WindowSize, d.Alpha, d.Beta, raw( inputDiff ) ) );
}

void CHipMathEngine::MultiplySparseMatrixByTransposedMatrix( int firstHeight, int firstWidth, int secondHeight,
	const CSparseMatrixDesc& firstDesc, const CConstFloatHandle& secondHandle, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMultiplySparseMatrixByTransposedMatrix( stream, firstHeight, firstWidth, secondHeight, raw( firstDesc.Rows ),
		OPTIONAL( firstDesc.Columns ), OPTIONAL( firstDesc.Values ), raw( secondHandle ), raw( resultHandle ) ) );
}

void CHipMathEngine::MultiplyTransposedMatrixBySparseMatrix( int firstHeight, int firstWidth, int resultWidth,
	const CConstFloatHandle& firstHandle, const CSparseMatrixDesc& secondDesc, const CFloatHandle& resultHandle, bool isTransposedSparse )
{
	NH_CALL( nhMultiplyTransposedMatrixBySparseMatrix( stream, firstHeight, firstWidth, resultWidth, raw( firstHandle ),
		raw( secondDesc.Rows ), OPTIONAL( secondDesc.Columns ), OPTIONAL( secondDesc.Values ), raw( resultHandle ),
		isTransposedSparse ? 1 : 0, 0 ) );
}

void CHipMathEngine::MultiplyTransposedMatrixBySparseMatrixAndAdd( int firstHeight, int firstWidth, int secondWidth,
	const CConstFloatHandle& firstHandle, const CSparseMatrixDesc& secondDesc, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMultiplyTransposedMatrixBySparseMatrix( stream, firstHeight, firstWidth, secondWidth, raw( firstHandle ),
		raw( secondDesc.Rows ), OPTIONAL( secondDesc.Columns ), OPTIONAL( secondDesc.Values ), raw( resultHandle ), 0, 1 ) );
}

void CHipMathEngine::MultiplySparseMatrixByMatrix( int firstHeight, int firstWidth, int secondWidth, const CSparseMatrixDesc& firstDesc,
	const CConstFloatHandle& secondHandle, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMultiplySparseMatrixByMatrix( stream, firstHeight, firstWidth, secondWidth, raw( firstDesc.Rows ),
		OPTIONAL( firstDesc.Columns ), OPTIONAL( firstDesc.Values ), raw( secondHandle ), raw( resultHandle ) ) );
}

void CHipMathEngine::MultiplyTransposedSparseMatrixByMatrix( int firstHeight, int firstWidth, int secondWidth,
	const CSparseMatrixDesc& firstDesc, const CConstFloatHandle& secondHandle, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMultiplyTransposedSparseMatrixByMatrix( stream, firstHeight, firstWidth, secondWidth, raw( firstDesc.Rows ),
		OPTIONAL( firstDesc.Columns ), OPTIONAL( firstDesc.Values ), raw( secondHandle ), raw( resultHandle ) ) );
}

void CHipMathEngine::VectorTopK( const CConstFloatHandle& first, int firstSize, int k, const CFloatHandle& result, const CIntHandle& indices )
{
	NH_CALL( nhVectorTopK( stream, raw( first ), firstSize, k, raw( result ), raw( indices ) ) );
}

void CHipMathEngine::VectorTopKDiff( const CConstFloatHandle& sourceGrad, int sourceGradHeight, int sourceGradWidth,
	const CConstIntHandle& indices, int k, const CFloatHandle& resultGrad )
{
	NH_CALL( nhVectorTopKDiff( stream, raw( sourceGrad ), sourceGradHeight, sourceGradWidth, raw( indices ), k, raw( resultGrad ) ) );
}

void CHipMathEngine::CtcLossForward( int resultLen, int batchSize, int classCount, int labelLen, int blankLabel, bool skipBlanks,
	const CConstFloatHandle& result, const CConstIntHandle& labels, const CConstIntHandle& labelLens, const CConstIntHandle& resultLens,
	const CConstFloatHandle& labelWeights, const CFloatHandle& loss, const CFloatHandle& lossGradient )
{
	size_t workspaceSize = 0;
	NH_CALL( nhCtcLossWorkspaceSize( resultLen, batchSize, classCount, labelLen, &workspaceSize ) );
	const CMemoryHandle workspace = StackAlloc( workspaceSize );
	NH_CALL( nhCtcLossForward( stream, resultLen, batchSize, classCount, labelLen, blankLabel, skipBlanks ? 1 : 0, raw( result ),
		OPTIONAL( labels ), OPTIONAL( labelLens ), OPTIONAL( resultLens ), OPTIONAL( labelWeights ), raw( loss ), OPTIONAL( lossGradient ),
		rawBytes( workspace ), workspaceSize ) );
	StackFree( workspace );
}

// ---- 3-D convolution and pooling ---------------------------------------------------------------------------------

struct CHip3dConvolutionDesc : public C3dConvolutionDesc {
	nh3dDesc D;
};
struct CHip3dMaxPoolingDesc : public C3dMaxPoolingDesc {
	nh3dDesc D;
};
struct CHip3dMeanPoolingDesc : public C3dMeanPoolingDesc {
	nh3dDesc D;
};

static void fill3dDesc( nh3dDesc& d, const CBlobDesc& source, int filterCount, int filterHeight, int filterWidth, int filterDepth,
	int paddingHeight, int paddingWidth, int paddingDepth, int strideHeight, int strideWidth, int strideDepth, const CBlobDesc& result )
{
	d.batch = source.ObjectCount();
	d.height = source.Height();
	d.width = source.Width();
	d.depth = source.Depth();
	d.channels = source.Channels();
	d.filterCount = filterCount;
	d.filterHeight = filterHeight;
	d.filterWidth = filterWidth;
	d.filterDepth = filterDepth;
	d.paddingHeight = paddingHeight;
	d.paddingWidth = paddingWidth;
	d.paddingDepth = paddingDepth;
	d.strideHeight = strideHeight;
	d.strideWidth = strideWidth;
	d.strideDepth = strideDepth;
	d.resultHeight = result.Height();
	d.resultWidth = result.Width();
	d.resultDepth = result.Depth();
}

C3dConvolutionDesc* CHipMathEngine::InitBlob3dConvolution( const CBlobDesc& input, int paddingHeight, int paddingWidth, int paddingDepth,
	int strideHeight, int strideWidth, int strideDepth, const CBlobDesc& filter, const CBlobDesc& output )
{
	ASSERT_EXPR( filter.Channels() == input.Channels() && output.Channels() == filter.ObjectCount() );
	ASSERT_EXPR( output.ObjectCount() == input.ObjectCount() );
	std::unique_ptr<CHip3dConvolutionDesc> desc( new CHip3dConvolutionDesc() );
	fill3dDesc( desc->D, input, filter.ObjectCount(), filter.Height(), filter.Width(), filter.Depth(), paddingHeight, paddingWidth,
		paddingDepth, strideHeight, strideWidth, strideDepth, output );
	return desc.release();
}

void CHipMathEngine::Blob3dConvolution( const C3dConvolutionDesc& desc, const CConstFloatHandle& source, const CConstFloatHandle& filter,
	const CConstFloatHandle* freeTerm, const CFloatHandle& result )
{
	const CHip3dConvolutionDesc& d = static_cast<const CHip3dConvolutionDesc&>( desc );
	NH_CALL( nhBlob3dConvolution( stream, &d.D, raw( source ), raw( filter ), freeTerm != nullptr ? raw( *freeTerm ) : nullptr, raw( result ) ) );
}

void CHipMathEngine::Blob3dConvolutionBackward( const C3dConvolutionDesc& desc, const CConstFloatHandle& source,
	const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm, const CFloatHandle& result )
{
	const CHip3dConvolutionDesc& d = static_cast<const CHip3dConvolutionDesc&>( desc );
	NH_CALL( nhBlob3dConvolutionBackward( stream, &d.D, raw( source ), raw( filter ), freeTerm != nullptr ? raw( *freeTerm ) : nullptr,
		raw( result ) ) );
}

void CHipMathEngine::Blob3dConvolutionLearnAdd( const C3dConvolutionDesc& desc, const CConstFloatHandle& input,
	const CConstFloatHandle& outputDiff, const CFloatHandle& filterDiff, const CFloatHandle* freeTermDiff, bool isFreeTermDiffFromInput )
{
	const CHip3dConvolutionDesc& d = static_cast<const CHip3dConvolutionDesc&>( desc );
	NH_CALL( nhBlob3dConvolutionLearnAdd( stream, &d.D, raw( input ), raw( outputDiff ), raw( filterDiff ),
		freeTermDiff != nullptr ? raw( *freeTermDiff ) : nullptr, isFreeTermDiffFromInput ? 1 : 0 ) );
}

C3dMaxPoolingDesc* CHipMathEngine::Init3dMaxPooling( const CBlobDesc& source, int filterHeight, int filterWidth, int filterDepth,
	int strideHeight, int strideWidth, int strideDepth, const CBlobDesc& result )
{
	ASSERT_EXPR( result.ObjectCount() == source.ObjectCount() && result.Channels() == source.Channels() );
	std::unique_ptr<CHip3dMaxPoolingDesc> desc( new CHip3dMaxPoolingDesc() );
	fill3dDesc( desc->D, source, 0, filterHeight, filterWidth, filterDepth, 0, 0, 0, strideHeight, strideWidth, strideDepth, result );
	return desc.release();
}

void CHipMathEngine::Blob3dMaxPooling( const C3dMaxPoolingDesc& desc, const CConstFloatHandle& source, const CIntHandle* maxIndices,
	const CFloatHandle& result )
{
	const CHip3dMaxPoolingDesc& d = static_cast<const CHip3dMaxPoolingDesc&>( desc );
	NH_CALL( nhBlob3dMaxPooling( stream, &d.D, raw( source ), maxIndices != nullptr ? raw( *maxIndices ) : nullptr, raw( result ) ) );
}

void CHipMathEngine::Blob3dMaxPoolingBackward( const C3dMaxPoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CConstIntHandle& maxIndices, const CFloatHandle& sourceDiff )
{
	const CHip3dMaxPoolingDesc& d = static_cast<const CHip3dMaxPoolingDesc&>( desc );
	NH_CALL( nhBlob3dMaxPoolingBackward( stream, &d.D, raw( resultDiff ), raw( maxIndices ), raw( sourceDiff ) ) );
}

C3dMeanPoolingDesc* CHipMathEngine::Init3dMeanPooling( const CBlobDesc& source, int filterHeight, int filterWidth, int filterDepth,
	int strideHeight, int strideWidth, int strideDepth, const CBlobDesc& result )
{
	ASSERT_EXPR( result.ObjectCount() == source.ObjectCount() && result.Channels() == source.Channels() );
	std::unique_ptr<CHip3dMeanPoolingDesc> desc( new CHip3dMeanPoolingDesc() );
	fill3dDesc( desc->D, source, 0, filterHeight, filterWidth, filterDepth, 0, 0, 0, strideHeight, strideWidth, strideDepth, result );
	return desc.release();
}

void CHipMathEngine::Blob3dMeanPooling( const C3dMeanPoolingDesc& desc, const CConstFloatHandle& source, const CFloatHandle& result )
{
	const CHip3dMeanPoolingDesc& d = static_cast<const CHip3dMeanPoolingDesc&>( desc );
	NH_CALL( nhBlob3dMeanPooling( stream, &d.D, raw( source ), raw( result ) ) );
}

void CHipMathEngine::Blob3dMeanPoolingBackward( const C3dMeanPoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CFloatHandle& sourceDiff )
{
	const CHip3dMeanPoolingDesc& d = static_cast<const CHip3dMeanPoolingDesc&>( desc );
	NH_CALL( nhBlob3dMeanPoolingBackward( stream, &d.D, raw( resultDiff ), raw( sourceDiff ) ) );
}

// ---- convolution over run-length encoded images: the images are decoded into a blob of stroke / non-stroke values on the
// stack, the ordinary convolution does the rest ( the reference's GPU engine does the same, CudaMathEngineDnnRleConv.cu:83-106 )

struct CHipRleConvolutionDesc : public CRleConvolutionDesc {
	std::unique_ptr<CConvolutionDesc> Conv;
	int Batch, Height, Width;
	float StrokeValue, NonStrokeValue;
};

CRleConvolutionDesc* CHipMathEngine::InitBlobRleConvolution( const CBlobDesc& input, float strokeValue, float nonStrokeValue,
	int strideHeight, int strideWidth, const CBlobDesc& filter, const CBlobDesc& output )
{
	ASSERT_EXPR( input.Depth() == 1 && input.Channels() == 1 && filter.Depth() == 1 && filter.Channels() == 1 );
	ASSERT_EXPR( input.Width() <= MaxRleConvImageWidth && filter.Width() <= MaxRleConvFilterWidth );
	std::unique_ptr<CHipRleConvolutionDesc> desc( new CHipRleConvolutionDesc() );
	desc->Conv.reset( InitBlobConvolution( input, 0, 0, strideHeight, strideWidth, 1, 1, filter, output ) );
	desc->Batch = input.ObjectCount();
	desc->Height = input.Height();
	desc->Width = input.Width();
	desc->StrokeValue = strokeValue;
	desc->NonStrokeValue = nonStrokeValue;
	return desc.release();
}

void CHipMathEngine::BlobRleConvolution( const CRleConvolutionDesc& desc, const CConstFloatHandle& source, const CConstFloatHandle& filter,
	const CConstFloatHandle* freeTerm, const CFloatHandle& result )
{
	const CHipRleConvolutionDesc& d = static_cast<const CHipRleConvolutionDesc&>( desc );
	const size_t count = static_cast<size_t>( d.Batch ) * d.Height * d.Width;
	const CFloatHandle dense( StackAlloc( count * sizeof( float ) ) );
	NH_CALL( nhRleImagesToDense( stream, raw( source ), d.Batch, d.Height, d.Width, d.StrokeValue, d.NonStrokeValue, raw( dense ) ) );
	BlobConvolution( *d.Conv, dense, filter, freeTerm, result );
	StackFree( dense );
}

void CHipMathEngine::BlobRleConvolutionLearnAdd( const CRleConvolutionDesc& desc, const CConstFloatHandle& input,
	const CConstFloatHandle& outputDiff, const CFloatHandle& filterDiff, const CFloatHandle* freeTermDiff )
{
	const CHipRleConvolutionDesc& d = static_cast<const CHipRleConvolutionDesc&>( desc );
	const size_t count = static_cast<size_t>( d.Batch ) * d.Height * d.Width;
	const CFloatHandle dense( StackAlloc( count * sizeof( float ) ) );
	NH_CALL( nhRleImagesToDense( stream, raw( input ), d.Batch, d.Height, d.Width, d.StrokeValue, d.NonStrokeValue, raw( dense ) ) );
	BlobConvolutionLearnAdd( *d.Conv, dense, outputDiff, filterDiff, freeTermDiff, false );
	StackFree( dense );
}

} // namespace NeoML
