// Test infrastructure, not part of the product: C entry points that build small networks out of NeoML's OWN layer
// classes (CDnn, CConvLayer, CChannelwiseConvLayer, CFullyConnectedLayer, CMaxPoolingLayer, CMeanPoolingLayer,
// CTransformerEncoderLayer, CLstmLayer; compiled from the reference's sources into _ref/libNeoML.so by the Makefile
// beside this file) on whatever IMathEngine* they are handed, run one forward pass and return the output.
// The tests call them once with the reference's CPU engine and once with the HIP engine: same layer code, same
// CRandom seed for the initialisers, same input, so the two outputs differ only by the engine underneath.
#include <NeoML/NeoML.h>
#include <NeoML/Dnn/Layers/Onnx/OnnxEltwiseLayer.h>
#include "HipLstmLayer.h" // neoml_amd/engine: the LSTM layer that reaches IMathEngine::Lstm on a non-CPU engine

#include <atomic>
#include <chrono>
#include <exception>
#include <string>
#include <string.h>
#include <thread>
#include <vector>

using namespace NeoML;

static thread_local std::string lastError;

#define EXPORT extern "C" __attribute__( ( visibility( "default" ) ) )

EXPORT const char* dnn_last_error() { return lastError.c_str(); }

// dnn_run also times `timedPasses` further forward passes when this is set above zero (wall clock around
// CDnn::RunOnce calls closed by a read-back of the result, i.e. what an application sees); the last timing is kept here
static int timedPasses = 0;
static double lastPassMs = 0;
EXPORT void dnn_set_timed_passes( int passes ) { timedPasses = passes; }
EXPORT double dnn_last_pass_ms() { return lastPassMs; }

// LSTM layers of the networks below: NeoML's own CLstmLayer (0) or this repository's CHipLstmLayer (1); hidden size of
// the two LSTM layers of network kind 4
static int fusedLstm = 0;
static int tailHidden = 32;
EXPORT void dnn_set_fused_lstm( int on ) { fusedLstm = on; }
EXPORT void dnn_set_tail_hidden( int hidden ) { tailHidden = hidden; }
static CLstmLayer* newLstm( IMathEngine& e ) { return fusedLstm != 0 ? new CHipLstmLayer( e ) : new CLstmLayer( e ); }

template<class T>
static CPtr<T> add( CDnn& dnn, T* layer, const char* name, CBaseLayer& input, int outputNumber = 0 )
{
	CPtr<T> holder = layer;
	layer->SetName( name );
	layer->Connect( 0, input, outputNumber );
	dnn.AddLayer( *layer );
	return holder;
}

// kind 0: CNN. Conv 3x3 p1 (16) - ReLU - MaxPool 2x2/2 - ChannelwiseConv 3x3 p1 - ReLU6 - Conv 1x1 (32) - MeanPool 2x2/2
//         - FullyConnected (10) - Softmax. Input dims: [1, N, 1, H, W, 1, C].
static CBaseLayer* buildCnn( CDnn& dnn, IMathEngine& e, CBaseLayer& source )
{
	CPtr<CConvLayer> conv = add( dnn, new CConvLayer( e ), "conv", source );
	conv->SetFilterCount( 16 ); conv->SetFilterHeight( 3 ); conv->SetFilterWidth( 3 );
	conv->SetPaddingHeight( 1 ); conv->SetPaddingWidth( 1 );
	CPtr<CReLULayer> relu = add( dnn, new CReLULayer( e ), "relu", *conv );
	CPtr<CMaxPoolingLayer> pool = add( dnn, new CMaxPoolingLayer( e ), "pool", *relu );
	pool->SetFilterHeight( 2 ); pool->SetFilterWidth( 2 ); pool->SetStrideHeight( 2 ); pool->SetStrideWidth( 2 );
	CPtr<CChannelwiseConvLayer> dw = add( dnn, new CChannelwiseConvLayer( e ), "dw", *pool );
	dw->SetFilterCount( 16 ); dw->SetFilterHeight( 3 ); dw->SetFilterWidth( 3 );
	dw->SetPaddingHeight( 1 ); dw->SetPaddingWidth( 1 );
	CPtr<CReLULayer> relu6 = add( dnn, new CReLULayer( e ), "relu6", *dw );
	relu6->SetUpperThreshold( 6.f );
	CPtr<CConvLayer> project = add( dnn, new CConvLayer( e ), "project", *relu6 );
	project->SetFilterCount( 32 ); project->SetFilterHeight( 1 ); project->SetFilterWidth( 1 );
	CPtr<CMeanPoolingLayer> mean = add( dnn, new CMeanPoolingLayer( e ), "mean", *project );
	mean->SetFilterHeight( 2 ); mean->SetFilterWidth( 2 ); mean->SetStrideHeight( 2 ); mean->SetStrideWidth( 2 );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *mean );
	fc->SetNumberOfElements( 10 );
	CPtr<CSoftmaxLayer> softmax = add( dnn, new CSoftmaxLayer( e ), "softmax", *fc );
	return softmax.Ptr();
}

// kind 1: two CTransformerEncoderLayer (4 heads, FFN 4x, GELU, post-norm, no dropout). Input: [1, B, S, 1, 1, 1, D].
static CBaseLayer* buildTransformer( CDnn& dnn, IMathEngine& e, CBaseLayer& source, int hidden, float dropout = 0.f )
{
	CBaseLayer* last = &source;
	for( int i = 0; i < 2; ++i ) {
		CPtr<CTransformerEncoderLayer> layer = add( dnn, new CTransformerEncoderLayer( e ), i == 0 ? "enc0" : "enc1", *last );
		layer->SetHeadCount( 4 );
		layer->SetHiddenSize( hidden );
		layer->SetDropoutRate( dropout );
		layer->SetSelfAttentionDropoutRate( dropout );
		layer->SetFeedForwardSize( 4 * hidden );
		layer->SetActivation( CActivationDesc( AF_GELU ) );
		last = layer.Ptr();
	}
	return last;
}

// kind 2: CLstmLayer (hidden = param) followed by a FullyConnected over every step. Input: [T, B, 1, 1, 1, 1, In].
static CBaseLayer* buildLstm( CDnn& dnn, IMathEngine& e, CBaseLayer& source, int hidden )
{
	CPtr<CLstmLayer> lstm = add( dnn, newLstm( e ), "lstm", source );
	lstm->SetHiddenSize( hidden );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *lstm );
	fc->SetNumberOfElements( 11 );
	return fc.Ptr();
}

// kind 3: ResNet-style stem and basic block. Conv 7x7/2 p3 (16) - ReLU - ImageResize (pad 1 each side) - MaxPool 3x3/2
//         - [Conv 3x3 p1 /2 (32) - ReLU - Conv 3x3 p1 (32)] + [Conv 1x1 /2 (32)] - EltwiseSum - ReLU - GlobalMeanPooling
//         - FullyConnected (10) - Softmax. Input dims: [1, N, 1, H, W, 1, 3].
static CBaseLayer* buildResNetBlock( CDnn& dnn, IMathEngine& e, CBaseLayer& source )
{
	CPtr<CConvLayer> stem = add( dnn, new CConvLayer( e ), "stem", source );
	stem->SetFilterCount( 16 ); stem->SetFilterHeight( 7 ); stem->SetFilterWidth( 7 );
	stem->SetPaddingHeight( 3 ); stem->SetPaddingWidth( 3 ); stem->SetStrideHeight( 2 ); stem->SetStrideWidth( 2 );
	CPtr<CReLULayer> relu0 = add( dnn, new CReLULayer( e ), "relu0", *stem );
	CPtr<CImageResizeLayer> pad = add( dnn, new CImageResizeLayer( e ), "pad", *relu0 );
	pad->SetDelta( CImageResizeLayer::IS_Left, 1 ); pad->SetDelta( CImageResizeLayer::IS_Right, 1 );
	pad->SetDelta( CImageResizeLayer::IS_Top, 1 ); pad->SetDelta( CImageResizeLayer::IS_Bottom, 1 );
	CPtr<CMaxPoolingLayer> pool = add( dnn, new CMaxPoolingLayer( e ), "pool", *pad );
	pool->SetFilterHeight( 3 ); pool->SetFilterWidth( 3 ); pool->SetStrideHeight( 2 ); pool->SetStrideWidth( 2 );

	CPtr<CConvLayer> c1 = add( dnn, new CConvLayer( e ), "c1", *pool );
	c1->SetFilterCount( 32 ); c1->SetFilterHeight( 3 ); c1->SetFilterWidth( 3 );
	c1->SetPaddingHeight( 1 ); c1->SetPaddingWidth( 1 ); c1->SetStrideHeight( 2 ); c1->SetStrideWidth( 2 );
	CPtr<CReLULayer> relu1 = add( dnn, new CReLULayer( e ), "relu1", *c1 );
	CPtr<CConvLayer> c2 = add( dnn, new CConvLayer( e ), "c2", *relu1 );
	c2->SetFilterCount( 32 ); c2->SetFilterHeight( 3 ); c2->SetFilterWidth( 3 );
	c2->SetPaddingHeight( 1 ); c2->SetPaddingWidth( 1 );
	CPtr<CConvLayer> shortcut = add( dnn, new CConvLayer( e ), "shortcut", *pool );
	shortcut->SetFilterCount( 32 ); shortcut->SetFilterHeight( 1 ); shortcut->SetFilterWidth( 1 );
	shortcut->SetStrideHeight( 2 ); shortcut->SetStrideWidth( 2 );
	CPtr<CEltwiseSumLayer> sum = new CEltwiseSumLayer( e );
	sum->SetName( "sum" );
	sum->Connect( 0, *c2 );
	sum->Connect( 1, *shortcut );
	dnn.AddLayer( *sum );
	CPtr<CReLULayer> relu2 = add( dnn, new CReLULayer( e ), "relu2", *sum );
	CPtr<CGlobalMeanPoolingLayer> gap = add( dnn, new CGlobalMeanPoolingLayer( e ), "gap", *relu2 );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *gap );
	fc->SetNumberOfElements( 10 );
	CPtr<CSoftmaxLayer> softmax = add( dnn, new CSoftmaxLayer( e ), "softmax", *fc );
	return softmax.Ptr();
}

// kind 4: the tail of the line recogniser. Two CLstmLayer over the same input, one reversed, CConcatChannelsLayer,
//         FullyConnected to param classes + blank. dnn_run returns the FC output; dnn_run_ctc also attaches a
//         CCtcDecodingLayer and returns every sequence's best labels. Input: [T, B, 1, 1, 1, 1, In].
static CBaseLayer* buildRecognizerTail( CDnn& dnn, IMathEngine& e, CBaseLayer& source, int classes )
{
	CPtr<CLstmLayer> fwd = add( dnn, newLstm( e ), "fwd", source );
	fwd->SetHiddenSize( tailHidden );
	CPtr<CLstmLayer> rev = add( dnn, newLstm( e ), "rev", source );
	rev->SetHiddenSize( tailHidden );
	rev->SetReverseSequence( true );
	CPtr<CConcatChannelsLayer> concat = new CConcatChannelsLayer( e );
	concat->SetName( "concat" );
	concat->Connect( 0, *fwd );
	concat->Connect( 1, *rev );
	dnn.AddLayer( *concat );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *concat );
	fc->SetNumberOfElements( classes + 1 );
	return fc.Ptr();
}

// kind 5: the whole ResNet-18-style network of the benchmark: 7x7/2 stem (64), pad + 3x3/2 max-pool, 4 stages of 2
//         basic blocks (64/128/256/512, 1x1/2 shortcut where the shape changes), global mean pool, FC (param classes),
//         softmax. Input dims: [1, N, 1, H, W, 1, 3].
static CPtr<CConvLayer> conv( CDnn& dnn, IMathEngine& e, const CString& name, CBaseLayer& input, int filters, int size,
	int padding, int stride )
{
	CPtr<CConvLayer> layer = add( dnn, new CConvLayer( e ), name, input );
	layer->SetFilterCount( filters ); layer->SetFilterHeight( size ); layer->SetFilterWidth( size );
	layer->SetPaddingHeight( padding ); layer->SetPaddingWidth( padding );
	layer->SetStrideHeight( stride ); layer->SetStrideWidth( stride );
	return layer;
}

static CBaseLayer* buildResNet18( CDnn& dnn, IMathEngine& e, CBaseLayer& source, int classes, bool withSoftmax = true )
{
	CPtr<CConvLayer> stem = conv( dnn, e, "stem", source, 64, 7, 3, 2 );
	CPtr<CReLULayer> relu0 = add( dnn, new CReLULayer( e ), "stem_relu", *stem );
	CPtr<CImageResizeLayer> pad = add( dnn, new CImageResizeLayer( e ), "pad", *relu0 );
	pad->SetDelta( CImageResizeLayer::IS_Left, 1 ); pad->SetDelta( CImageResizeLayer::IS_Right, 1 );
	pad->SetDelta( CImageResizeLayer::IS_Top, 1 ); pad->SetDelta( CImageResizeLayer::IS_Bottom, 1 );
	CPtr<CMaxPoolingLayer> pool = add( dnn, new CMaxPoolingLayer( e ), "pool", *pad );
	pool->SetFilterHeight( 3 ); pool->SetFilterWidth( 3 ); pool->SetStrideHeight( 2 ); pool->SetStrideWidth( 2 );
	CBaseLayer* last = pool.Ptr();
	const int widths[4] = { 64, 128, 256, 512 };
	int channels = 64;
	for( int stage = 0; stage < 4; ++stage ) {
		for( int block = 0; block < 2; ++block ) {
			const int stride = ( stage > 0 && block == 0 ) ? 2 : 1;
			const CString prefix = CString( "s" ) + Str( stage ) + "b" + Str( block );
			CPtr<CConvLayer> c1 = conv( dnn, e, prefix + "c1", *last, widths[stage], 3, 1, stride );
			CPtr<CReLULayer> r1 = add( dnn, new CReLULayer( e ), prefix + "r1", *c1 );
			CPtr<CConvLayer> c2 = conv( dnn, e, prefix + "c2", *r1, widths[stage], 3, 1, 1 );
			CBaseLayer* shortcut = last;
			if( stride != 1 || channels != widths[stage] ) {
				shortcut = conv( dnn, e, prefix + "sc", *last, widths[stage], 1, 0, stride ).Ptr();
			}
			CPtr<CEltwiseSumLayer> sum = new CEltwiseSumLayer( e );
			sum->SetName( prefix + "sum" );
			sum->Connect( 0, *c2 );
			sum->Connect( 1, *shortcut );
			dnn.AddLayer( *sum );
			CPtr<CReLULayer> r2 = add( dnn, new CReLULayer( e ), prefix + "r2", *sum );
			last = r2.Ptr();
			channels = widths[stage];
		}
	}
	CPtr<CGlobalMeanPoolingLayer> gap = add( dnn, new CGlobalMeanPoolingLayer( e ), "gap", *last );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *gap );
	fc->SetNumberOfElements( classes );
	if( !withSoftmax ) {
		return fc.Ptr(); // the loss layer applies its own softmax
	}
	CPtr<CSoftmaxLayer> softmax = add( dnn, new CSoftmaxLayer( e ), "softmax", *fc );
	return softmax.Ptr();
}

// kind 6: a small depthwise-separable network of plain layers, the patterns NeoML's graph optimizer rewrites:
//         stem 3x3/2 (16) - ReLU6 - inverted residual block (1x1 to 96 - ReLU6 - channelwise 3x3 - ReLU6 - 1x1 to 16, + input)
//         - inverted block with stride 2 (to 24 channels, no residual) - channelwise 3x3 - h-swish - 1x1 (32)
//         - global mean pool - FullyConnected (param) - softmax. Input dims: [1, N, 1, H, W, 1, 3].
static CBaseLayer* relu6( CDnn& dnn, IMathEngine& e, const CString& name, CBaseLayer& input )
{
	CPtr<CReLULayer> layer = add( dnn, new CReLULayer( e ), name, input );
	layer->SetUpperThreshold( 6.f );
	return layer.Ptr();
}

static CBaseLayer* channelwise3x3( CDnn& dnn, IMathEngine& e, const CString& name, CBaseLayer& input, int channels, int stride )
{
	CPtr<CChannelwiseConvLayer> layer = add( dnn, new CChannelwiseConvLayer( e ), name, input );
	layer->SetFilterCount( channels ); layer->SetFilterHeight( 3 ); layer->SetFilterWidth( 3 );
	layer->SetPaddingHeight( 1 ); layer->SetPaddingWidth( 1 );
	layer->SetStrideHeight( stride ); layer->SetStrideWidth( stride );
	return layer.Ptr();
}

static CBaseLayer* invertedBlock( CDnn& dnn, IMathEngine& e, const CString& name, CBaseLayer& input, int expanded,
	int outputChannels, int stride, bool residual )
{
	CBaseLayer* x = conv( dnn, e, name + "_expand", input, expanded, 1, 0, 1 ).Ptr();
	x = relu6( dnn, e, name + "_relu1", *x );
	x = channelwise3x3( dnn, e, name + "_dw", *x, expanded, stride );
	x = relu6( dnn, e, name + "_relu2", *x );
	x = conv( dnn, e, name + "_down", *x, outputChannels, 1, 0, 1 ).Ptr();
	if( residual ) {
		CPtr<CEltwiseSumLayer> sum = new CEltwiseSumLayer( e );
		sum->SetName( name + "_sum" );
		sum->Connect( 0, input );
		sum->Connect( 1, *x );
		dnn.AddLayer( *sum );
		x = sum.Ptr();
	}
	return x;
}

static CBaseLayer* buildSeparableNet( CDnn& dnn, IMathEngine& e, CBaseLayer& source, int classes, bool withSoftmax = true )
{
	CBaseLayer* x = conv( dnn, e, "stem", source, 16, 3, 1, 2 ).Ptr();
	x = relu6( dnn, e, "stem_relu", *x );
	x = invertedBlock( dnn, e, "b1", *x, 96, 16, 1, true );
	x = invertedBlock( dnn, e, "b2", *x, 96, 24, 2, false );
	x = channelwise3x3( dnn, e, "tail_dw", *x, 24, 1 );
	CPtr<CHSwishLayer> hswish = add( dnn, new CHSwishLayer( e ), "tail_hswish", *x );
	x = conv( dnn, e, "tail_conv", *hswish, 32, 1, 0, 1 ).Ptr();
	CPtr<CGlobalMeanPoolingLayer> gap = add( dnn, new CGlobalMeanPoolingLayer( e ), "gap", *x );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *gap );
	fc->SetNumberOfElements( classes );
	if( !withSoftmax ) {
		return fc.Ptr(); // the loss layer applies its own softmax
	}
	CPtr<CSoftmaxLayer> softmax = add( dnn, new CSoftmaxLayer( e ), "softmax", *fc );
	return softmax.Ptr();
}

// kind 7: a MobileNetV3-style network of plain layers: stem 3x3/2 (16) - h-swish - two blocks of
//         [1x1 expand - act - channelwise FxF - act - squeeze-and-excite (global mean - FC / 4 - ReLU - FC - hard sigmoid,
//         multiplied back through COnnxEltwiseLayer) - act - 1x1 down ( + input )]: (F 3, 64 wide, ReLU, residual) and
//         (F 5, 96 wide, h-swish, stride 2, to 24 channels) - global mean pool - FullyConnected (param) - softmax.
static CBaseLayer* blockActivation( CDnn& dnn, IMathEngine& e, const CString& name, CBaseLayer& input, bool hswish )
{
	if( hswish ) {
		return add( dnn, new CHSwishLayer( e ), name, input ).Ptr();
	}
	return add( dnn, new CReLULayer( e ), name, input ).Ptr();
}

static CBaseLayer* squeezeExciteBlock( CDnn& dnn, IMathEngine& e, const CString& name, CBaseLayer& input, int filterSize,
	int expanded, int outputChannels, int stride, bool hswish, bool residual )
{
	CBaseLayer* x = conv( dnn, e, name + "_expand", input, expanded, 1, 0, 1 ).Ptr();
	x = blockActivation( dnn, e, name + "_act1", *x, hswish );
	CPtr<CChannelwiseConvLayer> dw = add( dnn, new CChannelwiseConvLayer( e ), name + "_dw", *x );
	dw->SetFilterCount( expanded ); dw->SetFilterHeight( filterSize ); dw->SetFilterWidth( filterSize );
	dw->SetPaddingHeight( filterSize / 2 ); dw->SetPaddingWidth( filterSize / 2 );
	dw->SetStrideHeight( stride ); dw->SetStrideWidth( stride );
	x = blockActivation( dnn, e, name + "_act2", *dw, hswish );
	CPtr<CGlobalMeanPoolingLayer> pool = add( dnn, new CGlobalMeanPoolingLayer( e ), name + "_se_pool", *x );
	CPtr<CFullyConnectedLayer> fc1 = add( dnn, new CFullyConnectedLayer( e ), name + "_se_fc1", *pool );
	fc1->SetNumberOfElements( expanded / 4 );
	CPtr<CReLULayer> seRelu = add( dnn, new CReLULayer( e ), name + "_se_relu", *fc1 );
	CPtr<CFullyConnectedLayer> fc2 = add( dnn, new CFullyConnectedLayer( e ), name + "_se_fc2", *seRelu );
	fc2->SetNumberOfElements( expanded );
	CPtr<CHardSigmoidLayer> gate = add( dnn, new CHardSigmoidLayer( e ), name + "_se_gate", *fc2 );
	CPtr<COnnxEltwiseLayer> mul = new COnnxEltwiseLayer( e );
	mul->SetName( name + "_se_mul" );
	mul->SetOperation( COnnxEltwiseLayer::TOperation::Mul );
	mul->Connect( 0, *x );
	mul->Connect( 1, *gate );
	dnn.AddLayer( *mul );
	x = blockActivation( dnn, e, name + "_act3", *mul, hswish );
	x = conv( dnn, e, name + "_down", *x, outputChannels, 1, 0, 1 ).Ptr();
	if( residual ) {
		CPtr<CEltwiseSumLayer> sum = new CEltwiseSumLayer( e );
		sum->SetName( name + "_sum" );
		sum->Connect( 0, input );
		sum->Connect( 1, *x );
		dnn.AddLayer( *sum );
		x = sum.Ptr();
	}
	return x;
}

static CBaseLayer* buildSqueezeExciteNet( CDnn& dnn, IMathEngine& e, CBaseLayer& source, int classes )
{
	CBaseLayer* x = conv( dnn, e, "stem", source, 16, 3, 1, 2 ).Ptr();
	x = add( dnn, new CHSwishLayer( e ), "stem_hswish", *x ).Ptr();
	x = squeezeExciteBlock( dnn, e, "b1", *x, 3, 64, 16, 1, false, true );
	x = squeezeExciteBlock( dnn, e, "b2", *x, 5, 96, 24, 2, true, false );
	CPtr<CGlobalMeanPoolingLayer> gap = add( dnn, new CGlobalMeanPoolingLayer( e ), "gap", *x );
	CPtr<CFullyConnectedLayer> fc = add( dnn, new CFullyConnectedLayer( e ), "fc", *gap );
	fc->SetNumberOfElements( classes );
	CPtr<CSoftmaxLayer> softmax = add( dnn, new CSoftmaxLayer( e ), "softmax", *fc );
	return softmax.Ptr();
}

// When set, dnn_run hands the network to NeoML's own graph optimizer (OptimizeDnn) after its first pass (the pass
// that allocates and initialises the weights) and keeps what the optimizer reports
static int optimizeNetworks = 0;
static CDnnOptimizationReport lastReport;
EXPORT void dnn_set_optimize( int on ) { optimizeNetworks = on; }
EXPORT void dnn_last_optimization( int* mobileNetV2Blocks, int* channelwiseWith1x1, int* rowwiseChains )
{
	*mobileNetV2Blocks = lastReport.MobileNetV2NonResidualBlocks + lastReport.MobileNetV2ResidualBlocks;
	*channelwiseWith1x1 = lastReport.ChannelwiseWith1x1NonResidual + lastReport.ChannelwiseWith1x1Residual;
	*rowwiseChains = lastReport.RowwiseChainCount;
}
EXPORT int dnn_last_optimization_mobilenetv3_blocks()
{
	return lastReport.MobileNetV3NonResidualBlocks + lastReport.MobileNetV3ResidualBlocks;
}

// Runs network `kind` on `engine`. dims: the 7 blob dimensions of the input; param: kind-specific size.
// output receives at most outputCapacity floats; outputDims the 7 dimensions of the result.
EXPORT int dnn_run( void* engine, int kind, int seed, int param, const int* dims, const float* input,
	float* output, int outputCapacity, int* outputDims )
{
	try {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CRandom random( seed );
		CDnn dnn( random, e );
		CPtr<CSourceLayer> source = new CSourceLayer( e );
		source->SetName( "source" );
		dnn.AddLayer( *source );

		CBaseLayer* last = nullptr;
		switch( kind ) {
			case 0: last = buildCnn( dnn, e, *source ); break;
			case 1: last = buildTransformer( dnn, e, *source, param ); break;
			case 2: last = buildLstm( dnn, e, *source, param ); break;
			case 3: last = buildResNetBlock( dnn, e, *source ); break;
			case 4: last = buildRecognizerTail( dnn, e, *source, param ); break;
			case 5: last = buildResNet18( dnn, e, *source, param ); break;
			case 6: last = buildSeparableNet( dnn, e, *source, param ); break;
			case 7: last = buildSqueezeExciteNet( dnn, e, *source, param ); break;
			default: lastError = "unknown network kind"; return 1;
		}
		CPtr<CSinkLayer> sink = new CSinkLayer( e );
		sink->SetName( "sink" );
		sink->Connect( *last );
		dnn.AddLayer( *sink );

		CBlobDesc desc( CT_Float );
		for( int d = 0; d < 7; ++d ) {
			desc.SetDimSize( d, dims[d] );
		}
		CPtr<CDnnBlob> blob = CDnnBlob::CreateBlob( e, CT_Float, desc );
		blob->CopyFrom( input );
		source->SetBlob( blob );

		dnn.RunOnce();
		if( optimizeNetworks != 0 ) {
			lastReport = OptimizeDnn( dnn );
		}
		// a second pass over the same network: buffers are reused, results must not change
		dnn.RunOnce();

		if( timedPasses > 0 ) {
			float probe = 0;
			sink->GetBlob()->GetData().GetValue(); // drains the engine's queue before the clock starts
			const auto start = std::chrono::steady_clock::now();
			for( int i = 0; i < timedPasses; ++i ) {
				dnn.RunOnce();
			}
			probe = sink->GetBlob()->GetData().GetValue();
			( void )probe;
			lastPassMs = std::chrono::duration<double, std::milli>( std::chrono::steady_clock::now() - start ).count() / timedPasses;
		}

		const CPtr<CDnnBlob>& result = sink->GetBlob();
		for( int d = 0; d < 7; ++d ) {
			outputDims[d] = result->DimSize( d );
		}
		if( result->GetDataSize() > outputCapacity ) {
			lastError = "output buffer too small";
			return 2;
		}
		result->CopyTo( output );
		return 0;
	} catch( std::exception& ex ) {
		lastError = ex.what();
	} catch( CException* ex ) {
		lastError = "NeoML exception";
		delete ex;
	} catch( ... ) {
		lastError = "unknown exception";
	}
	return 3;
}

// The engine interface from several threads at once ( the reference: "the math engine interface is thread-safe; the same
// instance may be used in different networks and different threads", README.md:116-118; its own idiom is one engine and
// one CDnn per thread, NeoML/test/src/InferencePerformanceMultiThreadingTest.cpp:236-262 ).
// Thread t builds network kinds[t] ( dnn_run's kinds, params[t] ) on engines[t] - all the same engine, or one each -
// and runs `passes` forward passes over its own input, all threads released together; between the passes it asks the
// engine for its peak memory and calls CleanUp(), so that those run while the other threads' launches are in flight.
// outputs[t] receives the result of thread t's last pass. dims: 7 per thread; outputDims: 7 per thread.
// Returns 0, or 1 + the index of the first thread that failed ( dnn_last_error() then holds its message ).
EXPORT int dnn_run_threads( int threads, void* const* engines, const int* kinds, const int* params, int seed, const int* dims,
	const float* const* inputs, float* const* outputs, const int* capacities, int* outputDims, int passes )
{
	std::vector<std::string> errors( threads );
	std::vector<int> codes( threads, 0 );
	std::atomic<int> ready( 0 );
	std::atomic<bool> go( false );
	auto body = [&]( int t ) {
		bool counted = false; // in `ready`: a thread that fails while building must not leave the others waiting for ever
		try {
			IMathEngine& e = *static_cast<IMathEngine*>( engines[t] );
			CRandom random( seed );
			CDnn dnn( random, e );
			CPtr<CSourceLayer> source = new CSourceLayer( e );
			source->SetName( "source" );
			dnn.AddLayer( *source );
			CBaseLayer* last = nullptr;
			switch( kinds[t] ) {
				case 0: last = buildCnn( dnn, e, *source ); break;
				case 1: last = buildTransformer( dnn, e, *source, params[t] ); break;
				case 2: last = buildLstm( dnn, e, *source, params[t] ); break;
				case 3: last = buildResNetBlock( dnn, e, *source ); break;
				case 4: last = buildRecognizerTail( dnn, e, *source, params[t] ); break;
				case 5: last = buildResNet18( dnn, e, *source, params[t] ); break;
				case 6: last = buildSeparableNet( dnn, e, *source, params[t] ); break;
				default: errors[t] = "unknown network kind"; codes[t] = 1; break;
			}
			CPtr<CSinkLayer> sink;
			if( codes[t] == 0 ) {
				sink = new CSinkLayer( e );
				sink->SetName( "sink" );
				sink->Connect( *last );
				dnn.AddLayer( *sink );
				CBlobDesc desc( CT_Float );
				for( int d = 0; d < 7; ++d ) {
					desc.SetDimSize( d, dims[7 * t + d] );
				}
				CPtr<CDnnBlob> blob = CDnnBlob::CreateBlob( e, CT_Float, desc );
				blob->CopyFrom( inputs[t] );
				source->SetBlob( blob );
			}
			// every thread has built its network: from here on they all run at once
			counted = true;
			ready.fetch_add( 1 );
			while( !go.load() ) {
				std::this_thread::yield();
			}
			if( codes[t] != 0 ) {
				return;
			}
			size_t peak = 0;
			for( int pass = 0; pass < passes; ++pass ) {
				dnn.RunOnce();
				peak = e.GetPeakMemoryUsage() > peak ? e.GetPeakMemoryUsage() : peak;
				e.CleanUp();
			}
			const CPtr<CDnnBlob>& result = sink->GetBlob();
			for( int d = 0; d < 7; ++d ) {
				outputDims[7 * t + d] = result->DimSize( d );
			}
			if( peak == 0 ) {
				errors[t] = "GetPeakMemoryUsage returned zero while a network was running";
				codes[t] = 4;
			} else if( result->GetDataSize() > capacities[t] ) {
				errors[t] = "output buffer too small";
				codes[t] = 2;
			} else {
				result->CopyTo( outputs[t] );
			}
		} catch( std::exception& ex ) {
			errors[t] = ex.what();
			codes[t] = 3;
		} catch( CException* ex ) {
			errors[t] = "NeoML exception";
			codes[t] = 3;
			delete ex;
		} catch( ... ) {
			errors[t] = "unknown exception";
			codes[t] = 3;
		}
		if( !counted ) {
			ready.fetch_add( 1 );
		}
	};
	std::vector<std::thread> pool;
	for( int t = 0; t < threads; ++t ) {
		pool.emplace_back( body, t );
	}
	while( ready.load() < threads ) {
		std::this_thread::yield();
	}
	go.store( true );
	for( std::thread& th : pool ) {
		th.join();
	}
	for( int t = 0; t < threads; ++t ) {
		if( codes[t] != 0 ) {
			lastError = "thread " + std::to_string( t ) + ": " + errors[t];
			return 1 + t;
		}
	}
	return 0;
}

// Training: a small classifier, CCrossEntropyLossLayer on float labels, CDnnSimpleGradientSolver (momentum 0.9),
// `steps` calls of CDnn::RunAndLearnOnce on the same batch. kind 0: FullyConnected (32) - ReLU - FullyConnected
// (classes); kind 1: Conv 3x3 p1 (8) - ReLU - MaxPool 2x2/2 - Conv 3x3 p1 stride 2 (16) - ReLU - FullyConnected (classes).
// kind 2: Conv 3x3 p1 (16) - HSwish - [Conv 3x3 p1 (16) - ReLU - Conv 3x3 p1 (16)] + shortcut - ReLU - MeanPool 2x2/2 -
// FullyConnected (classes); kind 3: Lstm (24 units, over BatchLength) - FullyConnected (classes) at every step.
// kind 4: the ResNet-18-style network of dnn_run's kind 5; kind 5: the depthwise-separable network of its kind 6;
// kind 6: the transformer encoder of its kind 1 with a classifier over every position (input [1, B, seq, 1, 1, 1, hidden]);
// kind 7: the same with dropout; kind 8: a small CNN with CBatchNormalizationLayer behind each convolution.
// solver 0: CDnnSimpleGradientSolver, 1: CDnnAdaptiveGradientSolver (Adam), both with L2 regularisation 1e-3.
// losses receives the loss of every step, output the logits of a final forward pass with the trained weights.
// timedSteps > 0: that many further steps are timed (the loss is read after the last one, which waits for the device)
// and *msPerStep receives the mean.
EXPORT int dnn_train( void* engine, int kind, int solverKind, int seed, int classes, int steps, float learningRate,
	const int* dims, const float* input, const float* labels, float* losses, float* output, int outputCapacity,
	int timedSteps, float* msPerStep )
{
	try {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CRandom random( seed );
		CDnn dnn( random, e );
		CPtr<CSourceLayer> source = new CSourceLayer( e );
		source->SetName( "source" );
		dnn.AddLayer( *source );
		CPtr<CSourceLayer> labelSource = new CSourceLayer( e );
		labelSource->SetName( "labels" );
		dnn.AddLayer( *labelSource );

		CBaseLayer* last = source.Ptr();
		CBaseLayer* logits = nullptr;
		if( kind == 8 ) {
			// Conv 3x3 (8) - BatchNormalization (per channel) - ReLU - Conv 3x3 /2 (16) - BatchNormalization - ReLU - GlobalMeanPooling
			CPtr<CConvLayer> c1 = conv( dnn, e, "conv1", *last, 8, 3, 1, 1 );
			// (the normalization mode can only be set before the layer joins the network)
			CBatchNormalizationLayer* newBn1 = new CBatchNormalizationLayer( e );
			newBn1->SetChannelBased( true );
			CPtr<CBatchNormalizationLayer> bn1 = add( dnn, newBn1, "bn1", *c1 );
			CPtr<CReLULayer> r1 = add( dnn, new CReLULayer( e ), "relu1", *bn1 );
			CPtr<CConvLayer> c2 = conv( dnn, e, "conv2", *r1, 16, 3, 1, 2 );
			CBatchNormalizationLayer* newBn2 = new CBatchNormalizationLayer( e );
			newBn2->SetChannelBased( true );
			CPtr<CBatchNormalizationLayer> bn2 = add( dnn, newBn2, "bn2", *c2 );
			CPtr<CReLULayer> r2 = add( dnn, new CReLULayer( e ), "relu2", *bn2 );
			CPtr<CGlobalMeanPoolingLayer> gap = add( dnn, new CGlobalMeanPoolingLayer( e ), "gap", *r2 );
			last = gap.Ptr();
		} else if( kind == 6 || kind == 7 ) {
			// two CTransformerEncoderLayers (hidden = the input's channel count), a classifier over every position;
			// kind 7: with dropout 0.1 inside the layers (the masks come from the network's CRandom seeds)
			last = buildTransformer( dnn, e, *source, dims[6], kind == 7 ? 0.1f : 0.f );
		} else if( kind == 4 ) {
			logits = buildResNet18( dnn, e, *source, classes, false );
		} else if( kind == 5 ) {
			logits = buildSeparableNet( dnn, e, *source, classes, false );
		} else if( kind == 0 ) {
			CPtr<CFullyConnectedLayer> fc1 = add( dnn, new CFullyConnectedLayer( e ), "fc1", *last );
			fc1->SetNumberOfElements( 32 );
			CPtr<CReLULayer> relu = add( dnn, new CReLULayer( e ), "relu", *fc1 );
			last = relu.Ptr();
		} else if( kind == 2 ) {
			CPtr<CConvLayer> c0 = conv( dnn, e, "conv0", *last, 16, 3, 1, 1 );
			CPtr<CHSwishLayer> a0 = add( dnn, new CHSwishLayer( e ), "hswish0", *c0 );
			CPtr<CConvLayer> c1 = conv( dnn, e, "conv1", *a0, 16, 3, 1, 1 );
			CPtr<CReLULayer> r1 = add( dnn, new CReLULayer( e ), "relu1", *c1 );
			CPtr<CConvLayer> c2 = conv( dnn, e, "conv2", *r1, 16, 3, 1, 1 );
			CPtr<CEltwiseSumLayer> sum = add( dnn, new CEltwiseSumLayer( e ), "sum", *c2 );
			sum->Connect( 1, *a0 );
			CPtr<CReLULayer> r2 = add( dnn, new CReLULayer( e ), "relu2", *sum );
			CPtr<CMeanPoolingLayer> pool = add( dnn, new CMeanPoolingLayer( e ), "pool", *r2 );
			pool->SetFilterHeight( 2 ); pool->SetFilterWidth( 2 ); pool->SetStrideHeight( 2 ); pool->SetStrideWidth( 2 );
			last = pool.Ptr();
		} else if( kind == 3 ) {
			CPtr<CLstmLayer> lstm = add( dnn, new CLstmLayer( e ), "lstm", *last );
			lstm->SetHiddenSize( 24 );
			last = lstm.Ptr();
		} else {
			CPtr<CConvLayer> c1 = conv( dnn, e, "conv1", *last, 8, 3, 1, 1 );
			CPtr<CReLULayer> r1 = add( dnn, new CReLULayer( e ), "relu1", *c1 );
			CPtr<CMaxPoolingLayer> pool = add( dnn, new CMaxPoolingLayer( e ), "pool", *r1 );
			pool->SetFilterHeight( 2 ); pool->SetFilterWidth( 2 ); pool->SetStrideHeight( 2 ); pool->SetStrideWidth( 2 );
			CPtr<CConvLayer> c2 = conv( dnn, e, "conv2", *pool, 16, 3, 1, 2 );
			CPtr<CReLULayer> r2 = add( dnn, new CReLULayer( e ), "relu2", *c2 );
			last = r2.Ptr();
		}
		if( logits == nullptr ) {
			CPtr<CFullyConnectedLayer> fcLast = add( dnn, new CFullyConnectedLayer( e ), "fc", *last );
			fcLast->SetNumberOfElements( classes );
			logits = fcLast.Ptr();
		}
		CBaseLayer* fc = logits;
		CPtr<CCrossEntropyLossLayer> loss = new CCrossEntropyLossLayer( e );
		loss->SetName( "loss" );
		loss->Connect( 0, *fc );
		loss->Connect( 1, *labelSource );
		dnn.AddLayer( *loss );
		CPtr<CSinkLayer> sink = new CSinkLayer( e );
		sink->SetName( "sink" );
		sink->Connect( *fc );
		dnn.AddLayer( *sink );

		if( solverKind == 0 ) {
			CPtr<CDnnSimpleGradientSolver> solver = new CDnnSimpleGradientSolver( e );
			solver->SetMomentDecayRate( 0.9f );
			solver->SetLearningRate( learningRate );
			solver->SetL2Regularization( 1e-3f );
			dnn.SetSolver( solver );
		} else {
			CPtr<CDnnAdaptiveGradientSolver> solver = new CDnnAdaptiveGradientSolver( e );
			solver->SetLearningRate( learningRate );
			solver->SetL2Regularization( 1e-3f );
			dnn.SetSolver( solver );
		}

		CBlobDesc desc( CT_Float );
		for( int d = 0; d < 7; ++d ) {
			desc.SetDimSize( d, dims[d] );
		}
		CPtr<CDnnBlob> blob = CDnnBlob::CreateBlob( e, CT_Float, desc );
		blob->CopyFrom( input );
		source->SetBlob( blob );
		CBlobDesc labelDesc( CT_Float );
		labelDesc.SetDimSize( BD_BatchLength, dims[0] );
		labelDesc.SetDimSize( BD_BatchWidth, dims[1] );
		labelDesc.SetDimSize( BD_ListSize, dims[2] );
		labelDesc.SetDimSize( BD_Channels, classes );
		CPtr<CDnnBlob> labelBlob = CDnnBlob::CreateBlob( e, CT_Float, labelDesc );
		labelBlob->CopyFrom( labels );
		labelSource->SetBlob( labelBlob );

		for( int i = 0; i < steps; ++i ) {
			dnn.RunAndLearnOnce();
			losses[i] = loss->GetLastLoss();
		}
		if( timedSteps > 0 ) {
			const auto start = std::chrono::steady_clock::now();
			for( int i = 0; i < timedSteps; ++i ) {
				dnn.RunAndLearnOnce();
			}
			( void )loss->GetLastLoss();
			*msPerStep = std::chrono::duration<float, std::milli>( std::chrono::steady_clock::now() - start ).count() / timedSteps;
		}
		dnn.RunOnce();
		const CPtr<CDnnBlob>& result = sink->GetBlob();
		if( result->GetDataSize() > outputCapacity ) {
			lastError = "output buffer too small";
			return 2;
		}
		result->CopyTo( output );
		return 0;
	} catch( std::exception& ex ) {
		lastError = ex.what();
	} catch( CException* ex ) {
		lastError = "NeoML exception";
		delete ex;
	} catch( ... ) {
		lastError = "unknown exception";
	}
	return 3;
}

// The recogniser tail (kind 4) with NeoML's CCtcDecodingLayer on top: labels receives, sequence after sequence,
// the best label sequence of each of the B inputs (at most T each); lengths[b] its length.
EXPORT int dnn_run_ctc( void* engine, int seed, int classes, const int* dims, const float* input, int* labels, int* lengths )
{
	try {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CRandom random( seed );
		CDnn dnn( random, e );
		CPtr<CSourceLayer> source = new CSourceLayer( e );
		source->SetName( "source" );
		dnn.AddLayer( *source );
		CBaseLayer* fc = buildRecognizerTail( dnn, e, *source, classes );
		CPtr<CCtcDecodingLayer> ctc = new CCtcDecodingLayer( e );
		ctc->SetName( "ctc" );
		ctc->SetBlankLabel( classes );
		ctc->Connect( *fc );
		dnn.AddLayer( *ctc );

		CBlobDesc desc( CT_Float );
		for( int d = 0; d < 7; ++d ) {
			desc.SetDimSize( d, dims[d] );
		}
		CPtr<CDnnBlob> blob = CDnnBlob::CreateBlob( e, CT_Float, desc );
		blob->CopyFrom( input );
		source->SetBlob( blob );
		dnn.RunOnce();

		const int T = dims[0], B = dims[1];
		for( int b = 0; b < B; ++b ) {
			CArray<int> best;
			ctc->GetBestSequence( b, best );
			lengths[b] = best.Size();
			for( int i = 0; i < best.Size() && i < T; ++i ) {
				labels[b * T + i] = best[i];
			}
		}
		return 0;
	} catch( std::exception& ex ) {
		lastError = ex.what();
	} catch( CException* ex ) {
		lastError = "NeoML exception";
		delete ex;
	} catch( ... ) {
		lastError = "unknown exception";
	}
	return 3;
}
