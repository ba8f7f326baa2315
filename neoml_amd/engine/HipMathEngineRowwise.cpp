// CHipMathEngine: the fused blocks and rowwise operation chains the graph optimizer emits
// (NeoMathEngine.h:1066-1110; layer classes CMobileNetV2BlockLayer, CChannelwiseWith1x1Layer,
// CRowwiseOperationChainLayer).
//
// On the CPU engine a chain is executed a few image rows at a time so that intermediate rows stay in cache
// (src/CPU/CpuMathEngineDnnRowwise.cpp). On the device the counterpart of that idea is fewer, fatter launches:
// every operation of a chain is one launch over the whole blob (activations run in place on the output of the
// operation before them), and the two MobileNet blocks are three launches each with the activations and the
// residual sum in the epilogues of the producing kernels.
#include "HipMathEngine.h"

#include <algorithm>
#include <memory>
#include <vector>

namespace NeoML {

#define NH_CALL( expr ) check( ( expr ), #expr, __LINE__ )

static int fusedActivation( TActivationFunction type )
{
	// what the blocks support (src/CPU/Rowwise/CpuRowwiseCommon.h:79-86): ReLU, h-swish; anything else stores as is
	return type == AF_ReLU ? NH_ACT_RELU : ( type == AF_HSwish ? NH_ACT_HSWISH : NH_ACT_NONE );
}

// Base of every rowwise operation of this engine
struct IHipRowwiseOperation : public CRowwiseOperationDesc {
	// remembers the input size, returns the output size
	virtual CBlobDesc Reshape( const CBlobDesc& input ) = 0;
	virtual int OutputSize() const = 0;
	// true: the operation may run with output == input
	virtual bool IsInPlace() const { return false; }
	virtual void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) = 0;
};

// ---- activation -----------------------------------------------------------------------------------------------

struct CHipRowwiseActivation : public IHipRowwiseOperation {
	CActivationDesc Desc;
	int Size = 0;
	// the scalars that the vector operations of the interface take as engine memory
	std::unique_ptr<CFloatHandleVar> Scalars;

	explicit CHipRowwiseActivation( const CActivationDesc& desc ) : Desc( desc ) {}
	CBlobDesc Reshape( const CBlobDesc& input ) override { Size = input.BlobSize(); return input; }
	int OutputSize() const override { return Size; }
	bool IsInPlace() const override { return true; }

	void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) override
	{
		float values[2] = { 0.f, 0.f };
		switch( Desc.GetType() ) {
			case AF_ELU: values[0] = Desc.GetParam<CELUActivationParam>().Alpha; break;
			case AF_HardSigmoid:
				values[0] = Desc.GetParam<CHardSigmoidActivationParam>().Slope;
				values[1] = Desc.GetParam<CHardSigmoidActivationParam>().Bias;
				break;
			case AF_LeakyReLU: values[0] = Desc.GetParam<CLeakyReLUActivationParam>().Alpha; break;
			case AF_Linear:
				values[0] = Desc.GetParam<CLinearActivationParam>().Multiplier;
				values[1] = Desc.GetParam<CLinearActivationParam>().FreeTerm;
				break;
			case AF_ReLU: values[0] = Desc.GetParam<CReLUActivationParam>().UpperThreshold; break;
			default: break;
		}
		if( Scalars == nullptr ) {
			Scalars.reset( new CFloatHandleVar( engine, 2 ) );
			engine.DataExchangeRaw( Scalars->GetHandle(), values, sizeof( values ) );
		}
		const CConstFloatHandle first = Scalars->GetHandle();
		const CConstFloatHandle second = Scalars->GetHandle() + 1;
		switch( Desc.GetType() ) {
			case AF_ELU: engine.VectorELU( input, output, Size, first ); break;
			case AF_HardSigmoid: engine.VectorHardSigmoid( input, output, Size, first, second ); break;
			case AF_HardTanh: engine.VectorHardTanh( input, output, Size ); break;
			case AF_HSwish: engine.VectorHSwish( input, output, Size ); break;
			case AF_LeakyReLU: engine.VectorLeakyReLU( input, output, Size, first ); break;
			case AF_Linear: {
				CConstFloatHandle current = input;
				if( values[0] != 1.f ) {
					engine.VectorMultiply( current, output, Size, first );
					current = output;
				}
				if( values[1] != 0.f ) {
					engine.VectorAddValue( current, output, Size, second );
					current = output;
				}
				if( current != output ) {
					engine.VectorCopy( output, current, Size );
				}
				break;
			}
			case AF_ReLU: engine.VectorReLU( input, output, Size, first ); break;
			case AF_Sigmoid: engine.VectorSigmoid( input, output, Size ); break;
			case AF_Tanh: engine.VectorTanh( input, output, Size ); break;
			default: ASSERT_EXPR( !"rowwise activation: unsupported type" );
		}
	}
};

// ---- convolutions, pooling, resize: the engine's own blob operations over the whole blob ----------------------

struct CHipRowwiseConv : public IHipRowwiseOperation {
	int PaddingHeight, PaddingWidth, StrideHeight, StrideWidth, DilationHeight, DilationWidth;
	CBlobDesc FilterDesc;
	CConstFloatHandle Filter, FreeTerm;
	CBlobDesc Input, Output;
	std::unique_ptr<CConvolutionDesc> Desc;

	CBlobDesc Reshape( const CBlobDesc& input ) override
	{
		Input = input;
		Output = input;
		const int spanH = ( FilterDesc.Height() - 1 ) * DilationHeight + 1;
		const int spanW = ( FilterDesc.Width() - 1 ) * DilationWidth + 1;
		Output.SetDimSize( BD_Height, ( input.Height() + 2 * PaddingHeight - spanH ) / StrideHeight + 1 );
		Output.SetDimSize( BD_Width, ( input.Width() + 2 * PaddingWidth - spanW ) / StrideWidth + 1 );
		Output.SetDimSize( BD_Depth, 1 );
		Output.SetDimSize( BD_Channels, FilterDesc.ObjectCount() );
		Desc.reset();
		return Output;
	}
	int OutputSize() const override { return Output.BlobSize(); }
	void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) override
	{
		ProcessWithActivation( engine, input, output, NH_ACT_NONE, 0.f );
	}
	// the convolution and the ReLU / h-swish that follows it in the chain as one launch
	void ProcessWithActivation( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output,
		int activation, float param )
	{
		if( Desc == nullptr ) {
			Desc.reset( engine.InitBlobConvolution( Input, PaddingHeight, PaddingWidth, StrideHeight, StrideWidth,
				DilationHeight, DilationWidth, FilterDesc, Output ) );
		}
		engine.BlobConvolutionWithActivation( *Desc, input, Filter, FreeTerm.IsNull() ? nullptr : &FreeTerm, activation,
			param, output );
	}
};

struct CHipRowwiseChConv : public IHipRowwiseOperation {
	int PaddingHeight, PaddingWidth, StrideHeight, StrideWidth;
	CBlobDesc FilterDesc;
	CConstFloatHandle Filter, FreeTerm;
	CBlobDesc Input, Output;
	std::unique_ptr<CChannelwiseConvolutionDesc> Desc;

	CBlobDesc Reshape( const CBlobDesc& input ) override
	{
		Input = input;
		Output = input;
		Output.SetDimSize( BD_Height, ( input.Height() + 2 * PaddingHeight - FilterDesc.Height() ) / StrideHeight + 1 );
		Output.SetDimSize( BD_Width, ( input.Width() + 2 * PaddingWidth - FilterDesc.Width() ) / StrideWidth + 1 );
		Desc.reset();
		return Output;
	}
	int OutputSize() const override { return Output.BlobSize(); }
	void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) override
	{
		if( Desc == nullptr ) {
			CBlobDesc freeTermDesc( CT_Float );
			freeTermDesc.SetDimSize( BD_Channels, Input.Channels() );
			Desc.reset( engine.InitBlobChannelwiseConvolution( Input, PaddingHeight, PaddingWidth, StrideHeight,
				StrideWidth, FilterDesc, FreeTerm.IsNull() ? nullptr : &freeTermDesc, Output ) );
		}
		engine.BlobChannelwiseConvolution( *Desc, input, Filter, FreeTerm.IsNull() ? nullptr : &FreeTerm, output );
	}
};

struct CHipRowwisePooling : public IHipRowwiseOperation {
	bool IsMax;
	int FilterHeight, FilterWidth, StrideHeight, StrideWidth;
	CBlobDesc Input, Output;
	std::unique_ptr<CMaxPoolingDesc> MaxDesc;
	std::unique_ptr<CMeanPoolingDesc> MeanDesc;

	CBlobDesc Reshape( const CBlobDesc& input ) override
	{
		Input = input;
		Output = input;
		Output.SetDimSize( BD_Height, 1 + ( input.Height() - FilterHeight ) / StrideHeight );
		Output.SetDimSize( BD_Width, 1 + ( input.Width() - FilterWidth ) / StrideWidth );
		MaxDesc.reset();
		MeanDesc.reset();
		return Output;
	}
	int OutputSize() const override { return Output.BlobSize(); }
	void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) override
	{
		if( IsMax ) {
			if( MaxDesc == nullptr ) {
				MaxDesc.reset( engine.InitMaxPooling( Input, FilterHeight, FilterWidth, StrideHeight, StrideWidth, Output ) );
			}
			engine.BlobMaxPooling( *MaxDesc, input, nullptr, output );
		} else {
			if( MeanDesc == nullptr ) {
				MeanDesc.reset( engine.InitMeanPooling( Input, FilterHeight, FilterWidth, StrideHeight, StrideWidth, Output ) );
			}
			engine.BlobMeanPooling( *MeanDesc, input, output );
		}
	}
};

struct CHipRowwiseResizeImage : public IHipRowwiseOperation {
	TBlobResizePadding Padding;
	float DefaultValue;
	int DeltaLeft, DeltaRight, DeltaTop, DeltaBottom;
	CBlobDesc Input, Output;

	CBlobDesc Reshape( const CBlobDesc& input ) override
	{
		Input = input;
		Output = input;
		Output.SetDimSize( BD_Width, input.Width() + DeltaLeft + DeltaRight );
		Output.SetDimSize( BD_Height, input.Height() + DeltaTop + DeltaBottom );
		return Output;
	}
	int OutputSize() const override { return Output.BlobSize(); }
	void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) override
	{
		// the blob operation of the interface takes its source as a non-const handle
		const CFloatHandle source( CTypedMemoryHandle<float>( static_cast<const CTypedMemoryHandle<const float>&>( input ) ) );
		engine.BlobResizeImage( Input, source, DeltaLeft, DeltaRight, DeltaTop, DeltaBottom, Padding, DefaultValue, Output, output );
	}
};

// ---- the two MobileNet blocks ---------------------------------------------------------------------------------

struct CHipRowwiseSeparableBlock : public IHipRowwiseOperation {
	bool WithExpand; // MobileNetV2 block (expand 1x1 first) or channelwise + 1x1
	nhSeparableBlockDesc D;
	CConstFloatHandle ExpandFilter, ExpandFreeTerm, ChannelwiseFilter, ChannelwiseFreeTerm, DownFilter, DownFreeTerm;
	CBlobDesc Output;

	CBlobDesc Reshape( const CBlobDesc& input ) override
	{
		D.batch = input.ObjectCount();
		D.height = input.Height();
		D.width = input.Width();
		if( !WithExpand ) {
			D.expandedChannels = input.Channels(); // the channelwise + 1x1 block learns its channel count from its input
		}
		Output = input;
		Output.SetDimSize( BD_Height, ( input.Height() + D.stride - 1 ) / D.stride );
		Output.SetDimSize( BD_Width, ( input.Width() + D.stride - 1 ) / D.stride );
		Output.SetDimSize( BD_Channels, D.outputChannels );
		return Output;
	}
	int OutputSize() const override { return Output.BlobSize(); }
	// with a residual connection the blocks run in place (the layers reuse their input blob)
	bool IsInPlace() const override { return false; }
	void Process( CHipMathEngine& engine, const CConstFloatHandle& input, const CFloatHandle& output ) override
	{
		engine.RunSeparableBlock( *this, input, output );
	}
};

void CHipMathEngine::RunSeparableBlock( const CRowwiseOperationDesc& desc, const CConstFloatHandle& input,
	const CFloatHandle& output )
{
	const CHipRowwiseSeparableBlock& block = static_cast<const CHipRowwiseSeparableBlock&>( desc );
	ASSERT_EXPR( input.GetMathEngine() == this && output.GetMathEngine() == this );
	size_t workspaceSize = 0;
	if( block.WithExpand ) {
		NH_CALL( nhMobileNetV2BlockWorkspaceSize( &block.D, &workspaceSize ) );
	} else {
		NH_CALL( nhChannelwiseWith1x1WorkspaceSize( &block.D, &workspaceSize ) );
	}
	const CMemoryHandle workspace = StackAlloc( std::max<size_t>( workspaceSize, 16 ) );
	auto optional = [this]( const CConstFloatHandle& h ) -> const float* { return h.IsNull() ? nullptr : raw( h ); };
	if( block.WithExpand ) {
		NH_CALL( nhMobileNetV2Block( stream, &block.D, raw( input ), raw( block.ExpandFilter ), optional( block.ExpandFreeTerm ),
			raw( block.ChannelwiseFilter ), optional( block.ChannelwiseFreeTerm ), raw( block.DownFilter ),
			optional( block.DownFreeTerm ), raw( output ), rawBytes( workspace ), workspaceSize ) );
	} else {
		NH_CALL( nhChannelwiseWith1x1( stream, &block.D, raw( input ), raw( block.ChannelwiseFilter ),
			optional( block.ChannelwiseFreeTerm ), raw( block.DownFilter ), optional( block.DownFreeTerm ), raw( output ),
			rawBytes( workspace ), workspaceSize ) );
	}
	// the stack block is recycled in stream order: later work on the same stream cannot overtake these kernels
	StackFree( workspace );
}

void CHipMathEngine::ChannelwiseWith1x1( const CBlobDesc& inputDesc, const CBlobDesc& /*outputDesc*/,
	const CRowwiseOperationDesc& rowwiseDesc, const CChannelwiseConvolutionDesc& /*convDesc*/,
	const CConstFloatHandle& inputHandle, const CFloatHandle& outputHandle )
{
	CHipRowwiseSeparableBlock& block = const_cast<CHipRowwiseSeparableBlock&>(
		static_cast<const CHipRowwiseSeparableBlock&>( rowwiseDesc ) );
	ASSERT_EXPR( !block.WithExpand );
	block.Reshape( inputDesc );
	RunSeparableBlock( block, inputHandle, outputHandle );
}

void CHipMathEngine::MobileNetV2Block( const CBlobDesc& inputDesc, const CBlobDesc& outputDesc,
	const CRowwiseOperationDesc& rowwiseDesc, const CChannelwiseConvolutionDesc& /*convDesc*/,
	const CConstFloatHandle& inputHandle, const CFloatHandle& outputHandle )
{
	CHipRowwiseSeparableBlock& block = const_cast<CHipRowwiseSeparableBlock&>(
		static_cast<const CHipRowwiseSeparableBlock&>( rowwiseDesc ) );
	ASSERT_EXPR( block.WithExpand );
	const CBlobDesc reshaped = block.Reshape( inputDesc );
	ASSERT_EXPR( reshaped.HasEqualDimensions( outputDesc ) );
	RunSeparableBlock( block, inputHandle, outputHandle );
}

// The halves of a MobileNetV3 block around its squeeze-and-excite branch (CMobileNetV3PreSEBlockLayer /
// CMobileNetV3PostSEBlockLayer call these directly with their parameter blobs)
void CHipMathEngine::MobileNetV3PreSEBlock( const CBlobDesc& inputDesc, const CBlobDesc& outputDesc,
	const CChannelwiseConvolutionDesc& convDesc, const CConstFloatHandle& inputHandle,
	const CConstFloatHandle& expandFilter, const CConstFloatHandle* expandFreeTerm,
	TActivationFunction expandActivation, float expandReluParam, const CConstFloatHandle& channelwiseFilter,
	const CConstFloatHandle* channelwiseFreeTerm, TActivationFunction channelwiseActivation,
	float channelwiseReluParam, const CFloatHandle& outputHandle )
{
	const CHipChannelwiseConvolutionDesc& d = static_cast<const CHipChannelwiseConvolutionDesc&>( convDesc );
	ASSERT_EXPR( outputDesc.Channels() == d.D.channels && inputDesc.ObjectCount() == d.D.batch );
	ASSERT_EXPR( inputDesc.Height() == d.D.height && inputDesc.Width() == d.D.width );
	size_t workspaceSize = 0;
	NH_CALL( nhMobileNetV3PreSEBlockWorkspaceSize( &d.D, &workspaceSize ) );
	const CMemoryHandle workspace = StackAlloc( std::max<size_t>( workspaceSize, 16 ) );
	NH_CALL( nhMobileNetV3PreSEBlock( stream, &d.D, inputDesc.Channels(), raw( inputHandle ), raw( expandFilter ),
		expandFreeTerm != nullptr ? raw( *expandFreeTerm ) : nullptr, fusedActivation( expandActivation ), expandReluParam,
		raw( channelwiseFilter ), channelwiseFreeTerm != nullptr ? raw( *channelwiseFreeTerm ) : nullptr,
		fusedActivation( channelwiseActivation ), channelwiseReluParam, raw( outputHandle ), rawBytes( workspace ),
		workspaceSize ) );
	StackFree( workspace );
}

void CHipMathEngine::MobileNetV3PostSEBlock( const CBlobDesc& channelwiseOutputDesc, int outputChannels,
	const CConstFloatHandle& channelwiseOutputHandle, const CConstFloatHandle& squeezeAndExciteHandle,
	const CConstFloatHandle* residualHandle, TActivationFunction activation, float reluParam,
	const CConstFloatHandle& downFilterHandle, const CConstFloatHandle* downFreeTermHandle,
	const CFloatHandle& outputHandle )
{
	const int batch = channelwiseOutputDesc.ObjectCount();
	const int pixels = channelwiseOutputDesc.Height() * channelwiseOutputDesc.Width();
	const int channels = channelwiseOutputDesc.Channels();
	const size_t workspaceSize = static_cast<size_t>( batch ) * pixels * channels * sizeof( float );
	const CMemoryHandle workspace = StackAlloc( std::max<size_t>( workspaceSize, 16 ) );
	NH_CALL( nhMobileNetV3PostSEBlock( stream, batch, pixels, channels, outputChannels, raw( channelwiseOutputHandle ),
		raw( squeezeAndExciteHandle ), residualHandle != nullptr ? raw( *residualHandle ) : nullptr,
		fusedActivation( activation ), reluParam, raw( downFilterHandle ),
		downFreeTermHandle != nullptr ? raw( *downFreeTermHandle ) : nullptr, raw( outputHandle ), rawBytes( workspace ),
		workspaceSize ) );
	StackFree( workspace );
}

// ---- descriptors ----------------------------------------------------------------------------------------------

CRowwiseOperationDesc* CHipMathEngine::InitRowwiseActivation( const CActivationDesc& desc )
{
	return new CHipRowwiseActivation( desc );
}

CRowwiseOperationDesc* CHipMathEngine::InitRowwiseChWith1x1( int stride, const CConstFloatHandle& channelwiseFilter,
	const CConstFloatHandle* channelwiseFreeTerm, TActivationFunction activation, float reluParam,
	const CConstFloatHandle& convFilter, const CConstFloatHandle* convFreeTerm, int outputChannels, bool residual )
{
	CHipRowwiseSeparableBlock* block = new CHipRowwiseSeparableBlock();
	block->WithExpand = false;
	block->D = nhSeparableBlockDesc();
	block->D.stride = stride;
	block->D.residual = residual ? 1 : 0;
	block->D.outputChannels = outputChannels;
	block->D.channelwiseActivation = fusedActivation( activation );
	block->D.channelwiseParam = reluParam;
	block->ChannelwiseFilter = channelwiseFilter;
	block->ChannelwiseFreeTerm = channelwiseFreeTerm == nullptr ? CConstFloatHandle() : *channelwiseFreeTerm;
	block->DownFilter = convFilter;
	block->DownFreeTerm = convFreeTerm == nullptr ? CConstFloatHandle() : *convFreeTerm;
	return block;
}

CRowwiseOperationDesc* CHipMathEngine::InitRowwiseMobileNetV2( int inputChannels, const CConstFloatHandle& expandFilter,
	const CConstFloatHandle* expandFreeTerm, int expandedChannels, TActivationFunction expandActivation,
	float expandReluParam, const CConstFloatHandle& channelwiseFilter, const CConstFloatHandle* channelwiseFreeTerm,
	int stride, TActivationFunction channelwiseActivation, float channelwiseReluParam,
	const CConstFloatHandle& downFilter, const CConstFloatHandle* downFreeTerm, int outputChannels, bool residual )
{
	CHipRowwiseSeparableBlock* block = new CHipRowwiseSeparableBlock();
	block->WithExpand = true;
	block->D = nhSeparableBlockDesc();
	block->D.inputChannels = inputChannels;
	block->D.expandedChannels = expandedChannels;
	block->D.outputChannels = outputChannels;
	block->D.stride = stride;
	block->D.residual = residual ? 1 : 0;
	block->D.expandActivation = fusedActivation( expandActivation );
	block->D.expandParam = expandReluParam;
	block->D.channelwiseActivation = fusedActivation( channelwiseActivation );
	block->D.channelwiseParam = channelwiseReluParam;
	block->ExpandFilter = expandFilter;
	block->ExpandFreeTerm = expandFreeTerm == nullptr ? CConstFloatHandle() : *expandFreeTerm;
	block->ChannelwiseFilter = channelwiseFilter;
	block->ChannelwiseFreeTerm = channelwiseFreeTerm == nullptr ? CConstFloatHandle() : *channelwiseFreeTerm;
	block->DownFilter = downFilter;
	block->DownFreeTerm = downFreeTerm == nullptr ? CConstFloatHandle() : *downFreeTerm;
	return block;
}

CRowwiseOperationDesc* CHipMathEngine::InitRowwiseConv( int paddingHeight, int paddingWidth, int strideHeight,
	int strideWidth, int dilationHeight, int dilationWidth, const CBlobDesc& filterDesc,
	const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm )
{
	CHipRowwiseConv* op = new CHipRowwiseConv();
	op->PaddingHeight = paddingHeight; op->PaddingWidth = paddingWidth;
	op->StrideHeight = strideHeight; op->StrideWidth = strideWidth;
	op->DilationHeight = dilationHeight; op->DilationWidth = dilationWidth;
	op->FilterDesc = filterDesc;
	op->Filter = filter;
	op->FreeTerm = freeTerm == nullptr ? CConstFloatHandle() : *freeTerm;
	return op;
}

CRowwiseOperationDesc* CHipMathEngine::InitRowwiseChConv( int paddingHeight, int paddingWidth, int strideHeight,
	int strideWidth, const CBlobDesc& filterDesc, const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm )
{
	CHipRowwiseChConv* op = new CHipRowwiseChConv();
	op->PaddingHeight = paddingHeight; op->PaddingWidth = paddingWidth;
	op->StrideHeight = strideHeight; op->StrideWidth = strideWidth;
	op->FilterDesc = filterDesc;
	op->Filter = filter;
	op->FreeTerm = freeTerm == nullptr ? CConstFloatHandle() : *freeTerm;
	return op;
}

CRowwiseOperationDesc* CHipMathEngine::InitRowwise2DPooling( bool isMax, int filterHeight, int filterWidth,
	int strideHeight, int strideWidth )
{
	CHipRowwisePooling* op = new CHipRowwisePooling();
	op->IsMax = isMax;
	op->FilterHeight = filterHeight; op->FilterWidth = filterWidth;
	op->StrideHeight = strideHeight; op->StrideWidth = strideWidth;
	return op;
}

CRowwiseOperationDesc* CHipMathEngine::InitRowwiseResizeImage( TBlobResizePadding padding, float defaultValue,
	int deltaLeft, int deltaRight, int deltaTop, int deltaBottom )
{
	CHipRowwiseResizeImage* op = new CHipRowwiseResizeImage();
	op->Padding = padding;
	op->DefaultValue = defaultValue;
	op->DeltaLeft = deltaLeft; op->DeltaRight = deltaRight; op->DeltaTop = deltaTop; op->DeltaBottom = deltaBottom;
	return op;
}

// ---- chains ---------------------------------------------------------------------------------------------------

CBlobDesc CHipMathEngine::RowwiseReshape( CRowwiseOperationDesc** operations, int operationCount, const CBlobDesc& input )
{
	CBlobDesc output = input;
	for( int i = 0; i < operationCount; ++i ) {
		IHipRowwiseOperation* operation = dynamic_cast<IHipRowwiseOperation*>( operations[i] );
		ASSERT_EXPR( operation != nullptr );
		output = operation->Reshape( output );
	}
	return output;
}

void CHipMathEngine::RowwiseExecute( const CBlobDesc& /*inputDesc*/, CRowwiseOperationDesc** operations, int operationCount,
	const CFloatHandle& input, const CFloatHandle& output )
{
	// an in-place operation joins the stage of the operation before it: it runs on that stage's output
	std::vector<std::vector<IHipRowwiseOperation*>> stages;
	for( int i = 0; i < operationCount; ++i ) {
		IHipRowwiseOperation* operation = dynamic_cast<IHipRowwiseOperation*>( operations[i] );
		ASSERT_EXPR( operation != nullptr );
		if( i == 0 || !operation->IsInPlace() ) {
			stages.emplace_back();
		}
		stages.back().push_back( operation );
	}
	// intermediate results alternate between two buffers sized for the largest of them
	int largest = 0;
	for( size_t i = 0; i + 1 < stages.size(); ++i ) {
		largest = std::max( largest, stages[i][0]->OutputSize() );
	}
	std::unique_ptr<CFloatHandleVar> buffers[2];
	CConstFloatHandle current = input;
	for( size_t i = 0; i < stages.size(); ++i ) {
		CFloatHandle target = output;
		if( i + 1 < stages.size() ) {
			std::unique_ptr<CFloatHandleVar>& buffer = buffers[i & 1];
			if( buffer == nullptr ) {
				buffer.reset( new CFloatHandleVar( *this, static_cast<size_t>( largest ) ) );
			}
			target = buffer->GetHandle();
		}
		size_t next = 1;
		CHipRowwiseConv* conv = dynamic_cast<CHipRowwiseConv*>( stages[i][0] );
		CHipRowwiseActivation* activation = stages[i].size() > 1 ? dynamic_cast<CHipRowwiseActivation*>( stages[i][1] ) : nullptr;
		if( conv != nullptr && activation != nullptr && fusedActivation( activation->Desc.GetType() ) != NH_ACT_NONE ) {
			// convolution + ReLU / h-swish: the activation rides in the epilogue of the convolution
			const float param = activation->Desc.GetType() == AF_ReLU
				? activation->Desc.GetParam<CReLUActivationParam>().UpperThreshold : 0.f;
			conv->ProcessWithActivation( *this, current, target, fusedActivation( activation->Desc.GetType() ), param );
			next = 2;
		} else {
			stages[i][0]->Process( *this, current, target );
		}
		for( size_t j = next; j < stages[i].size(); ++j ) {
			stages[i][j]->Process( *this, target, target );
		}
		current = target;
	}
}

} // namespace NeoML
