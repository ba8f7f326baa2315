// CHipMathEngine implementation: every method resolves its handles and calls one entry point of the C ABI.
#include "HipMathEngine.h"

#include <chrono>
#include <cstring>
#include <memory>
#include <new>

namespace NeoML {

#define NH_CALL( expr ) check( ( expr ), #expr, __LINE__ )
#define OWN( handle ) ASSERT_EXPR( ( handle ).GetMathEngine() == this )

// ---------------------------------------------------------------------------------------------------------
// descriptors (deleted by the caller with plain delete, hence CCrtAllocatedObject through the base structs)

struct CHipMaxPoolingDesc : public CMaxPoolingDesc {
	nhPoolingDesc D;
};

struct CHipMeanPoolingDesc : public CMeanPoolingDesc {
	nhPoolingDesc D;
};

// Keeps pointers to caller-owned weights, as the reference's LSTM descriptor does
// (src/CPU/CpuMathEngineDnnLstm.cpp:66-78)
struct CHipLstmDesc : public CLstmDesc {
	int HiddenSize;
	int ObjectSize;
	CConstFloatHandle InputWeights, InputFreeTerm, RecurrentWeights, RecurrentFreeTerm;
	// The workspace of the calls with this descriptor, grown on demand and kept: two LSTMs with descriptors of their
	// own ( the two directions of a bidirectional layer ) then work in different memory, which is what lets the second
	// run beside the first ( nhStreamOverlapLstm ). Blocks handed back go to the engine's pool and are reused in stream
	// order, behind the kernels that used them.
	IMathEngine* Engine = nullptr;
	CMemoryHandle Workspace;
	size_t WorkspaceSize = 0;
	~CHipLstmDesc() override
	{
		if( !Workspace.IsNull() ) {
			Engine->HeapFree( Workspace );
		}
	}
};

static nhBlobDesc toBlobDesc( const CBlobDesc& desc )
{
	nhBlobDesc d;
	for( int i = 0; i < 7; ++i ) {
		d.dims[i] = desc.DimSize( i );
	}
	return d;
}

// ---------------------------------------------------------------------------------------------------------
// time counter: counter[0] = nanoseconds between two Synchronise() calls, the device stream drained first so
// that per-layer timings of CDnn::EnableProfile measure finished work (PerformanceCounters.h:27-60)

class CHipPerformanceCounters : public IPerformanceCounters {
public:
	explicit CHipPerformanceCounters( const CHipMathEngine& engine ) :
		IPerformanceCounters( &counter ), engine( engine ), last( now() )
	{
		counter.Name = "time ns";
		counter.Value = 0;
		CounterCount() = 1;
	}
	void Synchronise() override
	{
		engine.Synchronize();
		const uint_least64_t current = now();
		counter.Value = current - last;
		last = current;
	}

private:
	const CHipMathEngine& engine;
	CCounter counter;
	uint_least64_t last;

	static uint_least64_t now()
	{
		return static_cast<uint_least64_t>( std::chrono::duration_cast<std::chrono::nanoseconds>(
			std::chrono::steady_clock::now().time_since_epoch() ).count() );
	}
};

// ---------------------------------------------------------------------------------------------------------

CHipMathEngine::CHipMathEngine( int deviceIndex, size_t memoryLimit, int /*flags*/ ) :
	device( deviceIndex ),
	memoryLimit( memoryLimit ),
	stream( nullptr ),
	pool( nullptr ),
	deviceTotalMemory( 0 ),
	initialized( false )
{
	deviceName[0] = 0;
	NH_CALL( nhSetDevice( device ) );
	NH_CALL( nhGetDeviceInfo( device, deviceName, &deviceTotalMemory, nullptr, nullptr, nullptr ) );
	NH_CALL( nhStreamCreate( &stream ) );
	NH_CALL( nhPoolCreate( &pool, 0, memoryLimit ) );
	// what the kernels allocate behind the scenes for this stream is charged to the engine's pool
	NH_CALL( nhStreamBindPool( stream, pool ) );
	// all of this engine's work is enqueued through the library: independent one-launch LSTMs may run side by side
	NH_CALL( nhStreamOverlapLstm( stream, 1 ) );
	// ... and runs of small element-wise calls ( the per-row scalars of CObjectNormalizationLayer ) may share a launch:
	// every wait of this engine is nhStreamSynchronize or a copy through the library, which launch them first
	NH_CALL( nhStreamDeferSmallOps( stream, 1 ) );
	initialized = true;
}

CHipMathEngine::~CHipMathEngine()
{
	if( stream != nullptr ) {
		nhStreamSynchronize( stream );
	}
	for( auto& t : hostBuffers ) {
		for( CHostBuffer& b : t.second.Blocks ) {
			nhHostFree( b.Ptr );
		}
	}
	if( stream != nullptr ) {
		nhStreamBindPool( stream, nullptr ); // the stream's scratch goes back to the pool before the pool goes
	}
	if( pool != nullptr ) {
		nhPoolDestroy( pool );
	}
	if( stream != nullptr ) {
		nhStreamDestroy( stream );
	}
}

void CHipMathEngine::check( int code, const char* what, int line ) const
{
	if( code == NH_OK ) {
		return;
	}
	if( code == NH_ERR_MEMORY ) {
		GetMathEngineExceptionHandler()->OnMemoryError();
		return;
	}
	// the message of the failed call; `what` names the call for handlers that log it
	const char* message = nhGetLastError();
	GetMathEngineExceptionHandler()->OnAssert( ( message != nullptr && message[0] != 0 ) ? message : what,
		L"HipMathEngine.cpp", line, code );
}

void* CHipMathEngine::rawBytes( const CMemoryHandle& handle ) const
{
	ASSERT_EXPR( handle.GetMathEngine() == this );
	return CMemoryHandleInternal::GetRaw( handle );
}

void CHipMathEngine::Synchronize() const
{
	NH_CALL( nhStreamSynchronize( stream ) );
}

// ---------------------------------------------------------------------------------------------------------
// IVectorMathEngine

void CHipMathEngine::VectorCopy( const CFloatHandle& first, const CConstFloatHandle& second, int vectorSize )
{
	NH_CALL( nhVectorCopy( stream, raw( first ), raw( second ), vectorSize ) );
}

void CHipMathEngine::VectorCopy( const CIntHandle& first, const CConstIntHandle& second, int vectorSize )
{
	NH_CALL( nhVectorCopyInt( stream, raw( first ), raw( second ), vectorSize ) );
}

void CHipMathEngine::BroadcastCopy( const CIntHandle& toHandle, const CConstIntHandle& fromHandle, const CBlobDesc& toDesc,
	const CBlobDesc& fromDesc, int additionalWidth )
{
	const nhBlobDesc to = toBlobDesc( toDesc ), from = toBlobDesc( fromDesc );
	NH_CALL( nhBroadcastCopy( stream, raw( toHandle ), raw( fromHandle ), &to, &from, additionalWidth ) );
}

void CHipMathEngine::BroadcastCopy( const CFloatHandle& toHandle, const CConstFloatHandle& fromHandle,
	const CBlobDesc& toDesc, const CBlobDesc& fromDesc, int additionalWidth )
{
	const nhBlobDesc to = toBlobDesc( toDesc ), from = toBlobDesc( fromDesc );
	NH_CALL( nhBroadcastCopy( stream, raw( toHandle ), raw( fromHandle ), &to, &from, additionalWidth ) );
}

void CHipMathEngine::VectorFill( const CFloatHandle& result, float value, int vectorSize )
{
	NH_CALL( nhVectorFill( stream, raw( result ), value, vectorSize ) );
}

void CHipMathEngine::VectorFill( const CIntHandle& result, int value, int vectorSize )
{
	NH_CALL( nhVectorFillInt( stream, raw( result ), value, vectorSize ) );
}

void CHipMathEngine::VectorFill( const CFloatHandle& result, int vectorSize, const CConstFloatHandle& value )
{
	NH_CALL( nhVectorFillFromHandle( stream, raw( result ), vectorSize, raw( value ) ) );
}

void CHipMathEngine::VectorFill( const CIntHandle& result, int vectorSize, const CConstIntHandle& value )
{
	NH_CALL( nhVectorFillFromHandleInt( stream, raw( result ), vectorSize, raw( value ) ) );
}

void CHipMathEngine::VectorConvert( const CConstFloatHandle& from, const CIntHandle& to, int vectorSize )
{
	NH_CALL( nhVectorConvertFloatToInt( stream, raw( from ), raw( to ), vectorSize ) );
}

void CHipMathEngine::VectorConvert( const CConstIntHandle& from, const CFloatHandle& to, int vectorSize )
{
	NH_CALL( nhVectorConvertIntToFloat( stream, raw( from ), raw( to ), vectorSize ) );
}

void CHipMathEngine::VectorSum( const CConstFloatHandle& firstHandle, int vectorSize, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorSum( stream, raw( firstHandle ), vectorSize, raw( resultHandle ) ) );
}

void CHipMathEngine::VectorDotProduct( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	int vectorSize, const CFloatHandle& resultHandle )
{
	NH_CALL( nhVectorDotProduct( stream, raw( firstHandle ), raw( secondHandle ), vectorSize, raw( resultHandle ) ) );
}

// result = f( first )
#define HIP_UNARY( Method, entry ) \
	void CHipMathEngine::Method( const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle, int vectorSize ) \
	{ NH_CALL( entry( stream, raw( firstHandle ), raw( resultHandle ), vectorSize ) ); }

// result = f( first; scalar in engine memory )
#define HIP_UNARY_SCALAR( Method, entry ) \
	void CHipMathEngine::Method( const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle, int vectorSize, \
		const CConstFloatHandle& scalarHandle ) \
	{ NH_CALL( entry( stream, raw( firstHandle ), raw( resultHandle ), vectorSize, raw( scalarHandle ) ) ); }

// result = f( first, second )
#define HIP_BINARY( Method, THandle, TConstHandle, entry ) \
	void CHipMathEngine::Method( const TConstHandle& firstHandle, const TConstHandle& secondHandle, \
		const THandle& resultHandle, int vectorSize ) \
	{ NH_CALL( entry( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize ) ); }

HIP_UNARY( VectorHSwish, nhVectorHSwish )
HIP_UNARY( VectorAbs, nhVectorAbs )
HIP_UNARY( VectorHardTanh, nhVectorHardTanh )
HIP_UNARY( VectorNeg, nhVectorNeg )
HIP_UNARY( VectorExp, nhVectorExp )
HIP_UNARY( VectorLog, nhVectorLog )
HIP_UNARY( VectorErf, nhVectorErf )
HIP_UNARY( VectorSqrt, nhVectorSqrt )
HIP_UNARY( VectorInv, nhVectorInv )
HIP_UNARY( VectorSigmoid, nhVectorSigmoid )
HIP_UNARY( VectorTanh, nhVectorTanh )

HIP_UNARY( VectorNegLog, nhVectorNegLog )

HIP_UNARY( VectorHinge, nhVectorHinge )
HIP_UNARY( VectorSquaredHinge, nhVectorSquaredHinge )
HIP_UNARY( VectorHuber, nhVectorHuber )
HIP_UNARY( VectorHuberDerivative, nhVectorHuberDerivative )

HIP_UNARY_SCALAR( VectorELU, nhVectorELU )
HIP_UNARY_SCALAR( VectorReLU, nhVectorReLU )
HIP_UNARY_SCALAR( VectorLeakyReLU, nhVectorLeakyReLU )
HIP_UNARY_SCALAR( VectorAddValue, nhVectorAddValue )
HIP_UNARY_SCALAR( VectorMultiply, nhVectorMultiply )
HIP_UNARY_SCALAR( VectorNegMultiply, nhVectorNegMultiply )

HIP_BINARY( VectorEltwiseMax, CFloatHandle, CConstFloatHandle, nhVectorEltwiseMax )
HIP_BINARY( VectorEltwiseMin, CFloatHandle, CConstFloatHandle, nhVectorEltwiseMin )
HIP_BINARY( VectorAdd, CFloatHandle, CConstFloatHandle, nhVectorAdd )
HIP_BINARY( VectorAdd, CIntHandle, CConstIntHandle, nhVectorAddInt )
HIP_BINARY( VectorSub, CFloatHandle, CConstFloatHandle, nhVectorSub )
HIP_BINARY( VectorSub, CIntHandle, CConstIntHandle, nhVectorSubInt )
HIP_BINARY( VectorEltwiseMultiply, CFloatHandle, CConstFloatHandle, nhVectorEltwiseMultiply )
HIP_BINARY( VectorEltwiseMultiply, CIntHandle, CConstIntHandle, nhVectorEltwiseMultiplyInt )
HIP_BINARY( VectorEltwiseMultiplyAdd, CFloatHandle, CConstFloatHandle, nhVectorEltwiseMultiplyAdd )
HIP_BINARY( VectorEltwiseNegMultiply, CFloatHandle, CConstFloatHandle, nhVectorEltwiseNegMultiply )
HIP_BINARY( VectorEltwiseDivide, CFloatHandle, CConstFloatHandle, nhVectorEltwiseDivide )

// derivatives of the activations: result = f'( first ) * second; the Op forms take the activation's output as first
HIP_BINARY( VectorHSwishDiff, CFloatHandle, CConstFloatHandle, nhVectorHSwishDiff )
HIP_BINARY( VectorSigmoidDiff, CFloatHandle, CConstFloatHandle, nhVectorSigmoidDiff )
HIP_BINARY( VectorSigmoidDiffOp, CFloatHandle, CConstFloatHandle, nhVectorSigmoidDiffOp )
HIP_BINARY( VectorTanhDiff, CFloatHandle, CConstFloatHandle, nhVectorTanhDiff )
HIP_BINARY( VectorTanhDiffOp, CFloatHandle, CConstFloatHandle, nhVectorTanhDiffOp )

void CHipMathEngine::VectorReLUDiff( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& upperThresholdHandle )
{
	NH_CALL( nhVectorReLUDiff( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize,
		raw( upperThresholdHandle ) ) );
}

// ReLU's output is positive and below the threshold exactly where its input is: the same test on either
// (CpuMathEngine.h:763-767)
void CHipMathEngine::VectorReLUDiffOp( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& upperThresholdHandle )
{
	VectorReLUDiff( firstHandle, secondHandle, resultHandle, vectorSize, upperThresholdHandle );
}

HIP_BINARY( VectorHingeDiff, CFloatHandle, CConstFloatHandle, nhVectorHingeDiff )
HIP_BINARY( VectorSquaredHingeDiff, CFloatHandle, CConstFloatHandle, nhVectorSquaredHingeDiff )

void CHipMathEngine::VectorL1DiffAdd( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& hubertThresholdHandle,
	const CConstFloatHandle& multHandle )
{
	NH_CALL( nhVectorL1DiffAdd( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize,
		raw( hubertThresholdHandle ), raw( multHandle ) ) );
}

HIP_BINARY( VectorAbsDiff, CFloatHandle, CConstFloatHandle, nhVectorAbsDiff )
// inside ( -1, 1 ) on the input exactly where the output is: one test for both forms, as for ReLU
HIP_BINARY( VectorHardTanhDiff, CFloatHandle, CConstFloatHandle, nhVectorHardTanhDiff )
HIP_BINARY( VectorHardTanhDiffOp, CFloatHandle, CConstFloatHandle, nhVectorHardTanhDiff )

// result = f'( first; alpha in engine memory ) * second
#define HIP_BINARY_ALPHA( Method, entry ) \
	void CHipMathEngine::Method( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle, \
		const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& alpha ) \
	{ NH_CALL( entry( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize, raw( alpha ) ) ); }

HIP_BINARY_ALPHA( VectorELUDiff, nhVectorELUDiff )
HIP_BINARY_ALPHA( VectorELUDiffOp, nhVectorELUDiffOp )
HIP_BINARY_ALPHA( VectorLeakyReLUDiff, nhVectorLeakyReLUDiff )
HIP_BINARY_ALPHA( VectorLeakyReLUDiffOp, nhVectorLeakyReLUDiff ) // a positive alpha keeps the sign: same test

void CHipMathEngine::VectorHardSigmoidDiff( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& slopeHandle,
	const CConstFloatHandle& biasHandle )
{
	NH_CALL( nhVectorHardSigmoidDiff( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize,
		raw( slopeHandle ), raw( biasHandle ) ) );
}

void CHipMathEngine::VectorHardSigmoidDiffOp( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& slopeHandle,
	const CConstFloatHandle& /*biasHandle*/ )
{
	NH_CALL( nhVectorHardSigmoidDiffOp( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize,
		raw( slopeHandle ) ) );
}

void CHipMathEngine::VectorSub( const CConstFloatHandle& firstHandle, float second, const CFloatHandle& resultHandle,
	int vectorSize )
{
	NH_CALL( nhVectorSubValue( stream, raw( firstHandle ), second, 0, raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::VectorSub( float first, const CConstFloatHandle& secondHandle, const CFloatHandle& resultHandle,
	int vectorSize )
{
	NH_CALL( nhVectorSubValue( stream, raw( secondHandle ), first, 1, raw( resultHandle ), vectorSize ) );
}

void CHipMathEngine::MatrixSoftmaxDiffOpByRows( const CConstFloatHandle& first, const CConstFloatHandle& second,
	int height, int width, const CFloatHandle& result )
{
	NH_CALL( nhMatrixSoftmaxDiffOpByRows( stream, raw( first ), raw( second ), height, width, raw( result ) ) );
}

void CHipMathEngine::MultiplyDiagMatrixByMatrixAndAdd( int batchSize, const CConstFloatHandle& firstHandle,
	int firstSize, const CConstFloatHandle& secondHandle, int secondWidth, const CFloatHandle& resultHandle )
{
	NH_CALL( nhMultiplyDiagMatrixByMatrixAndAdd( stream, batchSize, raw( firstHandle ), firstSize, raw( secondHandle ),
		secondWidth, raw( resultHandle ) ) );
}

void CHipMathEngine::RowMultiplyMatrixByMatrix( const CConstFloatHandle& firstHandle,
	const CConstFloatHandle& secondHandle, int height, int width, const CFloatHandle& result )
{
	NH_CALL( nhRowMultiplyMatrixByMatrix( stream, raw( firstHandle ), raw( secondHandle ), height, width, raw( result ) ) );
}

void CHipMathEngine::VectorAddValue( const CConstIntHandle& firstHandle, const CIntHandle& resultHandle, int vectorSize,
	const CConstIntHandle& addition )
{
	NH_CALL( nhVectorAddValueInt( stream, raw( firstHandle ), raw( resultHandle ), vectorSize, raw( addition ) ) );
}

void CHipMathEngine::VectorMultiply( const CConstIntHandle& firstHandle, const CIntHandle& resultHandle, int vectorSize,
	const CConstIntHandle& multiplierHandle )
{
	NH_CALL( nhVectorMultiplyInt( stream, raw( firstHandle ), raw( resultHandle ), vectorSize, raw( multiplierHandle ) ) );
}

void CHipMathEngine::VectorHardSigmoid( const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle,
	int vectorSize, const CConstFloatHandle& slopeHandle, const CConstFloatHandle& biasHandle )
{
	NH_CALL( nhVectorHardSigmoid( stream, raw( firstHandle ), raw( resultHandle ), vectorSize, raw( slopeHandle ),
		raw( biasHandle ) ) );
}

void CHipMathEngine::VectorMinMax( const CConstFloatHandle& firstHandle, const CFloatHandle& resultHandle, int vectorSize,
	const CConstFloatHandle& minHandle, const CConstFloatHandle& maxHandle )
{
	NH_CALL( nhVectorMinMax( stream, raw( firstHandle ), raw( resultHandle ), vectorSize, raw( minHandle ), raw( maxHandle ) ) );
}

void CHipMathEngine::VectorMultiplyAndAdd( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& multHandle )
{
	NH_CALL( nhVectorMultiplyAndAdd( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize,
		raw( multHandle ) ) );
}

void CHipMathEngine::VectorMultiplyAndSub( const CConstFloatHandle& firstHandle, const CConstFloatHandle& secondHandle,
	const CFloatHandle& resultHandle, int vectorSize, const CConstFloatHandle& multHandle )
{
	NH_CALL( nhVectorMultiplyAndSub( stream, raw( firstHandle ), raw( secondHandle ), raw( resultHandle ), vectorSize,
		raw( multHandle ) ) );
}

// ---------------------------------------------------------------------------------------------------------
// IBlasEngine

void CHipMathEngine::SetVectorToMatrixRows( const CFloatHandle& resultHandle, int matrixHeight, int matrixWidth,
	const CConstFloatHandle& vectorHandle )
{
	NH_CALL( nhSetVectorToMatrixRows( stream, raw( resultHandle ), matrixHeight, matrixWidth, raw( vectorHandle ) ) );
}

void CHipMathEngine::AddVectorToMatrixRows( int batchSize, const CConstFloatHandle& matrixHandle,
	const CFloatHandle& resultHandle, int matrixHeight, int matrixWidth, const CConstFloatHandle& vectorHandle )
{
	NH_CALL( nhAddVectorToMatrixRows( stream, batchSize, raw( matrixHandle ), raw( resultHandle ), matrixHeight,
		matrixWidth, raw( vectorHandle ) ) );
}

void CHipMathEngine::AddVectorToMatrixColumns( const CConstFloatHandle& matrixHandle, const CFloatHandle& resultHandle,
	int matrixHeight, int matrixWidth, const CConstFloatHandle& vectorHandle )
{
	NH_CALL( nhAddVectorToMatrixColumns( stream, raw( matrixHandle ), raw( resultHandle ), matrixHeight, matrixWidth,
		raw( vectorHandle ) ) );
}

void CHipMathEngine::SubVectorFromMatrixColumns( const CConstFloatHandle& matrixHandle, const CFloatHandle& resultHandle,
	int matrixHeight, int matrixWidth, const CConstFloatHandle& vectorHandle )
{
	NH_CALL( nhSubVectorFromMatrixColumns( stream, raw( matrixHandle ), raw( resultHandle ), matrixHeight, matrixWidth,
		raw( vectorHandle ) ) );
}

void CHipMathEngine::SumMatrixRowsAdd( int batchSize, const CFloatHandle& resultHandle,
	const CConstFloatHandle& matrixHandle, int matrixHeight, int matrixWidth )
{
	NH_CALL( nhSumMatrixRowsAdd( stream, batchSize, raw( resultHandle ), raw( matrixHandle ), matrixHeight, matrixWidth ) );
}

void CHipMathEngine::SumMatrixRows( int batchSize, const CFloatHandle& resultHandle,
	const CConstFloatHandle& matrixHandle, int matrixHeight, int matrixWidth )
{
	NH_CALL( nhSumMatrixRows( stream, batchSize, raw( resultHandle ), raw( matrixHandle ), matrixHeight, matrixWidth ) );
}

void CHipMathEngine::SumMatrixColumns( const CFloatHandle& resultHandle, const CConstFloatHandle& matrixHandle,
	int matrixHeight, int matrixWidth )
{
	NH_CALL( nhSumMatrixColumns( stream, raw( resultHandle ), raw( matrixHandle ), matrixHeight, matrixWidth ) );
}

void CHipMathEngine::MatrixLogSumExpByRows( const CConstFloatHandle& matrix, int height, int width,
	const CFloatHandle& result, int resultSize )
{
	NH_CALL( nhMatrixLogSumExpByRows( stream, raw( matrix ), height, width, raw( result ), resultSize ) );
}

void CHipMathEngine::MatrixSoftmaxByRows( const CConstFloatHandle& matrix, int height, int width,
	const CFloatHandle& result )
{
	NH_CALL( nhMatrixSoftmaxByRows( stream, raw( matrix ), height, width, raw( result ) ) );
}

void CHipMathEngine::FindMaxValueInRows( const CConstFloatHandle& matrixHandle, int matrixHeight, int matrixWidth,
	const CFloatHandle& resultHandle, const CIntHandle& columnIndices, int vectorSize )
{
	NH_CALL( nhFindMaxValueInRows( stream, raw( matrixHandle ), matrixHeight, matrixWidth, raw( resultHandle ),
		raw( columnIndices ), vectorSize ) );
}

void CHipMathEngine::FindMaxValueInRows( const CConstFloatHandle& matrixHandle, int matrixHeight, int matrixWidth,
	const CFloatHandle& resultHandle, int vectorSize )
{
	NH_CALL( nhFindMaxValueInRows( stream, raw( matrixHandle ), matrixHeight, matrixWidth, raw( resultHandle ),
		nullptr, vectorSize ) );
}

void CHipMathEngine::FindMaxValueInColumns( int batchSize, const CConstFloatHandle& matrixHandle, int matrixHeight,
	int matrixWidth, const CFloatHandle& resultHandle, const CIntHandle& rowIndices, int vectorSize )
{
	NH_CALL( nhFindMaxValueInColumns( stream, batchSize, raw( matrixHandle ), matrixHeight, matrixWidth,
		raw( resultHandle ), raw( rowIndices ), vectorSize ) );
}

void CHipMathEngine::MultiplyMatrixByTransposedMatrix( const CConstFloatHandle& firstHandle, int firstHeight,
	int firstWidth, int firstRowSize, const CConstFloatHandle& secondHandle, int secondHeight, int secondRowSize,
	const CFloatHandle& resultHandle, int resultRowSize, int resultBufferSize )
{
	NH_CALL( nhMultiplyMatrixByTransposedMatrix( stream, raw( firstHandle ), firstHeight, firstWidth, firstRowSize,
		raw( secondHandle ), secondHeight, secondRowSize, raw( resultHandle ), resultRowSize, resultBufferSize ) );
}

void CHipMathEngine::MultiplyMatrixByTransposedMatrix( int batchSize, const CConstFloatHandle& firstHandle,
	int firstHeight, int firstWidth, const CConstFloatHandle& secondHandle, int secondHeight,
	const CFloatHandle& resultHandle, int resultBufferSize )
{
	NH_CALL( nhBatchMultiplyMatrixByTransposedMatrix( stream, batchSize, raw( firstHandle ), firstHeight, firstWidth,
		raw( secondHandle ), secondHeight, raw( resultHandle ), resultBufferSize ) );
}

void CHipMathEngine::MultiplyTransposedMatrixByMatrixAndAdd( const CConstFloatHandle& firstHandle, int firstHeight,
	int firstWidth, int firstRowSize, const CConstFloatHandle& secondHandle, int secondWidth, int secondRowSize,
	const CFloatHandle& resultHandle, int resultRowSize, int resultBufferSize )
{
	NH_CALL( nhMultiplyTransposedMatrixByMatrixAndAdd( stream, raw( firstHandle ), firstHeight, firstWidth, firstRowSize,
		raw( secondHandle ), secondWidth, secondRowSize, raw( resultHandle ), resultRowSize, resultBufferSize ) );
}

void CHipMathEngine::MultiplyTransposedMatrixByMatrix( int batchSize, const CConstFloatHandle& firstHandle,
	int firstHeight, int firstWidth, const CConstFloatHandle& secondHandle, int secondWidth,
	const CFloatHandle& resultHandle, int resultBufferSize )
{
	NH_CALL( nhBatchMultiplyTransposedMatrixByMatrix( stream, batchSize, raw( firstHandle ), firstHeight, firstWidth,
		raw( secondHandle ), secondWidth, raw( resultHandle ), resultBufferSize ) );
}

void CHipMathEngine::MultiplyDiagMatrixByMatrix( const CConstFloatHandle& firstHandle, int firstSize,
	const CConstFloatHandle& secondHandle, int secondWidth, const CFloatHandle& resultHandle, int resultBufferSize )
{
	NH_CALL( nhMultiplyDiagMatrixByMatrix( stream, raw( firstHandle ), firstSize, raw( secondHandle ), secondWidth,
		raw( resultHandle ), resultBufferSize ) );
}

void CHipMathEngine::MultiplyMatrixByMatrix( int batchSize, const CConstFloatHandle& firstHandle, int firstHeight,
	int firstWidth, const CConstFloatHandle& secondHandle, int secondWidth, const CFloatHandle& resultHandle,
	int resultBufferSize )
{
	NH_CALL( nhBatchMultiplyMatrixByMatrix( stream, batchSize, raw( firstHandle ), firstHeight, firstWidth,
		raw( secondHandle ), secondWidth, raw( resultHandle ), resultBufferSize ) );
}

void CHipMathEngine::BatchMultiplyMatrixByDiagMatrix( int batchSize, const CConstFloatHandle& firstHandle, int height,
	int width, int firstMatrixOffset, const CConstFloatHandle& secondHandle, int secondMatrixOffset,
	const CFloatHandle& resultHandle, int resultBufferSize )
{
	NH_CALL( nhBatchMultiplyMatrixByDiagMatrix( stream, batchSize, raw( firstHandle ), height, width, firstMatrixOffset,
		raw( secondHandle ), secondMatrixOffset, raw( resultHandle ), resultBufferSize ) );
}

void CHipMathEngine::TransposeMatrix( int batchSize, const CConstFloatHandle& firstHandle, int height, int medium,
	int width, int channels, const CFloatHandle& resultHandle, int resultBufferSize )
{
	NH_CALL( nhTransposeMatrix( stream, batchSize, raw( firstHandle ), height, medium, width, channels,
		raw( resultHandle ), resultBufferSize ) );
}

void CHipMathEngine::TransposeMatrix( int batchSize, const CConstIntHandle& firstHandle, int height, int medium,
	int width, int channels, const CIntHandle& resultHandle, int resultBufferSize )
{
	NH_CALL( nhTransposeMatrixInt( stream, batchSize, raw( firstHandle ), height, medium, width, channels,
		raw( resultHandle ), resultBufferSize ) );
}

// ---------------------------------------------------------------------------------------------------------
// IDnnEngine

void CHipMathEngine::BlobMergeByDim( TBlobDim dim, const CBlobDesc* from, const CFloatHandle* fromData, int fromCount,
	const CBlobDesc& to, const CFloatHandle& toData )
{
	ASSERT_EXPR( dim < BD_Count && fromCount <= MaxBlobDescs );
	nhBlobDesc descs[MaxBlobDescs];
	const float* ptrs[MaxBlobDescs];
	for( int i = 0; i < fromCount; ++i ) {
		descs[i] = toBlobDesc( from[i] );
		ptrs[i] = raw( fromData[i] );
	}
	const nhBlobDesc toDesc = toBlobDesc( to );
	NH_CALL( nhBlobMergeByDim( stream, dim, descs, ptrs, fromCount, &toDesc, raw( toData ) ) );
}

void CHipMathEngine::BlobMergeByDim( TBlobDim dim, const CBlobDesc* from, const CIntHandle* fromData, int fromCount,
	const CBlobDesc& to, const CIntHandle& toData )
{
	// same bytes: 4-byte elements
	ASSERT_EXPR( dim < BD_Count && fromCount <= MaxBlobDescs );
	nhBlobDesc descs[MaxBlobDescs];
	const float* ptrs[MaxBlobDescs];
	for( int i = 0; i < fromCount; ++i ) {
		descs[i] = toBlobDesc( from[i] );
		ptrs[i] = reinterpret_cast<const float*>( raw( fromData[i] ) );
	}
	const nhBlobDesc toDesc = toBlobDesc( to );
	NH_CALL( nhBlobMergeByDim( stream, dim, descs, ptrs, fromCount, &toDesc, reinterpret_cast<float*>( raw( toData ) ) ) );
}

void CHipMathEngine::BlobSplitByDim( TBlobDim dim, const CBlobDesc& from, const CConstFloatHandle& fromData,
	const CBlobDesc* to, const CFloatHandle* toData, int toCount )
{
	ASSERT_EXPR( dim < BD_Count && toCount <= MaxBlobDescs );
	nhBlobDesc descs[MaxBlobDescs];
	float* ptrs[MaxBlobDescs];
	for( int i = 0; i < toCount; ++i ) {
		descs[i] = toBlobDesc( to[i] );
		ptrs[i] = raw( toData[i] );
	}
	const nhBlobDesc fromDesc = toBlobDesc( from );
	NH_CALL( nhBlobSplitByDim( stream, dim, &fromDesc, raw( fromData ), descs, ptrs, toCount ) );
}

void CHipMathEngine::BlobSplitByDim( TBlobDim dim, const CBlobDesc& from, const CConstIntHandle& fromData,
	const CBlobDesc* to, const CIntHandle* toData, int toCount )
{
	ASSERT_EXPR( dim < BD_Count && toCount <= MaxBlobDescs );
	nhBlobDesc descs[MaxBlobDescs];
	float* ptrs[MaxBlobDescs];
	for( int i = 0; i < toCount; ++i ) {
		descs[i] = toBlobDesc( to[i] );
		ptrs[i] = reinterpret_cast<float*>( raw( toData[i] ) );
	}
	const nhBlobDesc fromDesc = toBlobDesc( from );
	NH_CALL( nhBlobSplitByDim( stream, dim, &fromDesc, reinterpret_cast<const float*>( raw( fromData ) ), descs, ptrs, toCount ) );
}

void CHipMathEngine::BlobResizeImage( const CBlobDesc& from, const CFloatHandle& fromData, int deltaLeft, int deltaRight,
	int deltaTop, int deltaBottom, TBlobResizePadding padding, float defaultValue,
	const CBlobDesc& to, const CFloatHandle& toData )
{
	const nhBlobDesc fromDesc = toBlobDesc( from );
	const nhBlobDesc toDesc = toBlobDesc( to );
	const int mode = padding == TBlobResizePadding::Constant ? NH_PAD_CONSTANT
		: ( padding == TBlobResizePadding::Edge ? NH_PAD_EDGE : NH_PAD_REFLECT );
	NH_CALL( nhBlobResizeImage( stream, &fromDesc, raw( fromData ), deltaLeft, deltaRight, deltaTop, deltaBottom, mode,
		defaultValue, &toDesc, raw( toData ) ) );
}

CConvolutionDesc* CHipMathEngine::InitBlobConvolution( const CBlobDesc& input, int paddingHeight, int paddingWidth,
	int strideHeight, int strideWidth, int dilationHeight, int dilationWidth, const CBlobDesc& filter,
	const CBlobDesc& output )
{
	// the Depth dimension is folded into the channels, as in the reference (CpuMathEngineDnnConv.cpp:43-73)
	std::unique_ptr<CHipConvolutionDesc> desc( new CHipConvolutionDesc() );
	nhConvDesc& d = desc->D;
	d.batch = input.ObjectCount();
	d.height = input.Height();
	d.width = input.Width();
	d.channels = input.Depth() * input.Channels();
	d.filterCount = filter.ObjectCount();
	d.filterHeight = filter.Height();
	d.filterWidth = filter.Width();
	d.paddingHeight = paddingHeight;
	d.paddingWidth = paddingWidth;
	d.strideHeight = strideHeight;
	d.strideWidth = strideWidth;
	d.dilationHeight = dilationHeight;
	d.dilationWidth = dilationWidth;
	ASSERT_EXPR( filter.Depth() * filter.Channels() == d.channels );
	NH_CALL( nhInitBlobConvolution( &d ) );
	ASSERT_EXPR( output.Height() == d.resultHeight && output.Width() == d.resultWidth );
	ASSERT_EXPR( output.ObjectCount() == d.batch && output.Depth() * output.Channels() == d.filterCount );
	return desc.release();
}

void CHipMathEngine::BlobConvolution( const CConvolutionDesc& desc, const CConstFloatHandle& source,
	const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm, const CFloatHandle& result )
{
	const CHipConvolutionDesc& d = static_cast<const CHipConvolutionDesc&>( desc );
	NH_CALL( nhBlobConvolution( stream, &d.D, raw( source ), raw( filter ),
		freeTerm != nullptr ? raw( *freeTerm ) : nullptr, raw( result ) ) );
}

void CHipMathEngine::BlobConvolutionWithActivation( const CConvolutionDesc& desc, const CConstFloatHandle& source,
	const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm, int activation, float param,
	const CFloatHandle& result )
{
	const CHipConvolutionDesc& d = static_cast<const CHipConvolutionDesc&>( desc );
	NH_CALL( nhBlobConvolutionWithActivation( stream, &d.D, raw( source ), raw( filter ),
		freeTerm != nullptr ? raw( *freeTerm ) : nullptr, activation, param, raw( result ) ) );
}

void CHipMathEngine::BlobConvolutionBackward( const CConvolutionDesc& desc, const CConstFloatHandle& outputDiff,
	const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm, const CFloatHandle& inputDiff )
{
	const CHipConvolutionDesc& d = static_cast<const CHipConvolutionDesc&>( desc );
	size_t workspaceSize = 0;
	NH_CALL( nhBlobConvolutionBackwardWorkspaceSize( &d.D, &workspaceSize ) );
	const CMemoryHandle workspace = StackAlloc( std::max<size_t>( workspaceSize, 16 ) );
	NH_CALL( nhBlobConvolutionBackward( stream, &d.D, raw( outputDiff ), raw( filter ),
		freeTerm != nullptr ? raw( *freeTerm ) : nullptr, raw( inputDiff ), rawBytes( workspace ), workspaceSize ) );
	StackFree( workspace );
}

void CHipMathEngine::BlobConvolutionLearnAdd( const CConvolutionDesc& desc, const CConstFloatHandle& input,
	const CConstFloatHandle& outputDiff, const CFloatHandle& filterDiff, const CFloatHandle* freeTermDiff,
	bool isFreeTermDiffFromInput )
{
	const CHipConvolutionDesc& d = static_cast<const CHipConvolutionDesc&>( desc );
	NH_CALL( nhBlobConvolutionLearnAdd( stream, &d.D, raw( input ), raw( outputDiff ), raw( filterDiff ) ) );
	if( freeTermDiff != nullptr ) {
		// the free term's gradient is the sum of the pixels of outputDiff, channel by channel; the transposed
		// convolution asks for the same over the input instead (CpuMathEngineDnnConv.cpp:860-883)
		if( isFreeTermDiffFromInput ) {
			SumMatrixRowsAdd( 1, *freeTermDiff, input, d.D.batch * d.D.height * d.D.width, d.D.channels );
		} else {
			SumMatrixRowsAdd( 1, *freeTermDiff, outputDiff, d.D.batch * d.D.resultHeight * d.D.resultWidth,
				d.D.filterCount );
		}
	}
}

CChannelwiseConvolutionDesc* CHipMathEngine::InitBlobChannelwiseConvolution( const CBlobDesc& input, int paddingHeight,
	int paddingWidth, int strideHeight, int strideWidth, const CBlobDesc& filter, const CBlobDesc* freeTerm,
	const CBlobDesc& output )
{
	ASSERT_EXPR( input.Depth() == 1 && filter.ObjectCount() == 1 && filter.Channels() == input.Channels() );
	ASSERT_EXPR( freeTerm == nullptr || freeTerm->BlobSize() == filter.Channels() );
	std::unique_ptr<CHipChannelwiseConvolutionDesc> desc( new CHipChannelwiseConvolutionDesc() );
	nhConvDesc& d = desc->D;
	std::memset( &d, 0, sizeof( d ) );
	d.batch = input.ObjectCount();
	d.height = input.Height();
	d.width = input.Width();
	d.channels = input.Channels();
	d.filterHeight = filter.Height();
	d.filterWidth = filter.Width();
	d.paddingHeight = paddingHeight;
	d.paddingWidth = paddingWidth;
	d.strideHeight = strideHeight;
	d.strideWidth = strideWidth;
	NH_CALL( nhInitBlobChannelwiseConvolution( &d ) );
	ASSERT_EXPR( output.Height() == d.resultHeight && output.Width() == d.resultWidth );
	return desc.release();
}

void CHipMathEngine::BlobChannelwiseConvolution( const CChannelwiseConvolutionDesc& desc, const CConstFloatHandle& source,
	const CConstFloatHandle& filter, const CConstFloatHandle* freeTerm, const CFloatHandle& result )
{
	const CHipChannelwiseConvolutionDesc& d = static_cast<const CHipChannelwiseConvolutionDesc&>( desc );
	NH_CALL( nhBlobChannelwiseConvolution( stream, &d.D, raw( source ), raw( filter ),
		freeTerm != nullptr ? raw( *freeTerm ) : nullptr, raw( result ) ) );
}

static nhPoolingDesc makePoolingDesc( const CBlobDesc& source, int filterHeight, int filterWidth, int strideHeight,
	int strideWidth )
{
	nhPoolingDesc d;
	d.batch = source.ObjectCount();
	d.height = source.Height();
	d.width = source.Width();
	d.channels = source.Depth() * source.Channels();
	d.filterHeight = filterHeight;
	d.filterWidth = filterWidth;
	d.strideHeight = strideHeight;
	d.strideWidth = strideWidth;
	d.resultHeight = 0;
	d.resultWidth = 0;
	return d;
}

void CHipMathEngine::BlobChannelwiseConvolutionBackward( const CChannelwiseConvolutionDesc& desc,
	const CConstFloatHandle& source, const CConstFloatHandle& filter, const CFloatHandle& result )
{
	const CHipChannelwiseConvolutionDesc& d = static_cast<const CHipChannelwiseConvolutionDesc&>( desc );
	NH_CALL( nhBlobChannelwiseConvolutionBackward( stream, &d.D, raw( source ), raw( filter ), raw( result ) ) );
}

void CHipMathEngine::BlobChannelwiseConvolutionLearnAdd( const CChannelwiseConvolutionDesc& desc,
	const CConstFloatHandle& input, const CConstFloatHandle& outputDiff, const CFloatHandle& filterDiff,
	const CFloatHandle* freeTermDiff )
{
	const CHipChannelwiseConvolutionDesc& d = static_cast<const CHipChannelwiseConvolutionDesc&>( desc );
	NH_CALL( nhBlobChannelwiseConvolutionLearnAdd( stream, &d.D, raw( input ), raw( outputDiff ), raw( filterDiff ),
		freeTermDiff != nullptr ? raw( *freeTermDiff ) : nullptr ) );
}

CMaxPoolingDesc* CHipMathEngine::InitMaxPooling( const CBlobDesc& source, int filterHeight, int filterWidth,
	int strideHeight, int strideWidth, const CBlobDesc& result )
{
	std::unique_ptr<CHipMaxPoolingDesc> desc( new CHipMaxPoolingDesc() );
	desc->D = makePoolingDesc( source, filterHeight, filterWidth, strideHeight, strideWidth );
	NH_CALL( nhInitPooling( &desc->D ) );
	ASSERT_EXPR( result.Height() == desc->D.resultHeight && result.Width() == desc->D.resultWidth );
	return desc.release();
}

void CHipMathEngine::BlobMaxPooling( const CMaxPoolingDesc& desc, const CConstFloatHandle& source,
	const CIntHandle* maxIndices, const CFloatHandle& result )
{
	const CHipMaxPoolingDesc& d = static_cast<const CHipMaxPoolingDesc&>( desc );
	NH_CALL( nhBlobMaxPooling( stream, &d.D, raw( source ), maxIndices != nullptr ? raw( *maxIndices ) : nullptr,
		raw( result ) ) );
}

void CHipMathEngine::BlobMaxPoolingBackward( const CMaxPoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CConstIntHandle& maxIndices, const CFloatHandle& sourceDiff )
{
	const CHipMaxPoolingDesc& d = static_cast<const CHipMaxPoolingDesc&>( desc );
	NH_CALL( nhBlobMaxPoolingBackward( stream, &d.D, raw( resultDiff ), raw( maxIndices ), raw( sourceDiff ) ) );
}

CMeanPoolingDesc* CHipMathEngine::InitMeanPooling( const CBlobDesc& source, int filterHeight, int filterWidth,
	int strideHeight, int strideWidth, const CBlobDesc& result )
{
	std::unique_ptr<CHipMeanPoolingDesc> desc( new CHipMeanPoolingDesc() );
	desc->D = makePoolingDesc( source, filterHeight, filterWidth, strideHeight, strideWidth );
	NH_CALL( nhInitPooling( &desc->D ) );
	ASSERT_EXPR( result.Height() == desc->D.resultHeight && result.Width() == desc->D.resultWidth );
	return desc.release();
}

void CHipMathEngine::BlobMeanPooling( const CMeanPoolingDesc& desc, const CConstFloatHandle& source,
	const CFloatHandle& result )
{
	const CHipMeanPoolingDesc& d = static_cast<const CHipMeanPoolingDesc&>( desc );
	NH_CALL( nhBlobMeanPooling( stream, &d.D, raw( source ), raw( result ) ) );
}

void CHipMathEngine::BlobMeanPoolingBackward( const CMeanPoolingDesc& desc, const CConstFloatHandle& resultDiff,
	const CFloatHandle& sourceDiff )
{
	const CHipMeanPoolingDesc& d = static_cast<const CHipMeanPoolingDesc&>( desc );
	NH_CALL( nhBlobMeanPoolingBackward( stream, &d.D, raw( resultDiff ), raw( sourceDiff ) ) );
}

struct CHipDropoutDesc : public CDropoutDesc {
	nhBlobDesc Input;
	float Rate;
	bool IsSpatial, IsBatchwise;
	int Seed;
};

CDropoutDesc* CHipMathEngine::InitDropout( float rate, bool isSpatial, bool isBatchwise, const CBlobDesc& input,
	const CBlobDesc& output, int seed )
{
	ASSERT_EXPR( rate >= 0.f && rate < 1.f );
	ASSERT_EXPR( input.HasEqualDimensions( output ) );
	CHipDropoutDesc* desc = new CHipDropoutDesc();
	desc->Input = toBlobDesc( input );
	desc->Rate = rate;
	desc->IsSpatial = isSpatial;
	desc->IsBatchwise = isBatchwise;
	desc->Seed = seed;
	return desc;
}

void CHipMathEngine::Dropout( const CDropoutDesc& desc, const CFloatHandle& input, const CFloatHandle& output )
{
	const CHipDropoutDesc& d = static_cast<const CHipDropoutDesc&>( desc );
	NH_CALL( nhDropout( stream, &d.Input, d.Rate, d.IsSpatial ? 1 : 0, d.IsBatchwise ? 1 : 0, d.Seed, raw( input ),
		raw( output ) ) );
}

CLstmDesc* CHipMathEngine::InitLstm( int hiddenSize, int objectSize, const CConstFloatHandle& inputWeights,
	const CConstFloatHandle& inputFreeTerm, const CConstFloatHandle& recurrentWeights,
	const CConstFloatHandle& recurrentFreeTerm )
{
	CHipLstmDesc* desc = new CHipLstmDesc();
	desc->HiddenSize = hiddenSize;
	desc->ObjectSize = objectSize;
	desc->InputWeights = inputWeights;
	desc->InputFreeTerm = inputFreeTerm;
	desc->RecurrentWeights = recurrentWeights;
	desc->RecurrentFreeTerm = recurrentFreeTerm;
	desc->Engine = this;
	return desc;
}

void CHipMathEngine::Lstm( CLstmDesc& desc, bool reverse, int sequenceLength, int sequenceCount,
	const CConstFloatHandle& inputStateBackLink, const CConstFloatHandle& inputMainBackLink,
	const CConstFloatHandle& input, const CFloatHandle& outputStateBackLink, const CFloatHandle& outputMainBackLink )
{
	CHipLstmDesc& d = static_cast<CHipLstmDesc&>( desc );
	size_t workspaceSize = 0;
	NH_CALL( nhLstmWorkspaceSize( d.HiddenSize, d.ObjectSize, sequenceLength, sequenceCount, &workspaceSize ) );
	if( d.WorkspaceSize < workspaceSize ) {
		if( !d.Workspace.IsNull() ) {
			HeapFree( d.Workspace );
			d.Workspace = CMemoryHandle();
			d.WorkspaceSize = 0;
		}
		d.Workspace = HeapAlloc( workspaceSize );
		d.WorkspaceSize = workspaceSize;
	}
	const CMemoryHandle& workspace = d.Workspace;
	NH_CALL( nhLstm( stream, d.HiddenSize, d.ObjectSize, raw( d.InputWeights ),
		d.InputFreeTerm.IsNull() ? nullptr : raw( d.InputFreeTerm ), raw( d.RecurrentWeights ),
		d.RecurrentFreeTerm.IsNull() ? nullptr : raw( d.RecurrentFreeTerm ), reverse ? 1 : 0, sequenceLength,
		sequenceCount, inputStateBackLink.IsNull() ? nullptr : raw( inputStateBackLink ),
		inputMainBackLink.IsNull() ? nullptr : raw( inputMainBackLink ), raw( input ),
		outputStateBackLink.IsNull() ? nullptr : raw( outputStateBackLink ), raw( outputMainBackLink ),
		rawBytes( workspace ), workspaceSize ) );
}

// ---------------------------------------------------------------------------------------------------------
// IMathEngine

// The interface has no enumerator for this device family; layers branch on "not MET_Cpu" and one of them accepts
// only MET_Cpu or MET_Cuda, so the engine reports the generic GPU value.
TMathEngineType CHipMathEngine::GetType() const
{
	return MET_Cuda;
}

void CHipMathEngine::GetMathEngineInfo( CMathEngineInfo& info ) const
{
	info.Type = MET_Cuda;
	std::strncpy( info.Name, deviceName, sizeof( info.Name ) - 1 );
	info.Name[sizeof( info.Name ) - 1] = 0;
	info.AvailableMemory = memoryLimit != 0 && memoryLimit < deviceTotalMemory ? memoryLimit : deviceTotalMemory;
	info.Id = device;
}

bool CHipMathEngine::IsInitialized() const
{
	return initialized;
}

// Allocation from the device synchronises it, so blocks are always cached (the reference does the same for its
// GPU engine, src/MemoryEngineMixin.cpp:38-60)
void CHipMathEngine::SetReuseMemoryMode( bool )
{
}

bool CHipMathEngine::GetReuseMemoryMode() const
{
	return true;
}

void CHipMathEngine::SetThreadBufferMemoryThreshold( size_t threshold )
{
	NH_CALL( nhPoolSetThreadBufferMemoryThreshold( pool, threshold ) );
}

size_t CHipMathEngine::GetThreadBufferMemoryThreshold() const
{
	size_t threshold = 0;
	NH_CALL( nhPoolGetThreadBufferMemoryThreshold( pool, &threshold ) );
	return threshold;
}

CMemoryHandle CHipMathEngine::HeapAlloc( size_t count )
{
	void* ptr = nullptr;
	NH_CALL( nhPoolHeapAlloc( pool, count, &ptr ) );
	return CMemoryHandleInternal::Create( this, ptr );
}

void CHipMathEngine::HeapFree( const CMemoryHandle& handle )
{
	OWN( handle );
	NH_CALL( nhPoolHeapFree( pool, CMemoryHandleInternal::GetRaw( handle ) ) );
}

void CHipMathEngine::TransferHandleToThisThread( const CMemoryHandle& handle, size_t size )
{
	OWN( handle );
	NH_CALL( nhPoolTransferToThisThread( pool, CMemoryHandleInternal::GetRaw( handle ), size ) );
}

CMemoryHandle CHipMathEngine::StackAlloc( size_t count )
{
	void* ptr = nullptr;
	NH_CALL( nhPoolStackAlloc( pool, count, &ptr ) );
	return CMemoryHandleInternal::Create( this, ptr );
}

void CHipMathEngine::StackFree( const CMemoryHandle& handle )
{
	if( handle.IsNull() ) {
		return;
	}
	OWN( handle );
	NH_CALL( nhPoolStackFree( pool, CMemoryHandleInternal::GetRaw( handle ) ) );
}

size_t CHipMathEngine::GetFreeMemorySize() const
{
	size_t current = 0;
	NH_CALL( nhPoolGetCurrentMemoryUsage( pool, &current ) );
	size_t inPools = 0;
	NH_CALL( nhPoolGetMemoryInPools( pool, &inPools ) );
	const size_t limit = memoryLimit != 0 ? memoryLimit : deviceTotalMemory;
	const size_t used = current - inPools;
	return limit > used ? limit - used : 0;
}

size_t CHipMathEngine::GetPeakMemoryUsage() const
{
	size_t bytes = 0;
	NH_CALL( nhPoolGetPeakMemoryUsage( pool, &bytes ) );
	return bytes;
}

void CHipMathEngine::ResetPeakMemoryUsage()
{
	NH_CALL( nhPoolResetPeakMemoryUsage( pool ) );
}

size_t CHipMathEngine::GetCurrentMemoryUsage() const
{
	size_t bytes = 0;
	NH_CALL( nhPoolGetCurrentMemoryUsage( pool, &bytes ) );
	return bytes;
}

size_t CHipMathEngine::GetMemoryInPools() const
{
	size_t bytes = 0;
	NH_CALL( nhPoolGetMemoryInPools( pool, &bytes ) );
	return bytes;
}

void CHipMathEngine::CleanUp()
{
	// cached blocks may still be referenced by kernels in flight: drain the stream before they go back to the device
	NH_CALL( nhStreamSynchronize( stream ) );
	{
		std::lock_guard<std::mutex> lock( hostMutex );
		auto it = hostBuffers.find( std::this_thread::get_id() );
		if( it != hostBuffers.end() ) {
			CHostStack& stack = it->second;
			while( stack.Blocks.size() > stack.Depth ) {
				nhHostFree( stack.Blocks.back().Ptr );
				stack.Blocks.pop_back();
			}
			if( stack.Blocks.empty() ) {
				hostBuffers.erase( it );
			}
		}
	}
	CleanUpSpecial();
	// the scratch block the kernels keep for the stream came from the pool: back it goes, then the pool lets go
	NH_CALL( nhStreamReleaseScratch( stream ) );
	NH_CALL( nhPoolCleanUp( pool ) );
}

void CHipMathEngine::CleanUpSpecial()
{
}

// Host view of a piece of a blob: pinned staging memory, filled from the device when `exchange` is set.
// Strictly LIFO per thread, like the reference's host stack (src/MemoryEngineMixin.cpp:185-216); the bytes are read
// from handle + pos.
void* CHipMathEngine::GetBuffer( const CMemoryHandle& handle, size_t pos, size_t size, bool exchange )
{
	OWN( handle );
	constexpr size_t headerSize = 2 * sizeof( size_t );
	char* block = nullptr;
	{
		std::lock_guard<std::mutex> lock( hostMutex );
		CHostStack& stack = hostBuffers[std::this_thread::get_id()];
		const size_t need = size + headerSize;
		if( stack.Blocks.size() > stack.Depth && stack.Blocks[stack.Depth].Size < need ) {
			// the idle block at this depth is too small; the ones behind it are idle too
			while( stack.Blocks.size() > stack.Depth ) {
				nhHostFree( stack.Blocks.back().Ptr );
				stack.Blocks.pop_back();
			}
		}
		if( stack.Blocks.size() == stack.Depth ) {
			void* fresh = nullptr;
			NH_CALL( nhHostAlloc( &fresh, need ) );
			stack.Blocks.push_back( CHostBuffer{ static_cast<char*>( fresh ), need } );
		}
		block = stack.Blocks[stack.Depth].Ptr;
		++stack.Depth;
	}
	size_t* header = reinterpret_cast<size_t*>( block );
	header[0] = pos;
	header[1] = size;
	char* data = block + headerSize;
	if( exchange ) {
		NH_CALL( nhCopyDeviceToHost( stream, data, static_cast<char*>( CMemoryHandleInternal::GetRaw( handle ) ) + pos, size ) );
	}
	return data;
}

void CHipMathEngine::ReleaseBuffer( const CMemoryHandle& handle, void* ptr, bool exchange )
{
	OWN( handle );
	constexpr size_t headerSize = 2 * sizeof( size_t );
	char* block = static_cast<char*>( ptr ) - headerSize;
	{
		std::lock_guard<std::mutex> lock( hostMutex );
		CHostStack& stack = hostBuffers[std::this_thread::get_id()];
		ASSERT_EXPR( stack.Depth > 0 && stack.Blocks[stack.Depth - 1].Ptr == block );
	}
	if( exchange ) {
		// ( waits for the copy: the block may be handed out again right away )
		const size_t* header = reinterpret_cast<const size_t*>( block );
		NH_CALL( nhCopyHostToDevice( stream, static_cast<char*>( CMemoryHandleInternal::GetRaw( handle ) ) + header[0],
			ptr, header[1] ) );
	}
	std::lock_guard<std::mutex> lock( hostMutex );
	--hostBuffers[std::this_thread::get_id()].Depth;
}

void CHipMathEngine::DataExchangeRaw( const CMemoryHandle& result, const void* source, size_t size )
{
	OWN( result );
	NH_CALL( nhCopyHostToDevice( stream, CMemoryHandleInternal::GetRaw( result ), source, size ) );
}

void CHipMathEngine::DataExchangeRaw( void* result, const CMemoryHandle& source, size_t size )
{
	OWN( source );
	NH_CALL( nhCopyDeviceToHost( stream, result, CMemoryHandleInternal::GetRaw( source ), size ) );
}

// Creates a blob of this engine holding the bytes of a blob of another engine (staged through host memory)
CMemoryHandle CHipMathEngine::CopyFrom( const CMemoryHandle& handle, size_t size )
{
	const CMemoryHandle result = HeapAlloc( size );
	IMathEngine* other = handle.GetMathEngine();
	ASSERT_EXPR( other != nullptr );
	void* host = other->GetBuffer( handle, 0, size, true );
	NH_CALL( nhCopyHostToDevice( stream, CMemoryHandleInternal::GetRaw( result ), host, size ) );
	other->ReleaseBuffer( handle, host, false );
	return result;
}

IPerformanceCounters* CHipMathEngine::CreatePerformanceCounters( bool ) const
{
	return new CHipPerformanceCounters( *this );
}

// one engine, one device: nothing to exchange (IsDistributed() is false)
void CHipMathEngine::AllReduce( const CFloatHandle&, int )
{
}

void CHipMathEngine::Broadcast( const CFloatHandle&, int, int )
{
}

} // namespace NeoML

// ---------------------------------------------------------------------------------------------------------

extern "C" NeoML::IMathEngine* CreateHipMathEngine( int deviceIndex, size_t memoryLimit, int flags )
{
	try {
		int count = 0;
		if( nhGetDeviceCount( &count ) != NH_OK || deviceIndex < 0 || deviceIndex >= count ) {
			return nullptr;
		}
		std::unique_ptr<NeoML::CHipMathEngine> engine( new NeoML::CHipMathEngine( deviceIndex, memoryLimit, flags ) );
		if( !engine->IsInitialized() ) {
			return nullptr;
		}
		return engine.release();
	} catch( ... ) {
		return nullptr;
	}
}

extern "C" int GetHipMathEngineCount()
{
	int count = 0;
	return nhGetDeviceCount( &count ) == NH_OK ? count : 0;
}
