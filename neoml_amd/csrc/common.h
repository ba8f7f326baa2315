// Shared helpers for the gfx950 kernels: error reporting across the C ABI, launch-shape helpers,
// wavefront (64-lane) reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/neoml_hip.h"

namespace nh {

// Stores the message returned by nhGetLastError() for the calling thread.
void setLastError( const char* fmt, ... );

// Streams on which two one-launch LSTMs that do not depend on each other may run side by side ( nhStreamOverlapLstm,
// dnn_ops.hip ) need to know whether anything was enqueued between two nhLstm calls: every entry point turns its stream
// handle into a stream here, so here is where that is noted. Costs one relaxed load unless some stream's last launch is a
// one-launch LSTM that still waits for a partner ( lstmPartnersAwaited: between an nhLstm call and the next call on its
// stream ); only then are the device asked for and the lock taken.
extern int overlapLstmStreams;
extern int lstmPartnersAwaited;
void noteStreamUse( hipStream_t stream );

// Small element-wise calls that a stream has put aside ( nhStreamDeferSmallOps, vector_ops.hip ) run before anything else
// that is asked of the stream, so they too are caught here: tinyChainsPending counts the streams that hold some.
// flushTinyOps launches what the stream of the current device holds; flushAllTinyOps does so for every stream of every
// device ( before device memory is given back ). releaseTinyQueue: the stream is being destroyed.
extern int tinyChainsPending;
bool flushTinyOps( hipStream_t stream ); // true: something was launched
void flushAllTinyOps();
void releaseTinyQueue( hipStream_t stream );
// On such a stream a product A * B^T with a dense result may wait for the call behind it ( deferProduct: true, nothing
// launched ); an AddVectorToMatrixRows over that result in place then launches both as one ( fusePendingProduct: true,
// *rc is the launch's code ), any other call sends the product out first, through toStream.
bool deferProduct( nhStream s, const float* a, int lda, const float* b, int ldb, float* c, int ldc, int M, int N, int K );
bool fusePendingProduct( nhStream s, const float* matrix, float* result, int height, int width, const float* vector, int* rc );
// An element-wise call over a height x width matrix ( more than 262144 elements ) whose second operand is a vector spread
// over the rows or the columns joins the stream's chain of large calls of one count: matrix (+ or *) vector -> result.
// alone: the call's own launch, for when nothing joins it.
enum TTinySpread { TS_None = 0, TS_PerRow = 1, TS_PerColumn = 2 };
typedef void ( *CSpreadAlone )( hipStream_t stream, bool multiply, int spread, const float* matrix, const float* vector, float* result,
	int height, int width );
bool deferSpreadOp( nhStream s, bool multiply, int spread, const float* matrix, const float* vector, float* result, int height, int width,
	CSpreadAlone alone );
// The sums of a matrix's rows ( nhSumMatrixColumns ) wait for the element-wise calls in place over them: one launch
bool deferColumnSum( nhStream s, float* result, const float* matrix, int height, int width );
// An image blob padded with a constant ( nhBlobResizeImage ) that waits for the call behind it: a 3 x 3 max pooling over the
// padded blob ( CImageResizeLayer + CMaxPoolingLayer, the way a pooling layer without padding of its own gets its border )
// writes the padded blob and the pooled one in one pass over the image.
struct CPendingPadding {
	bool Pending = false;
	const float* From = nullptr;
	float* To = nullptr;
	long long Batch = 0;
	int Height = 0, Width = 0, Channels = 0, ToHeight = 0, ToWidth = 0, DeltaLeft = 0, DeltaTop = 0, Padding = 0;
	float DefaultValue = 0.f;
};
bool deferPadding( nhStream s, const CPendingPadding& padding );
bool fusePendingPadding( nhStream s, const nhPoolingDesc& d, const float* source, float* result, int* rc );
// ( dnn_ops.hip ) the padding by itself; the padding with the pooling over it, false if the pair is not one it takes
int launchPadding( hipStream_t stream, const CPendingPadding& padding );
bool launchPaddingWithPooling( hipStream_t stream, const CPendingPadding& padding, const nhPoolingDesc& d, float* result, int* rc );
// A batch of small dense row-major products that waits for the call behind it ( nhBatchMultiplyMatrixByMatrix followed by
// nhVectorMultiply over the whole result in place: one launch )
bool deferBatchedProduct( nhStream s, int batch, const float* first, int height, int width, const float* second, int secondWidth,
	float* result );
// The same for a convolution ( plain or channelwise, its descriptor checked by the caller ) and the VectorReLU over its
// result in place that follows it in most networks.
bool deferConvolution( nhStream s, bool channelwise, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result );
bool fusePendingConvolution( nhStream s, const float* first, float* result, long long count, int activation,
	const float* upperThreshold, int* rc );

inline hipStream_t toStream( nhStream s )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	if( __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0 ) {
		flushTinyOps( stream );
	}
	if( __atomic_load_n( &lstmPartnersAwaited, __ATOMIC_RELAXED ) != 0 ) {
		noteStreamUse( stream );
	}
	return stream;
}

// Frees the scratch blocks that sliced reductions keep for a stream of the current device ( gemm_mfma.hip ); the stream
// must have been drained. unbind: the stream is going away, its binding to a pool goes with the blocks.
void releaseSliceScratch( hipStream_t stream, bool unbind );

// Scratch of the stream for reductions that meet inside a launch ( gemm_mfma.hip ): `partialFloats` floats and one arrival
// counter that is zero between launches and must be left at zero. false: none to be had, take another way.
bool streamMeetingPlace( hipStream_t stream, size_t partialFloats, float** partials, unsigned** counter );

constexpr int WaveSize = 64;

inline int ceilDiv( long long a, long long b ) { return static_cast<int>( ( a + b - 1 ) / b ); }

inline bool isAligned16( const void* p ) { return ( reinterpret_cast<uintptr_t>( p ) & 15 ) == 0; }

} // namespace nh

// Argument check: the reference asserts, the C ABI returns NH_ERR_ARGUMENT.
#define NH_REQUIRE( expr ) \
	do { if( !( expr ) ) { nh::setLastError( "%s: requirement failed: %s", __func__, #expr ); return NH_ERR_ARGUMENT; } } while( 0 )

#define NH_HIP( call ) \
	do { hipError_t nhErr_ = ( call ); if( nhErr_ != hipSuccess ) { \
		nh::setLastError( "%s: %s failed: %s", __func__, #call, hipGetErrorString( nhErr_ ) ); return NH_ERR_HIP; } } while( 0 )

// After a kernel launch: report launch-configuration errors (asynchronous faults surface at the next sync).
#define NH_LAUNCH_CHECK() NH_HIP( hipGetLastError() )

#ifdef __HIPCC__
namespace nh {

// Wavefront reductions on the data-parallel-primitive path of the vector ALU: a DPP operand reads another lane's
// register as part of the arithmetic instruction itself, where a shuffle is a round trip through the LDS crossbar
// ( ds_bpermute + wait ) per step. Four shifts inside each row of 16 lanes ( a lane outside the row contributes the
// operation's identity ), then lane 15 of a row is broadcast into the following row, then lane 31 into the upper half:
// lane 63 holds the result of all 64 lanes, and a read of that lane hands it to every lane as a scalar.
// All 64 lanes must be active ( the callers reduce in wave-uniform control flow ).
constexpr int DppRowShr1 = 0x111, DppRowShr2 = 0x112, DppRowShr4 = 0x114, DppRowShr8 = 0x118;
constexpr int DppRowBcast15 = 0x142, DppRowBcast31 = 0x143;

template<int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dppMove( float identity, float v )
{
	return __uint_as_float( static_cast<unsigned>( __builtin_amdgcn_update_dpp( static_cast<int>( __float_as_uint( identity ) ),
		static_cast<int>( __float_as_uint( v ) ), CTRL, ROW_MASK, 0xF, false ) ) );
}

template<int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ int dppMove( int identity, int v )
{
	return __builtin_amdgcn_update_dpp( identity, v, CTRL, ROW_MASK, 0xF, false );
}

__device__ __forceinline__ float waveReduceSum( float v )
{
	v += dppMove<DppRowShr1>( 0.f, v );
	v += dppMove<DppRowShr2>( 0.f, v );
	v += dppMove<DppRowShr4>( 0.f, v );
	v += dppMove<DppRowShr8>( 0.f, v );
	v += dppMove<DppRowBcast15, 0xA>( 0.f, v );
	v += dppMove<DppRowBcast31, 0xC>( 0.f, v );
	return __uint_as_float( static_cast<unsigned>( __builtin_amdgcn_readlane( static_cast<int>( __float_as_uint( v ) ), 63 ) ) );
}

__device__ __forceinline__ float waveReduceMax( float v )
{
	const float lowest = -__builtin_inff();
	v = fmaxf( v, dppMove<DppRowShr1>( lowest, v ) );
	v = fmaxf( v, dppMove<DppRowShr2>( lowest, v ) );
	v = fmaxf( v, dppMove<DppRowShr4>( lowest, v ) );
	v = fmaxf( v, dppMove<DppRowShr8>( lowest, v ) );
	v = fmaxf( v, dppMove<DppRowBcast15, 0xA>( lowest, v ) );
	v = fmaxf( v, dppMove<DppRowBcast31, 0xC>( lowest, v ) );
	return __uint_as_float( static_cast<unsigned>( __builtin_amdgcn_readlane( static_cast<int>( __float_as_uint( v ) ), 63 ) ) );
}

// The largest value of the wavefront and the smallest index among the lanes that hold it. A lane without a candidate
// passes index 0x7fffffff, which loses against every real one.
__device__ __forceinline__ void waveReduceArgMax( float& best, int& bestIndex )
{
	auto take = [&]( float otherValue, int otherIndex ) {
		const bool better = otherIndex != 0x7fffffff
			&& ( bestIndex == 0x7fffffff || otherValue > best || ( otherValue == best && otherIndex < bestIndex ) );
		best = better ? otherValue : best;
		bestIndex = better ? otherIndex : bestIndex;
	};
	take( dppMove<DppRowShr1>( 0.f, best ), dppMove<DppRowShr1>( 0x7fffffff, bestIndex ) );
	take( dppMove<DppRowShr2>( 0.f, best ), dppMove<DppRowShr2>( 0x7fffffff, bestIndex ) );
	take( dppMove<DppRowShr4>( 0.f, best ), dppMove<DppRowShr4>( 0x7fffffff, bestIndex ) );
	take( dppMove<DppRowShr8>( 0.f, best ), dppMove<DppRowShr8>( 0x7fffffff, bestIndex ) );
	take( dppMove<DppRowBcast15, 0xA>( 0.f, best ), dppMove<DppRowBcast15, 0xA>( 0x7fffffff, bestIndex ) );
	take( dppMove<DppRowBcast31, 0xC>( 0.f, best ), dppMove<DppRowBcast31, 0xC>( 0x7fffffff, bestIndex ) );
	best = __uint_as_float( static_cast<unsigned>( __builtin_amdgcn_readlane( static_cast<int>( __float_as_uint( best ) ), 63 ) ) );
	bestIndex = __builtin_amdgcn_readlane( bestIndex, 63 );
}

// Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous range of tiles so that
// neighbouring tiles (which share rows of A and the halo of the image) meet in the same L2.
__device__ __forceinline__ int xcdSwizzle( int bid, int total )
{
	const int xcd = bid & 7;
	const int idx = bid >> 3;
	const int per = total >> 3;
	const int rem = total & 7;
	return xcd * per + ( xcd < rem ? xcd : rem ) + idx;
}

// Activation applied by a producing kernel before it stores: the fused blocks of the MobileNet family put ReLU
// (optionally clipped at Param > 0) or h-swish behind a convolution; any other type stores the value as it is
// (src/CPU/Rowwise/CpuRowwiseCommon.h:79-86).
struct CFusedActivation {
	int Type;    // NH_ACT_*
	float Param; // upper threshold of NH_ACT_RELU when above zero
	// where the threshold lives in device memory instead ( the engine's VectorReLU takes it there ): a kernel that is
	// handed one reads it once, through withParam, before it looks at Param
	const float* ParamPtr;
};

__device__ __forceinline__ CFusedActivation withParam( CFusedActivation a )
{
	if( a.ParamPtr != nullptr ) {
		a.Param = *a.ParamPtr;
		a.ParamPtr = nullptr;
	}
	return a;
}

__device__ __forceinline__ float applyActivation( float v, const CFusedActivation& a )
{
	if( a.Type == NH_ACT_RELU ) {
		v = v > 0.f ? v : 0.f; // NaN becomes 0, as in VectorReLU
		if( a.Param > 0.f ) {
			v = v < a.Param ? v : a.Param;
		}
	} else if( a.Type == NH_ACT_HSWISH ) {
		v = v <= -3.f ? 0.f : ( v >= 3.f ? v : v * ( v + 3.f ) * ( 1.f / 6.f ) );
	}
	return v;
}

// The same activation with its type fixed at compile time and the upper threshold of ReLU given as a value that is
// +infinity when there is none: what the epilogue of a matrix product applies to every element of a tile, after one
// decision per tile instead of one per element.
template<int TYPE>
__device__ __forceinline__ float applyActivationOf( float v, float reluTop )
{
	if constexpr( TYPE == NH_ACT_RELU ) {
		v = v > 0.f ? v : 0.f; // NaN becomes 0, as in VectorReLU
		v = v < reluTop ? v : reluTop;
	} else if constexpr( TYPE == NH_ACT_HSWISH ) {
		v = v <= -3.f ? 0.f : ( v >= 3.f ? v : v * ( v + 3.f ) * ( 1.f / 6.f ) );
	}
	return v;
}

// Operands are read with raw buffer loads: a 32-bit byte offset from a base held in scalar registers, and a range
// check done by the memory unit. An offset at or above BufferBytes reads as zero, which serves as the zero padding
// of the convolution and as the mask of tile rows / columns / k beyond the matrix, without a branch or a select.
typedef unsigned int u32x4 __attribute__( ( ext_vector_type( 4 ) ) );
constexpr unsigned BufferBytes = 0x80000000u;
constexpr unsigned OutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t makeBuffer( const float* p )
{
	return __builtin_amdgcn_make_buffer_rsrc( const_cast<float*>( p ), 0, BufferBytes, 0x00020000 );
}

__device__ __forceinline__ float bufferLoad1( __amdgpu_buffer_rsrc_t rsrc, unsigned offset )
{
	return __uint_as_float( __builtin_amdgcn_raw_buffer_load_b32( rsrc, offset, 0, 0 ) );
}

__device__ __forceinline__ float4 bufferLoad4( __amdgpu_buffer_rsrc_t rsrc, unsigned offset )
{
	const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128( rsrc, offset, 0, 0 );
	return make_float4( __uint_as_float( v.x ), __uint_as_float( v.y ), __uint_as_float( v.z ), __uint_as_float( v.w ) );
}

// Streaming variant: the line is marked for early replacement in the caches ( data that is read once ).
__device__ __forceinline__ float4 bufferLoad4Stream( __amdgpu_buffer_rsrc_t rsrc, unsigned offset )
{
	const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128( rsrc, offset, 0, 2 ); // aux bit 1: nt
	return make_float4( __uint_as_float( v.x ), __uint_as_float( v.y ), __uint_as_float( v.z ), __uint_as_float( v.w ) );
}

// Store through a buffer descriptor: an offset at or beyond the descriptor's size drops the store.
__device__ __forceinline__ void bufferStore4( __amdgpu_buffer_rsrc_t rsrc, unsigned offset, const float4& v )
{
	u32x4 u;
	u.x = __float_as_uint( v.x );
	u.y = __float_as_uint( v.y );
	u.z = __float_as_uint( v.z );
	u.w = __float_as_uint( v.w );
	__builtin_amdgcn_raw_buffer_store_b128( u, rsrc, offset, 0, 0 );
}

// The same with a second, wave-uniform byte offset that travels in a scalar register: what a loop adds per iteration
// costs no vector instruction. The range check looks at the per-lane offset, so OutOfRange still reads as zero.
__device__ __forceinline__ float4 bufferLoad4( __amdgpu_buffer_rsrc_t rsrc, unsigned offset, unsigned uniformOffset )
{
	const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128( rsrc, offset, uniformOffset, 0 );
	return make_float4( __uint_as_float( v.x ), __uint_as_float( v.y ), __uint_as_float( v.z ), __uint_as_float( v.w ) );
}

} // namespace nh
#endif
