// Bandwidth-bound blob kernels of IDnnEngine on channels-last images: depthwise (channelwise) convolution,
// 2-D max / mean pooling, image padding / cropping, split / merge along a blob dimension, and the LSTM
// recurrence (matrix products on the MFMA kernels + one fused gate kernel per step).
#include "common.h"
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>

namespace nh {

// matrix products defined in gemm_mfma.hip
struct CSliceMeeting;
int convImplicitGemm( hipStream_t stream, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act, const CSliceMeeting* fixedMeeting );
int launchDeferredConvolution( hipStream_t stream, bool channelwise, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act );
int matMulNT( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate );
int matMulNTFused( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC,
	const float* bias, bool accumulate, const CFusedActivation& act, const float* residual );

// ---------------------------------------------------------------------------------------------------------
// Channelwise convolution: out[n,ho,wo,c] = bias[c] + sum_{kh,kw} in[n, ho*s-p+kh, wo*s-p+kw, c] * filt[kh,kw,c]
// One thread owns VECW channels of WPT horizontally adjacent output pixels, so that the input columns shared
// by neighbouring windows are loaded once and the filter taps stay in registers.

template<int VECW> struct CChanVec;
template<> struct CChanVec<4> {
	typedef float4 Type;
	static __device__ __forceinline__ float4 load( const float* p ) { return *reinterpret_cast<const float4*>( p ); }
	static __device__ __forceinline__ void store( float* p, float4 v ) { *reinterpret_cast<float4*>( p ) = v; }
	static __device__ __forceinline__ float4 zero() { return make_float4( 0.f, 0.f, 0.f, 0.f ); }
	static __device__ __forceinline__ float4 fma( float4 a, float4 b, float4 c )
	{
		return make_float4( fmaf( a.x, b.x, c.x ), fmaf( a.y, b.y, c.y ), fmaf( a.z, b.z, c.z ), fmaf( a.w, b.w, c.w ) );
	}
	static __device__ __forceinline__ float4 mul( float4 a, float4 b ) { return make_float4( a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w ); }
	static __device__ __forceinline__ float4 activate( float4 v, const CFusedActivation& a )
	{
		return make_float4( applyActivation( v.x, a ), applyActivation( v.y, a ), applyActivation( v.z, a ), applyActivation( v.w, a ) );
	}
};
template<> struct CChanVec<1> {
	typedef float Type;
	static __device__ __forceinline__ float load( const float* p ) { return *p; }
	static __device__ __forceinline__ void store( float* p, float v ) { *p = v; }
	static __device__ __forceinline__ float zero() { return 0.f; }
	static __device__ __forceinline__ float fma( float a, float b, float c ) { return fmaf( a, b, c ); }
	static __device__ __forceinline__ float activate( float v, const CFusedActivation& a ) { return applyActivation( v, a ); }
};

template<int VECW, int WPT>
__global__ __launch_bounds__( 256 )
void channelwiseConvKernel( const nhConvDesc d, const float* source, const float* filter, const float* freeTerm,
	float* result, int wGroups, long long totalItems, const CFusedActivation actAsGiven )
{
	const CFusedActivation act = withParam( actAsGiven );
	typedef CChanVec<VECW> V;
	typedef typename V::Type T;
	const int cg = d.channels / VECW;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < totalItems; item += step ) {
		long long t = item;
		const int c = static_cast<int>( t % cg ) * VECW; t /= cg;
		const int wo0 = static_cast<int>( t % wGroups ) * WPT; t /= wGroups;
		const int ho = static_cast<int>( t % d.resultHeight ); t /= d.resultHeight;
		const long long n = t;

		T acc[WPT];
		const T bias = freeTerm != nullptr ? V::load( freeTerm + c ) : V::zero();
#pragma unroll
		for( int j = 0; j < WPT; ++j ) {
			acc[j] = bias;
		}
		const float* image = source + n * d.height * d.width * d.channels + c;
		const int hi0 = ho * d.strideHeight - d.paddingHeight;
		const int wi0 = wo0 * d.strideWidth - d.paddingWidth;
		for( int kh = 0; kh < d.filterHeight; ++kh ) {
			const int hi = hi0 + kh;
			if( hi < 0 || hi >= d.height ) {
				continue;
			}
			const float* row = image + static_cast<long long>( hi ) * d.width * d.channels;
			for( int kw = 0; kw < d.filterWidth; ++kw ) {
				const T f = V::load( filter + ( kh * d.filterWidth + kw ) * d.channels + c );
#pragma unroll
				for( int j = 0; j < WPT; ++j ) {
					const int wi = wi0 + j * d.strideWidth + kw;
					if( wi >= 0 && wi < d.width && wo0 + j < d.resultWidth ) {
						acc[j] = V::fma( V::load( row + static_cast<long long>( wi ) * d.channels ), f, acc[j] );
					}
				}
			}
		}
		float* out = result + ( ( n * d.resultHeight + ho ) * d.resultWidth + wo0 ) * d.channels + c;
#pragma unroll
		for( int j = 0; j < WPT; ++j ) {
			if( wo0 + j < d.resultWidth ) {
				V::store( out + static_cast<long long>( j ) * d.channels, V::activate( acc[j], act ) );
			}
		}
	}
}

// The 3x3 case of the depthwise convolution (every depthwise layer of the MobileNet family), 4 channels per thread.
// One thread owns a strip WPT output pixels wide and rowsPerItem output rows tall and slides down it with the
// input rows of the window in registers: every input row is loaded once per strip instead of once per output row
// that touches it, and the index arithmetic is paid once per strip. The registers form a ring of 3 + PRE * STRIDE
// rows: the rows that enter the window for the output row PRE steps ahead are requested before the current row is
// computed and stored, so a thread always has PRE rows' worth of loads in flight ( the ring turns by renaming: the
// row loop is unrolled by the ring size, no register is moved ). Loads are raw buffer loads, so the zero padding is an
// out-of-range offset instead of a branch. Workgroups of one XCD cover a contiguous range of strips: the halo columns
// shared by neighbouring strips meet in that XCD's L2.
// STREAM: loads carry the streaming hint ( tensors far larger than the caches, every line used by one strip ).
// The row loop has no branch: rows below the strip and columns beyond the image get out-of-range offsets, for the
// loads ( zeros ) and for the stores ( dropped: the result is written through a buffer descriptor ), and the activation's
// type ( ACT ) is fixed when the kernel is compiled. With a branch per output pixel in the loop ( is the row inside? the
// column? which activation? ) the compiler no longer knew how many loads and stores were in flight at the top of the
// loop and waited for all of them, stores included, once per turn of the ring: every few rows each wave stood still
// for a whole memory round trip ( layers that fit the caches: 14 x 14 x 384 17.4 -> 13.8 us, 7 x 7 x 960 10.6 -> 8.7 us ).
// On inputs that come from memory ( measured with launches that rotate through 1.2 GB of input / output pairs, as
// inside a network: 112 x 112 x 32 90 us = 4.6 TB/s, 56 x 56 x 144 113 us = 4.1 TB/s, against 68 and 84 us on repeated
// buffers ) neither a second row of loads in flight ( PRE = 2: 88 / 106 us ) nor stores with the streaming hint ( 85 /
// 106 us, and 83 / 104 us on repeated buffers ) change the picture: not a matter of loads in flight.
template<int STRIDE, int WPT, int PRE, bool STREAM, int ACT>
__global__ __launch_bounds__( 256 )
void channelwiseConv3x3Kernel( const nhConvDesc d, const float* source, const float* filter, const float* freeTerm,
	float* result, int wGroups, int rowChunks, int rowsPerItem, int totalItems, const CFusedActivation actAsGiven, int flipTaps,
	unsigned resultBytes )
{
	const CFusedActivation act = withParam( actAsGiven );
	constexpr int NC = ( WPT - 1 ) * STRIDE + 3;
	constexpr int Ring = 3 + PRE * STRIDE;
	const int item = xcdSwizzle( blockIdx.x, gridDim.x ) * blockDim.x + threadIdx.x;
	if( item >= totalItems ) {
		return;
	}
	const int cg = d.channels / 4;
	int t = item;
	const int c = ( t % cg ) * 4; t /= cg;
	const int wo0 = ( t % wGroups ) * WPT; t /= wGroups;
	const int ho0 = ( t % rowChunks ) * rowsPerItem;
	const int n = t / rowChunks;
	const int hoEnd = min( ho0 + rowsPerItem, d.resultHeight );

	const __amdgpu_buffer_rsrc_t image = makeBuffer( source );
	const unsigned rowBytes = static_cast<unsigned>( d.width ) * d.channels * 4;
	const unsigned imageBytes = n * d.height * rowBytes;
	unsigned colOff[NC];
	const int wi0 = wo0 * STRIDE - d.paddingWidth;
#pragma unroll
	for( int j = 0; j < NC; ++j ) {
		const int wi = wi0 + j;
		colOff[j] = wi >= 0 && wi < d.width ? static_cast<unsigned>( wi * d.channels + c ) * 4 : OutOfRange;
	}
	float4 f[9];
#pragma unroll
	for( int k = 0; k < 9; ++k ) {
		// flipTaps: the filter turned by 180 degrees, which makes this kernel the gradient by the input of the stride-1 case
		f[k] = *reinterpret_cast<const float4*>( filter + ( flipTaps != 0 ? 8 - k : k ) * d.channels + c );
	}
	const float4 bias = freeTerm != nullptr ? *reinterpret_cast<const float4*>( freeTerm + c ) : make_float4( 0.f, 0.f, 0.f, 0.f );

	// input row hi of the strip lives in ring[ ( hi - hiFirst ) % Ring ]
	float4 ring[Ring][NC];
	const int hiFirst = ho0 * STRIDE - d.paddingHeight;
	const int hiLast = ( hoEnd - 1 ) * STRIDE - d.paddingHeight + 2; // last input row any output row of the strip needs
	auto loadRow = [&]( float4* row, int hi ) {
		const bool valid = hi >= 0 && hi < d.height && hi <= hiLast;
		const unsigned rowOff = imageBytes + static_cast<unsigned>( hi ) * rowBytes;
#pragma unroll
		for( int j = 0; j < NC; ++j ) {
			// a valid row offset is below 2 GiB, so adding an out-of-range column stays out of range
			const unsigned offset = valid ? rowOff + colOff[j] : OutOfRange;
			row[j] = STREAM ? bufferLoad4Stream( image, offset ) : bufferLoad4( image, offset );
		}
	};
#pragma unroll
	for( int r = 0; r < Ring - STRIDE; ++r ) {
		loadRow( ring[r], hiFirst + r );
	}
	const __amdgpu_buffer_rsrc_t outBuffer = __builtin_amdgcn_make_buffer_rsrc( result, 0, resultBytes, 0x00020000 );
	const unsigned outRowBytes = static_cast<unsigned>( d.resultWidth ) * d.channels * 4;
	unsigned outCol[WPT];
#pragma unroll
	for( int j = 0; j < WPT; ++j ) {
		outCol[j] = wo0 + j < d.resultWidth ? static_cast<unsigned>( ( wo0 + j ) * d.channels + c ) * 4 : OutOfRange;
	}
	unsigned outRowOffset = static_cast<unsigned>( n * d.resultHeight + ho0 ) * outRowBytes;
	const float reluTop = act.Param > 0.f ? act.Param : __builtin_inff();
	for( int hoBase = ho0; hoBase < hoEnd; hoBase += Ring ) {
#pragma unroll
		for( int k = 0; k < Ring; ++k ) {
			// output row hoBase + k: its window starts at ring position ( k * STRIDE ) % Ring ( Ring output rows
			// advance the window by Ring * STRIDE rows: a whole number of turns ); the rows PRE steps ahead go in
			// behind the ones already there. Behind the strip's last row nothing is fetched and nothing stored.
#pragma unroll
			for( int r = 0; r < STRIDE; ++r ) {
				const int ahead = k * STRIDE + Ring - STRIDE + r;
				loadRow( ring[ahead % Ring], hiFirst + ( hoBase - ho0 ) * STRIDE + ahead );
			}
			const bool rowInside = hoBase + k < hoEnd;
#pragma unroll
			for( int j = 0; j < WPT; ++j ) {
				float4 acc = bias;
#pragma unroll
				for( int kh = 0; kh < 3; ++kh ) {
#pragma unroll
					for( int kw = 0; kw < 3; ++kw ) {
						acc = CChanVec<4>::fma( ring[( k * STRIDE + kh ) % Ring][j * STRIDE + kw], f[kh * 3 + kw], acc );
					}
				}
				acc.x = applyActivationOf<ACT>( acc.x, reluTop );
				acc.y = applyActivationOf<ACT>( acc.y, reluTop );
				acc.z = applyActivationOf<ACT>( acc.z, reluTop );
				acc.w = applyActivationOf<ACT>( acc.w, reluTop );
				// ( a valid row offset is below 2 GiB, so adding an out-of-range column stays out of range )
				bufferStore4( outBuffer, rowInside ? outRowOffset + outCol[j] : OutOfRange, acc );
			}
			outRowOffset += outRowBytes;
		}
	}
}

// ---------------------------------------------------------------------------------------------------------
// Pooling: one thread owns VECW channels of one output column and walks down rowsPerItem output rows of it.
// Workgroups of one XCD cover a contiguous range of the image, so the input rows that overlapping windows
// share are fetched into one L2 only.

// FILTER > 0: the window is FILTER x FILTER and its loops unroll, so all loads of a window are in flight together.
template<int VECW, bool MEAN, int FILTER>
__global__ __launch_bounds__( 256 )
void poolingKernel( const nhPoolingDesc d, const float* source, float* result, int rowChunks, int rowsPerItem, long long totalItems )
{
	const int filterHeight = FILTER > 0 ? FILTER : d.filterHeight;
	const int filterWidth = FILTER > 0 ? FILTER : d.filterWidth;
	const int cg = d.channels / VECW;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	// ( 1 / fh ) / fw as the reference computes it (src/CPU/CpuMathEngineDnnPooling.h:68-69)
	const float scale = 1.f / d.filterHeight / d.filterWidth;
	const long long inRow = static_cast<long long>( d.width ) * d.channels;
	const long long outRow = static_cast<long long>( d.resultWidth ) * d.channels;
	for( long long item = xcdSwizzle( blockIdx.x, gridDim.x ) * 256LL + threadIdx.x; item < totalItems; item += step ) {
		long long t = item;
		const int c = static_cast<int>( t % cg ) * VECW; t /= cg;
		const int wo = static_cast<int>( t % d.resultWidth ); t /= d.resultWidth;
		const int ho0 = static_cast<int>( t % rowChunks ) * rowsPerItem; t /= rowChunks;
		const long long n = t;
		const int hoEnd = min( ho0 + rowsPerItem, d.resultHeight );
		const float* window = source + ( ( n * d.height + ho0 * d.strideHeight ) * d.width + wo * d.strideWidth ) * d.channels + c;
		float* out = result + ( ( n * d.resultHeight + ho0 ) * d.resultWidth + wo ) * d.channels + c;
		for( int ho = ho0; ho < hoEnd; ++ho ) {
			float acc[VECW];
			// columns outside, rows inside: the reference reduces over the rows of each column first
#pragma unroll
			for( int kw = 0; kw < filterWidth; ++kw ) {
				float col[VECW];
#pragma unroll
				for( int kh = 0; kh < filterHeight; ++kh ) {
					const float* p = window + kh * inRow + kw * d.channels;
					float v[VECW];
					if constexpr( VECW == 4 ) {
						const float4 q = *reinterpret_cast<const float4*>( p );
						v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
					} else {
						v[0] = *p;
					}
#pragma unroll
					for( int e = 0; e < VECW; ++e ) {
						if( kh == 0 ) {
							col[e] = v[e];
						} else if( MEAN ) {
							col[e] += v[e];
						} else if( v[e] > col[e] ) {
							col[e] = v[e];
						}
					}
				}
#pragma unroll
				for( int e = 0; e < VECW; ++e ) {
					if( kw == 0 ) {
						acc[e] = col[e];
					} else if( MEAN ) {
						acc[e] += col[e];
					} else if( col[e] > acc[e] ) {
						acc[e] = col[e];
					}
				}
			}
			if constexpr( VECW == 4 ) {
				float4 q;
				q.x = MEAN ? acc[0] * scale : acc[0];
				q.y = MEAN ? acc[1] * scale : acc[1];
				q.z = MEAN ? acc[2] * scale : acc[2];
				q.w = MEAN ? acc[3] * scale : acc[3];
				*reinterpret_cast<float4*>( out ) = q;
			} else {
				*out = MEAN ? acc[0] * scale : acc[0];
			}
			window += d.strideHeight * inRow;
			out += outRow;
		}
	}
}

// An image padded with a constant and the 3 x 3 max pooling over the padded image, one launch: the thread of poolingKernel
// ( four channels of one output column, a few output rows down ) takes its nine taps from the image itself, the constant
// where a tap lies in the border, and also writes the pixels of the padded image that are its own: the rows and columns
// from the first of its window up to the first of the next window ( up to the edge for the last window of a row or column ),
// so every padded pixel is written once. The padded image is not read back: 470 MB move where the two launches moved 683 MB
// ( 64 x 112 x 112 x 64 padded by one pixel, pooled with stride 2 ). Strides of at most 3, so that the pixels a thread
// owns lie in its window ( the few beyond it, at the far edges, are fetched on their own ). The maxima are taken in
// poolingKernel's order ( rows of a column first ), with the same comparisons. A thread walks down a few output rows and
// keeps the rows that a window shares with the one above it in registers ( 97.6 -> 88.8 us on that shape ).
struct CPadPoolArgs {
	const float* From;
	float* Padded;
	float* Result;
	int Height, Width, Channels, ToHeight, ToWidth, DeltaTop, DeltaLeft;
	float DefaultValue;
	int StrideHeight, StrideWidth, ResultHeight, ResultWidth, RowChunks, RowsPerItem;
	long long TotalItems;
};

__device__ __forceinline__ float4 paddedPixel( const CPadPoolArgs& a, const float* image, int py, int px )
{
	const int sy = py - a.DeltaTop, sx = px - a.DeltaLeft;
	if( sy >= 0 && sy < a.Height && sx >= 0 && sx < a.Width ) {
		return *reinterpret_cast<const float4*>( image + ( static_cast<long long>( sy ) * a.Width + sx ) * a.Channels );
	}
	return make_float4( a.DefaultValue, a.DefaultValue, a.DefaultValue, a.DefaultValue );
}

__global__ __launch_bounds__( 256 )
void padMaxPool3x3Kernel( const CPadPoolArgs a )
{
	const int cg = a.Channels / 4;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	for( long long item = xcdSwizzle( blockIdx.x, gridDim.x ) * 256LL + threadIdx.x; item < a.TotalItems; item += step ) {
		long long t = item;
		const int c = static_cast<int>( t % cg ) * 4; t /= cg;
		const int wo = static_cast<int>( t % a.ResultWidth ); t /= a.ResultWidth;
		const int ho0 = static_cast<int>( t % a.RowChunks ) * a.RowsPerItem; t /= a.RowChunks;
		const long long n = t;
		const int hoEnd = min( ho0 + a.RowsPerItem, a.ResultHeight );
		const float* image = a.From + n * a.Height * a.Width * a.Channels + c;
		float* padded = a.Padded + n * a.ToHeight * a.ToWidth * a.Channels + c;
		float* out = a.Result + ( ( n * a.ResultHeight + ho0 ) * a.ResultWidth + wo ) * a.Channels + c;
		const int px0 = wo * a.StrideWidth;
		const int columnsOwned = ( wo == a.ResultWidth - 1 ? a.ToWidth : px0 + a.StrideWidth ) - px0;
		float4 taps[3][3];
		for( int ho = ho0; ho < hoEnd; ++ho ) {
			const int py0 = ho * a.StrideHeight;
			const int rowsOwned = ( ho == a.ResultHeight - 1 ? a.ToHeight : py0 + a.StrideHeight ) - py0;
			// ( the rows that this window shares with the one above it are still in registers )
			const int kept = ho > ho0 ? 3 - a.StrideHeight : 0;
			if( kept == 2 ) {
#pragma unroll
				for( int kw = 0; kw < 3; ++kw ) {
					taps[0][kw] = taps[1][kw];
					taps[1][kw] = taps[2][kw];
				}
			} else if( kept == 1 ) {
#pragma unroll
				for( int kw = 0; kw < 3; ++kw ) {
					taps[0][kw] = taps[2][kw];
				}
			}
#pragma unroll
			for( int kh = 0; kh < 3; ++kh ) {
				if( kh >= kept ) {
#pragma unroll
					for( int kw = 0; kw < 3; ++kw ) {
						taps[kh][kw] = paddedPixel( a, image, py0 + kh, px0 + kw );
					}
				}
			}
			float acc[4];
#pragma unroll
			for( int kw = 0; kw < 3; ++kw ) {
				float col[4];
#pragma unroll
				for( int kh = 0; kh < 3; ++kh ) {
					const float v[4] = { taps[kh][kw].x, taps[kh][kw].y, taps[kh][kw].z, taps[kh][kw].w };
#pragma unroll
					for( int e = 0; e < 4; ++e ) {
						if( kh == 0 ) {
							col[e] = v[e];
						} else if( v[e] > col[e] ) {
							col[e] = v[e];
						}
					}
				}
#pragma unroll
				for( int e = 0; e < 4; ++e ) {
					if( kw == 0 ) {
						acc[e] = col[e];
					} else if( col[e] > acc[e] ) {
						acc[e] = col[e];
					}
				}
			}
			*reinterpret_cast<float4*>( out ) = make_float4( acc[0], acc[1], acc[2], acc[3] );
			out += static_cast<long long>( a.ResultWidth ) * a.Channels;
			// the thread's own pixels of the padded image: from its window where they lie in it
#pragma unroll
			for( int dy = 0; dy < 3; ++dy ) {
#pragma unroll
				for( int dx = 0; dx < 3; ++dx ) {
					if( dy < rowsOwned && dx < columnsOwned ) {
						*reinterpret_cast<float4*>( padded + ( static_cast<long long>( py0 + dy ) * a.ToWidth + px0 + dx ) * a.Channels ) = taps[dy][dx];
					}
				}
			}
			if( rowsOwned > 3 || columnsOwned > 3 ) {
				for( int dy = 0; dy < rowsOwned; ++dy ) {
					for( int dx = 0; dx < columnsOwned; ++dx ) {
						if( dy >= 3 || dx >= 3 ) {
							*reinterpret_cast<float4*>( padded + ( static_cast<long long>( py0 + dy ) * a.ToWidth + px0 + dx ) * a.Channels )
								= paddedPixel( a, image, py0 + dy, px0 + dx );
						}
					}
				}
			}
		}
	}
}

// Max pooling with the index output used by the backward pass. The index reproduces the reference CPU engine
// (src/CPU/CpuMathEngineDnnPooling.cpp:40-84) exactly:
//   - column maxima over the window rows keep the topmost row on ties (strict >);
//   - the window maximum over those column maxima keeps the leftmost column on ties (strict >);
//   - the row stored for the winning column is looked up in the row-index buffer at the column's position
//     RELATIVE to the window ( columnIndex * channels + c ), i.e. it is the arg-max row of image column
//     `columnIndex` of the same strip, not of column `wo * stride + columnIndex`.
// VECW channels per thread ( 4: 128-bit loads and stores when the channel count allows ).
template<int VECW>
__global__ __launch_bounds__( 256 )
void maxPoolingIndexKernel( const nhPoolingDesc d, const float* source, int* maxIndices, float* result, long long total )
{
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	const int rowSize = d.width * d.channels;
	const int channelGroups = d.channels / VECW;
	auto load = []( const float* p, float ( &v )[VECW] ) {
		if( VECW == 4 ) {
			const float4 q = *reinterpret_cast<const float4*>( p );
			v[0] = q.x; v[1 % VECW] = q.y; v[2 % VECW] = q.z; v[3 % VECW] = q.w;
		} else {
			v[0] = *p;
		}
	};
	const bool narrow = total <= 0x7fffffffLL; // ( 32-bit divisions where the count allows it )
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < total; item += step ) {
		int c, wo, ho;
		long long n;
		if( narrow ) {
			unsigned t = static_cast<unsigned>( item );
			c = static_cast<int>( t % static_cast<unsigned>( channelGroups ) ) * VECW; t /= static_cast<unsigned>( channelGroups );
			wo = static_cast<int>( t % static_cast<unsigned>( d.resultWidth ) ); t /= static_cast<unsigned>( d.resultWidth );
			ho = static_cast<int>( t % static_cast<unsigned>( d.resultHeight ) ); t /= static_cast<unsigned>( d.resultHeight );
			n = t;
		} else {
			long long t = item;
			c = static_cast<int>( t % channelGroups ) * VECW; t /= channelGroups;
			wo = static_cast<int>( t % d.resultWidth ); t /= d.resultWidth;
			ho = static_cast<int>( t % d.resultHeight ); t /= d.resultHeight;
			n = t;
		}
		const int stripRow = ho * d.strideHeight;
		const float* strip = source + ( n * d.height + stripRow ) * rowSize;
		const int windowColumn = wo * d.strideWidth * d.channels;
		float best[VECW];
		int bestCol[VECW];
		for( int kw = 0; kw < d.filterWidth; ++kw ) {
			const float* p = strip + windowColumn + kw * d.channels + c;
			float col[VECW];
			load( p, col );
			for( int kh = 1; kh < d.filterHeight; ++kh ) {
				float v[VECW];
				load( p + static_cast<long long>( kh ) * rowSize, v );
#pragma unroll
				for( int e = 0; e < VECW; ++e ) {
					if( v[e] > col[e] ) {
						col[e] = v[e];
					}
				}
			}
#pragma unroll
			for( int e = 0; e < VECW; ++e ) {
				if( kw == 0 || col[e] > best[e] ) {
					best[e] = col[e];
					bestCol[e] = kw;
				}
			}
		}
		int index[VECW];
#pragma unroll
		for( int e = 0; e < VECW; ++e ) {
			const int windowIndex = bestCol[e] * d.channels + c + e;
			const float* q = strip + windowIndex;
			float rowBest = *q;
			int rowIdx = 0;
			for( int kh = 1; kh < d.filterHeight; ++kh ) {
				const float v = q[static_cast<long long>( kh ) * rowSize];
				if( v > rowBest ) {
					rowBest = v;
					rowIdx = kh;
				}
			}
			index[e] = ( stripRow + rowIdx ) * rowSize + windowColumn + windowIndex;
		}
		const long long out = item * VECW;
		if( VECW == 4 ) {
			*reinterpret_cast<float4*>( result + out ) = make_float4( best[0], best[1 % VECW], best[2 % VECW], best[3 % VECW] );
			*reinterpret_cast<int4*>( maxIndices + out ) = make_int4( index[0], index[1 % VECW], index[2 % VECW], index[3 % VECW] );
		} else {
			result[out] = best[0];
			maxIndices[out] = index[0];
		}
	}
}

// The same for a square window of FILTER x FILTER and 4 channels per thread: the window's loads and the loads of the
// row-index lookup ( image columns 0 .. FILTER - 1 of the strip, whatever the window's column ) all go out together, and
// the lookup's answer is picked by the winning column afterwards. Same comparisons in the same order as above.
template<int FILTER>
__global__ __launch_bounds__( 256 )
void maxPoolingIndexSquareKernel( const nhPoolingDesc d, const float* source, int* maxIndices, float* result, int total )
{
	const int rowSize = d.width * d.channels;
	const unsigned channelGroups = static_cast<unsigned>( d.channels / 4 );
	for( int item = xcdSwizzle( blockIdx.x, gridDim.x ) * 256 + threadIdx.x; item < total; item += gridDim.x * 256 ) {
		unsigned t = static_cast<unsigned>( item );
		const int c = static_cast<int>( t % channelGroups ) * 4; t /= channelGroups;
		const int wo = static_cast<int>( t % static_cast<unsigned>( d.resultWidth ) ); t /= static_cast<unsigned>( d.resultWidth );
		const int ho = static_cast<int>( t % static_cast<unsigned>( d.resultHeight ) );
		const long long n = t / static_cast<unsigned>( d.resultHeight );
		const int stripRow = ho * d.strideHeight;
		const float* strip = source + ( n * d.height + stripRow ) * rowSize;
		const int windowColumn = wo * d.strideWidth * d.channels;
		float4 window[FILTER][FILTER], lookup[FILTER][FILTER]; // [kh][kw]
#pragma unroll
		for( int kh = 0; kh < FILTER; ++kh ) {
#pragma unroll
			for( int kw = 0; kw < FILTER; ++kw ) {
				window[kh][kw] = *reinterpret_cast<const float4*>( strip + static_cast<long long>( kh ) * rowSize + windowColumn + kw * d.channels + c );
				lookup[kh][kw] = *reinterpret_cast<const float4*>( strip + static_cast<long long>( kh ) * rowSize + kw * d.channels + c );
			}
		}
		float best[4];
		int index[4];
#pragma unroll
		for( int e = 0; e < 4; ++e ) {
			auto lane = [e]( const float4& v ) { return e == 0 ? v.x : ( e == 1 ? v.y : ( e == 2 ? v.z : v.w ) ); };
			int bestCol = 0;
#pragma unroll
			for( int kw = 0; kw < FILTER; ++kw ) {
				float col = lane( window[0][kw] );
#pragma unroll
				for( int kh = 1; kh < FILTER; ++kh ) {
					const float v = lane( window[kh][kw] );
					if( v > col ) {
						col = v;
					}
				}
				if( kw == 0 || col > best[e] ) {
					best[e] = col;
					bestCol = kw;
				}
			}
			int rowIdx = 0;
#pragma unroll
			for( int kw = 0; kw < FILTER; ++kw ) {
				float rowBest = lane( lookup[0][kw] );
				int idx = 0;
#pragma unroll
				for( int kh = 1; kh < FILTER; ++kh ) {
					const float v = lane( lookup[kh][kw] );
					if( v > rowBest ) {
						rowBest = v;
						idx = kh;
					}
				}
				rowIdx = bestCol == kw ? idx : rowIdx;
			}
			index[e] = ( stripRow + rowIdx ) * rowSize + windowColumn + bestCol * d.channels + c + e;
		}
		const long long out = static_cast<long long>( item ) * 4;
		*reinterpret_cast<float4*>( result + out ) = make_float4( best[0], best[1], best[2], best[3] );
		*reinterpret_cast<int4*>( maxIndices + out ) = make_int4( index[0], index[1], index[2], index[3] );
	}
}

// ---------------------------------------------------------------------------------------------------------
// BlobResizeImage: pad (constant / edge / reflect) or crop the H and W dimensions

__device__ __forceinline__ int resizeInputCoord( int x, int size, int padding )
{
	if( x >= 0 && x < size ) {
		return x;
	}
	if( padding == NH_PAD_CONSTANT ) {
		return -1;
	}
	if( padding == NH_PAD_EDGE ) {
		return x < 0 ? 0 : size - 1;
	}
	// reflect, with the reference's arithmetic (src/CPU/Rowwise/CpuRowwiseResizeImage.h:177-195)
	return x < 0 ? -( x % size ) : ( 2 * size - 2 - ( x % size ) ) % size;
}

template<int VECW>
__global__ __launch_bounds__( 256 )
void resizeImageKernel( const float* from, float* to, int height, int width, int channels, int toHeight, int toWidth,
	int deltaLeft, int deltaTop, int padding, float defaultValue, long long totalItems )
{
	const int cg = channels / VECW;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < totalItems; item += step ) {
		long long t = item;
		const int c = static_cast<int>( t % cg ) * VECW; t /= cg;
		const int x = static_cast<int>( t % toWidth ); t /= toWidth;
		const int y = static_cast<int>( t % toHeight ); t /= toHeight;
		const long long n = t;
		const int sy = resizeInputCoord( y - deltaTop, height, padding );
		const int sx = resizeInputCoord( x - deltaLeft, width, padding );
		const bool inside = sy >= 0 && sy < height && sx >= 0 && sx < width;
		const float* p = from + ( ( n * height + sy ) * width + sx ) * channels + c;
		if( VECW == 4 ) {
			float4 v = make_float4( defaultValue, defaultValue, defaultValue, defaultValue );
			if( inside ) {
				v = *reinterpret_cast<const float4*>( p );
			}
			*reinterpret_cast<float4*>( to + item * 4 ) = v;
		} else {
			to[item] = inside ? *p : defaultValue;
		}
	}
}

// ---------------------------------------------------------------------------------------------------------
// Split / merge along a blob dimension: the big blob is [objectCount][objectSize]; part i owns the columns
// [Offset[i], Offset[i+1]) of every row and is itself dense [objectCount][size_i].

struct CSplitParts {
	float* Data[NH_MAX_BLOB_DESCS];
	int Offset[NH_MAX_BLOB_DESCS + 1];
	int Count;
};

template<int VECW, bool MERGE>
__global__ __launch_bounds__( 256 )
void splitMergeKernel( float* big, const CSplitParts parts, int objectSize, long long totalItems )
{
	const int rowItems = objectSize / VECW;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < totalItems; item += step ) {
		const long long x = item / rowItems;
		const int pos = static_cast<int>( item - x * rowItems ) * VECW;
		int part = 0;
		while( part + 1 < parts.Count && pos >= parts.Offset[part + 1] ) {
			++part;
		}
		const int size = parts.Offset[part + 1] - parts.Offset[part];
		float* small = parts.Data[part] + x * size + ( pos - parts.Offset[part] );
		float* large = big + x * objectSize + pos;
		if( VECW == 4 ) {
			if( MERGE ) {
				*reinterpret_cast<float4*>( large ) = *reinterpret_cast<const float4*>( small );
			} else {
				*reinterpret_cast<float4*>( small ) = *reinterpret_cast<const float4*>( large );
			}
		} else {
			if( MERGE ) {
				*large = *small;
			} else {
				*small = *large;
			}
		}
	}
}

static long long dimProduct( const nhBlobDesc& d, int from, int to )
{
	long long p = 1;
	for( int i = from; i < to; ++i ) {
		p *= d.dims[i];
	}
	return p;
}

template<bool MERGE>
static int splitMergeImpl( nhStream s, int dim, const nhBlobDesc& bigDesc, float* big, const nhBlobDesc* partDescs,
	float* const* partData, int count )
{
	if( dim < 0 || dim >= 7 || count < 1 || count > NH_MAX_BLOB_DESCS ) {
		setLastError( "BlobSplitByDim/BlobMergeByDim: bad dimension or part count" );
		return NH_ERR_ARGUMENT;
	}
	const long long objectCount = dimProduct( bigDesc, 0, dim );
	const long long blobSize = dimProduct( bigDesc, 0, 7 );
	CSplitParts parts;
	parts.Count = count;
	parts.Offset[0] = 0;
	bool vec = isAligned16( big );
	long long objectSize = 0;
	if( dim == 0 ) {
		// concatenation of whole blobs: one row, part sizes are the blob sizes
		for( int i = 0; i < count; ++i ) {
			objectSize += dimProduct( partDescs[i], 0, 7 );
			if( objectSize > 0x7fffffffLL ) {
				setLastError( "BlobSplitByDim/BlobMergeByDim: blob is too large" );
				return NH_ERR_ARGUMENT;
			}
			parts.Offset[i + 1] = static_cast<int>( objectSize );
		}
	} else {
		for( int i = 0; i < count; ++i ) {
			objectSize += dimProduct( partDescs[i], dim, 7 );
			if( objectSize > 0x7fffffffLL ) {
				setLastError( "BlobSplitByDim/BlobMergeByDim: blob is too large" );
				return NH_ERR_ARGUMENT;
			}
			parts.Offset[i + 1] = static_cast<int>( objectSize );
		}
	}
	const long long rows = dim == 0 ? 1 : objectCount;
	if( rows * objectSize != blobSize ) {
		setLastError( "BlobSplitByDim/BlobMergeByDim: part sizes do not add up to the blob" );
		return NH_ERR_ARGUMENT;
	}
	if( blobSize == 0 ) {
		return NH_OK;
	}
	for( int i = 0; i < count; ++i ) {
		parts.Data[i] = partData[i];
		if( parts.Offset[i + 1] > parts.Offset[i] && partData[i] == nullptr ) {
			setLastError( "BlobSplitByDim/BlobMergeByDim: null part pointer" );
			return NH_ERR_ARGUMENT;
		}
		vec = vec && isAligned16( partData[i] ) && parts.Offset[i + 1] % 4 == 0;
	}
	const long long items = vec ? blobSize / 4 : blobSize;
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 262144 ? 262144 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( ( splitMergeKernel<4, MERGE> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			big, parts, static_cast<int>( objectSize ), items );
	} else {
		hipLaunchKernelGGL( ( splitMergeKernel<1, MERGE> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			big, parts, static_cast<int>( objectSize ), items );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// ---------------------------------------------------------------------------------------------------------
// LSTM gate kernel: gates [B x 4H] = main | forget | input | output (pre-activation, free term included)
//   c = sigmoid( f ) * cPrev + sigmoid( i ) * tanh( a );  h = sigmoid( o ) * tanh( c )
// (src/CPU/CpuMathEngineDnnLstm.h:49-90)

__device__ __forceinline__ float lstmExp( float x )
{
	if( x < -87.33654474f ) return 0.f;
	if( x > 88.f ) return FLT_MAX;
	return expf( x );
}
__device__ __forceinline__ float lstmSigmoid( float x )
{
	const float e = lstmExp( x );
	return e / ( e + 1.f );
}

__global__ __launch_bounds__( 256 )
void lstmGatesKernel( const float* gates, const float* statePrev, float* stateOut, float* mainOut, int hidden, int total )
{
	const int i = blockIdx.x * 256 + threadIdx.x;
	if( i >= total ) {
		return;
	}
	const int b = i / hidden;
	const int j = i - b * hidden;
	const float* g = gates + static_cast<long long>( b ) * 4 * hidden + j;
	const float a = tanhf( g[0] );
	const float f = lstmSigmoid( g[hidden] );
	const float in = lstmSigmoid( g[2 * hidden] );
	const float o = lstmSigmoid( g[3 * hidden] );
	const float cPrev = statePrev != nullptr ? statePrev[i] : 0.f;
	const float c = f * cPrev + in * a;
	stateOut[i] = c;
	mainOut[i] = o * tanhf( c );
}

// One LSTM step in one launch: gates = pre + hPrev * Wrec^T on the matrix cores, then the gate non-linearities.
// A workgroup owns 64 sequences x 8 hidden units = a 64 x 32 block of the gate matrix (columns = 4 gates x 8
// units), so every value the cell update of those units needs meets inside the workgroup. 8 wavefronts: two
// 32-row halves x four slices of the reduction over H. Operands go from L2 straight into MFMA registers
// (each lane reads 64 contiguous bytes of its row per 32 k), the four K slices meet in LDS.
// The step is latency-bound (about 34 MFLOP); the point is one launch instead of a product, a bias add and
// a gate kernel per step.
constexpr int LstmRows = 64;
constexpr int LstmUnits = 8;
constexpr int LstmKSlices = 4;
constexpr int LstmThreads = 64 * 2 * LstmKSlices;
typedef float lstmAcc __attribute__( ( ext_vector_type( 16 ) ) );

__global__ __launch_bounds__( LstmThreads )
void lstmStepKernel( const float* pre, const float* hPrev, const float* wRec, const float* statePrev,
	float* stateOut, float* mainOut, int batch, int hidden )
{
	__shared__ float partial[LstmKSlices][LstmRows][33];
	const int wave = threadIdx.x >> 6;
	const int lane = threadIdx.x & 63;
	const int l32 = lane & 31;
	const int half = lane >> 5;
	const int mHalf = wave & 1;
	const int slice = wave >> 1;
	const int unit0 = blockIdx.x * LstmUnits;
	const int row0 = blockIdx.y * LstmRows;

	// the cell update this thread does after the product: its inputs are requested first, so that their
	// latency (they were written long ago and come from HBM) hides behind the product
	const int row = threadIdx.x >> 3;
	const int unit = threadIdx.x & 7;
	const int b = row0 + row;
	const bool active = b < batch;
	const int cell = b * hidden + unit0 + unit;
	float g[4] = { 0.f, 0.f, 0.f, 0.f };
	float cPrev = 0.f;
	if( active ) {
#pragma unroll
		for( int q = 0; q < 4; ++q ) {
			g[q] = pre[static_cast<long long>( b ) * 4 * hidden + q * hidden + unit0 + unit];
		}
		if( statePrev != nullptr ) {
			cPrev = statePrev[cell];
		}
	}

	lstmAcc acc;
#pragma unroll
	for( int r = 0; r < 16; ++r ) {
		acc[r] = 0.f;
	}
	if( hPrev != nullptr ) {
		const __amdgpu_buffer_rsrc_t bufA = makeBuffer( hPrev );
		const __amdgpu_buffer_rsrc_t bufB = makeBuffer( wRec );
		const int aRow = row0 + mHalf * 32 + l32;
		const int bRow = ( l32 >> 3 ) * hidden + unit0 + ( l32 & 7 ); // column l32 of the block = gate l32/8, unit l32%8
		// lanes 0-31 take k0..k0+15 of their row, lanes 32-63 k0+16..k0+31: MFMA e of a 32-k chunk reduces over
		// { k0+e, k0+16+e }, the same pairing for both operands
		const unsigned aBase = aRow < batch ? static_cast<unsigned>( aRow * hidden + half * 16 ) * 4 : OutOfRange;
		const unsigned bBase = static_cast<unsigned>( bRow * hidden + half * 16 ) * 4;
		for( int k0 = slice * 32; k0 < hidden; k0 += 32 * LstmKSlices ) {
			float4 a[4], w[4];
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				a[q] = bufferLoad4( bufA, aBase + static_cast<unsigned>( k0 + q * 4 ) * 4 );
				w[q] = bufferLoad4( bufB, bBase + static_cast<unsigned>( k0 + q * 4 ) * 4 );
			}
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[q].x, w[q].x, acc, 0, 0, 0 );
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[q].y, w[q].y, acc, 0, 0, 0 );
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[q].z, w[q].z, acc, 0, 0, 0 );
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[q].w, w[q].w, acc, 0, 0, 0 );
			}
		}
	}
#pragma unroll
	for( int r = 0; r < 16; ++r ) {
		partial[slice][mHalf * 32 + ( r >> 2 ) * 8 + half * 4 + ( r & 3 )][l32] = acc[r];
	}
	__syncthreads();
	if( !active ) {
		return;
	}
#pragma unroll
	for( int q = 0; q < 4; ++q ) {
#pragma unroll
		for( int sl = 0; sl < LstmKSlices; ++sl ) {
			g[q] += partial[sl][row][q * 8 + unit];
		}
	}
	const float a = tanhf( g[0] );
	const float f = lstmSigmoid( g[1] );
	const float in = lstmSigmoid( g[2] );
	const float o = lstmSigmoid( g[3] );
	const float c = f * cPrev + in * a;
	stateOut[cell] = c;
	mainOut[cell] = o * tanhf( c );
}

// ---------------------------------------------------------------------------------------------------------
// The whole sequence in ONE launch. The per-step launch above costs about 7 us per step, nearly all of it the
// launch latency between dependent kernels; here the workgroups stay resident for all T steps and hand each
// step's output to one another through memory.
//   workgroup  = 4*CB hidden units x RB (16 or 32) sequences, W wavefronts: the gate columns of those units are CB
//                16-wide MFMA blocks; their rows of Wrec (16*CB x H) are copied to LDS once and stay there for all
//                steps, the cell state of the workgroup's cells lives in registers for all steps;
//   per step   : the wavefronts split the reduction over H in chunks of 16 k (v_mfma_f32_16x16x4_f32), meet in
//                LDS, and every wavefront does the cell update of its share of the (sequence, unit) cells;
//   exchange   : besides the plain store into the output blob, every h value is published as a 64-bit word
//                { float bits, step tag } with ONE device-scope relaxed atomic store (it goes to the level where the
//                eight L2s of the device agree). A consumer loads the words of the rows it multiplies with
//                device-scope atomic loads and repeats the loads until every tag names the step it needs: value and
//                "it has been written" arrive in the same word, so a step costs one store-to-load visibility
//                latency, with no counter, no flag and no fence. (An arrival counter bumped by 256 workgroups cost
//                6 us per step; device-scope fences, which write back and invalidate L2, 27 us.)
//                Such loads are not served by L2 and their round trip grows with the volume in flight, so wide
//                workgroups (many units, every published word read by few workgroups) beat many narrow ones.
//                Two exchange buffers alternate by step parity: a workgroup can only write step i+2 after it has
//                read step i+1 from every producer of its rows, i.e. after all of them finished reading step i.
//                The host clears the buffers before the launch, tags start at 1, so stale memory never matches.
// All workgroups must be resident together: the host only takes this path when the grid fits the device. The wait
// is bounded: after MaxSpins rounds of loads, or when another workgroup gave up, a wavefront raises the abort word
// and the workgroup leaves at its next barrier, so the grid always drains.
constexpr int SeqUnits = 4; // hidden units per 16-column block: column n = unit n/4, gate n%4
typedef float f32x4v __attribute__( ( ext_vector_type( 4 ) ) );

struct CLstmSeqArgs {
	const float* Gates;            // [T][B][4H] input contribution + free term
	const float* Wrec;             // [4H][H]
	const float* H0;               // [B][H] or null
	const float* C0;               // [B][H] or null
	float* HOut;                   // [T][B][H]
	float* COut;                   // [T][B][H] or null
	unsigned long long* Exchange;  // [2][B][H] tagged h values, zero at launch
	unsigned* Abort;               // one word, zero at launch
	unsigned* GaveUp;              // host-visible word of the launch stream: set when a wavefront gives up
	int T, B, H, Reverse;
	unsigned MaxSpins;
	// ( lstmDirectKernel ) XcdLayout != 0: the workgroups that share a block of sequences are meant to sit on one XCD
	// ( workgroup i of a launch goes to XCD i mod 8: that is how the dispatcher deals them out ) and publish into
	// ExchangeLocal as well, with plain stores, which stay in that XCD's L2; XcdTable[ workgroup ] receives 1 + the XCD
	// each one really runs on, and only when all of a block's workgroups report the same one is ExchangeLocal read
	int XcdLayout, XcdBase, RowBlocks;
	unsigned long long* ExchangeLocal; // [2][B][H], zero at launch
	unsigned* XcdTable;                // [ LstmXcdTableWords ], zero at launch
};
constexpr int LstmXcdTableWords = 256; // one word per workgroup of the layout by XCDs ( 8 x 32 )
typedef unsigned u32x2 __attribute__( ( ext_vector_type( 2 ) ) );

// Gate non-linearities on the hardware exp2 / reciprocal: 1 ulp each, and the cell update of a step sits on the
// critical path of the whole device. Saturation: exp2 gives +inf / 0 at the ends, the reciprocal turns them into the
// 0 / 1 (-1 / 1) that the clamped reference formulas give.
__device__ __forceinline__ float seqSigmoid( float x )
{
	return __builtin_amdgcn_rcpf( 1.f + __builtin_amdgcn_exp2f( -1.4426950408889634f * x ) );
}
__device__ __forceinline__ float seqTanh( float x )
{
	return 1.f - 2.f * __builtin_amdgcn_rcpf( 1.f + __builtin_amdgcn_exp2f( 2.8853900817779268f * x ) );
}


template<int RB, int CB, int W>
__global__ __launch_bounds__( 64 * W )
void lstmSequenceKernel( const CLstmSeqArgs a )
{
	extern __shared__ __attribute__( ( aligned( 16 ) ) ) float seqLds[];
	__shared__ int giveUp;
	constexpr int Threads = 64 * W;
	constexpr int RBlocks = RB / 16;
	constexpr int Units = CB * SeqUnits;  // hidden units of this workgroup
	constexpr int Cols = CB * 16;         // their gate columns
	constexpr int PartPitch = Cols + 4;   // rows stay 16-byte aligned: a cell reads its four gates with one 128-bit load
	constexpr int Batch = 16; // words per thread whose loads are in flight together
	// The first half of the wavefronts update the cells and publish, the second half fetch the next step's values.
	// A wavefront's loads and stores complete in issue order, so a wavefront that has just published could only
	// consume a load once its stores have been acknowledged by the far end (about half a microsecond).
	constexpr int CellWaves = W / 2;
	constexpr int CellsPerWave = RB * Units / CellWaves;
	constexpr int LoadThreads = ( W - CellWaves ) * 64;
	static_assert( CellsPerWave <= 64 && CellsPerWave * CellWaves == RB * Units, "the cells divide evenly over the cell wavefronts" );
	const int H = a.H, B = a.B;
	const int pitch = H + 4;
	float* wLds = seqLds;                   // [Cols][pitch]  this workgroup's rows of Wrec
	float* hTile = wLds + Cols * pitch;     // [RB][pitch]    the previous step's output of this workgroup's sequences
	float* partial = hTile + RB * pitch + 4; // [W][RB][PartPitch]; the 4 floats between are the loaders' spare slot
	const int tid = threadIdx.x;
	const int wave = tid >> 6;
	const int lane = tid & 63;
	const int col = lane & 15; // MFMA: row of the A block / column of the B block
	const int kq = lane >> 4;  // MFMA: which 4 of the 16 k of a chunk
	const int unitBlocks = H / Units;
	const int unit0 = ( blockIdx.x % unitBlocks ) * Units;
	const int row0 = ( blockIdx.x / unitBlocks ) * RB;
	const int rowsHere = min( RB, B - row0 );

	// gate column n of this workgroup = unit unit0 + n/4, gate n%4: the four gates of a cell are neighbours
	for( int idx = tid; idx < Cols * ( H / 4 ); idx += Threads ) {
		const int n = idx / ( H / 4 );
		const int k4 = idx - n * ( H / 4 );
		const int gate = n & 3;
		const int unit = unit0 + ( n >> 2 );
		const float4 v = *reinterpret_cast<const float4*>( a.Wrec + ( static_cast<long long>( gate ) * H + unit ) * H + k4 * 4 );
		*reinterpret_cast<float4*>( wLds + n * pitch + k4 * 4 ) = v;
	}
	// rows of the tile beyond the last sequence stay zero for all steps
	for( int idx = tid; idx < RB * pitch; idx += Threads ) {
		hTile[idx] = 0.f;
	}
	__syncthreads();
	if( a.H0 != nullptr ) {
		const int rows = min( RB, B - row0 );
		for( int j = tid; j < rows * H; j += Threads ) {
			hTile[( j / H ) * pitch + j % H] = a.H0[static_cast<long long>( row0 ) * H + j];
		}
	}
	if( tid == 0 ) {
		giveUp = 0;
	}

	// the cell this thread updates
	const int cellId = wave * CellsPerWave + lane;
	const int cellRow = cellId / Units;
	const int cellUnit = cellId % Units;
	const int cellB = row0 + cellRow;
	const bool cellActive = wave < CellWaves && lane < CellsPerWave && cellB < B;
	const bool loader = wave >= CellWaves;
	const int loadTid = tid - CellWaves * 64;
	const int cellCol = cellUnit * 4; // its four gate columns
	float cState = ( cellActive && a.C0 != nullptr ) ? a.C0[static_cast<long long>( cellB ) * H + unit0 + cellUnit] : 0.f;
	const long long stepSize = static_cast<long long>( B ) * H;
	const int chunks = H / 16;
	const int tileWords = rowsHere * H; // the tile's rows are contiguous in [B][H]
	const long long tileBase = static_cast<long long>( row0 ) * H;
	__syncthreads();

	// the input contribution of the step after the current one is requested a step ahead, before the current
	// step's stores are issued: loads return in order, so a load issued after the (slow, device-coherent) stores
	// could only be consumed once those stores have been acknowledged
	float gNext[4] = { 0.f, 0.f, 0.f, 0.f };
	auto requestGates = [&]( int step ) {
		if( cellActive && step < a.T ) {
			const int p = a.Reverse ? a.T - 1 - step : step;
			const float* src = a.Gates + ( static_cast<long long>( p ) * B + cellB ) * 4 * H + unit0 + cellUnit;
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				gNext[q] = src[q * H];
			}
		}
	};
	requestGates( 0 );

	// Loader thread t fetches words t, t + LoadThreads, ... of the tile ( word j = row j / H, column j % H ): a
	// wavefront's load covers 64 consecutive words, whole cache lines, each requested once. The positions are worked
	// out once: integer division by H inside the step loop would cost more than the loads. The host only picks a
	// shape whose loaders cover the tile in one batch ( RB * H <= Batch * LoadThreads ).
	int wordIndex[Batch], ldsIndex[Batch];
	unsigned wordMask[Batch]; // all ones inside the tile, zero beyond it
#pragma unroll
	for( int n = 0; n < Batch; ++n ) {
		const int j = n * LoadThreads + loadTid;
		const bool inside = loader && j < tileWords;
		wordIndex[n] = inside ? j : 0;
		wordMask[n] = inside ? 0xffffffffu : 0u;
		ldsIndex[n] = inside ? ( j / H ) * pitch + j % H : RB * pitch;
	}

	for( int i = 0; i < a.T; ++i ) {
		const int pos = a.Reverse ? a.T - 1 - i : i;
		const bool havePrev = i > 0 || a.H0 != nullptr;
		// ---- the previous output of this workgroup's sequences -> hTile (step 0: put there before the loop)
		if( i > 0 && loader ) {
			const unsigned long long* published = a.Exchange + ( ( i - 1 ) & 1 ) * stepSize + tileBase;
			const unsigned tag = static_cast<unsigned>( i ); // step i-1 publishes with tag i
			// Every load of a round is unconditional and all are in flight together (a conditional atomic load cannot be
			// hoisted): words beyond the tile read word 0, are not checked and land in the spare LDS slot.
			unsigned long long word[Batch];
			unsigned spins = 0;
			// A round of Batch loads per thread takes about half a microsecond, one load a fifth of that: wait on the
			// first word of every thread (together they touch every producer) before asking for everything.
			while( true ) {
				const unsigned long long first = __hip_atomic_load( published + wordIndex[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
				const unsigned mismatch = ( static_cast<unsigned>( first >> 32 ) ^ tag ) & wordMask[0];
				if( __builtin_amdgcn_ballot_w64( mismatch != 0 ) == 0 || ++spins > a.MaxSpins ) {
					break; // ( at the spin limit the full round below fails and gives up )
				}
			}
			while( true ) {
#pragma unroll
				for( int n = 0; n < Batch; ++n ) {
					word[n] = __hip_atomic_load( published + wordIndex[n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
				}
				unsigned mismatch = 0; // branch-free: every tag xor the wanted one, or-ed
#pragma unroll
				for( int n = 0; n < Batch; ++n ) {
					mismatch |= ( static_cast<unsigned>( word[n] >> 32 ) ^ tag ) & wordMask[n];
				}
				if( __builtin_amdgcn_ballot_w64( mismatch != 0 ) == 0 ) {
					break;
				}
				if( ++spins > a.MaxSpins || ( ( spins & 15 ) == 0
					&& __hip_atomic_load( a.Abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT ) != 0 ) )
				{
					__hip_atomic_store( a.Abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
					if( lane == 0 ) {
						// the abort word lives in the caller's workspace, which the caller is free to recycle: the host
						// learns of the give-up through this word of pinned host memory that belongs to the launch stream
						__hip_atomic_store( a.GaveUp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM );
					}
					giveUp = 1; // read by the whole workgroup after the next barrier
					break;
				}
			}
#pragma unroll
			for( int n = 0; n < Batch; ++n ) {
				hTile[ldsIndex[n]] = __uint_as_float( static_cast<unsigned>( word[n] ) );
			}
		}
		__syncthreads();
		if( giveUp != 0 ) {
			return; // uniform: every thread reads the same LDS word after the barrier
		}

		// ---- gates += hTile * Wrec^T for this workgroup's columns; the wavefronts split the reduction over H
		// One accumulator per ( column block, row block, k lane of the chunk ): consecutive MFMAs never wait for one
		// another's result; the four k lanes are summed at the end.
		f32x4v acc[CB][RBlocks][4];
#pragma unroll
		for( int cb = 0; cb < CB; ++cb ) {
#pragma unroll
			for( int rb = 0; rb < RBlocks; ++rb ) {
#pragma unroll
				for( int e = 0; e < 4; ++e ) {
					acc[cb][rb][e] = f32x4v{ 0.f, 0.f, 0.f, 0.f };
				}
			}
		}
		if( havePrev ) {
			for( int chunk = wave; chunk < chunks; chunk += W ) {
				const int k = chunk * 16 + kq * 4;
				// MFMA e of the chunk reduces over k = chunk*16 + { e, 4+e, 8+e, 12+e }: the same pairing on both operands
				float4 w[CB], h[RBlocks];
#pragma unroll
				for( int cb = 0; cb < CB; ++cb ) {
					w[cb] = *reinterpret_cast<const float4*>( wLds + ( cb * 16 + col ) * pitch + k );
				}
#pragma unroll
				for( int rb = 0; rb < RBlocks; ++rb ) {
					h[rb] = *reinterpret_cast<const float4*>( hTile + ( rb * 16 + col ) * pitch + k );
				}
#pragma unroll
				for( int rb = 0; rb < RBlocks; ++rb ) {
#pragma unroll
					for( int cb = 0; cb < CB; ++cb ) {
						acc[cb][rb][0] = __builtin_amdgcn_mfma_f32_16x16x4f32( h[rb].x, w[cb].x, acc[cb][rb][0], 0, 0, 0 );
						acc[cb][rb][1] = __builtin_amdgcn_mfma_f32_16x16x4f32( h[rb].y, w[cb].y, acc[cb][rb][1], 0, 0, 0 );
						acc[cb][rb][2] = __builtin_amdgcn_mfma_f32_16x16x4f32( h[rb].z, w[cb].z, acc[cb][rb][2], 0, 0, 0 );
						acc[cb][rb][3] = __builtin_amdgcn_mfma_f32_16x16x4f32( h[rb].w, w[cb].w, acc[cb][rb][3], 0, 0, 0 );
					}
				}
			}
		}
		// accumulator register r of lane l is element ( row 4*(l/16) + r, column l%16 ) of the 16 x 16 block
#pragma unroll
		for( int cb = 0; cb < CB; ++cb ) {
#pragma unroll
			for( int rb = 0; rb < RBlocks; ++rb ) {
#pragma unroll
				for( int r = 0; r < 4; ++r ) {
					partial[( wave * RB + rb * 16 + kq * 4 + r ) * PartPitch + cb * 16 + col] =
						( acc[cb][rb][0][r] + acc[cb][rb][1][r] ) + ( acc[cb][rb][2][r] + acc[cb][rb][3][r] );
				}
			}
		}
		__syncthreads();
		float g[4];
#pragma unroll
		for( int q = 0; q < 4; ++q ) {
			g[q] = gNext[q];
		}
		if( cellActive ) {
			float4 part[W];
#pragma unroll
			for( int wv = 0; wv < W; ++wv ) {
				part[wv] = *reinterpret_cast<const float4*>( partial + ( wv * RB + cellRow ) * PartPitch + cellCol );
			}
#pragma unroll
			for( int wv = 0; wv < W; ++wv ) {
				g[0] += part[wv].x; g[1] += part[wv].y; g[2] += part[wv].z; g[3] += part[wv].w;
			}
		}
		// ( `partial` and `hTile` are next written after the tile barrier of step i+1, which the cell wavefronts only
		// reach when they are done reading )
		requestGates( i + 1 );
		if( cellActive ) {
			const float m = seqTanh( g[0] );
			const float f = seqSigmoid( g[1] );
			const float in = seqSigmoid( g[2] );
			const float o = seqSigmoid( g[3] );
			cState = f * cState + in * m;
			const float h = o * seqTanh( cState );
			const long long cellInStep = static_cast<long long>( cellB ) * H + unit0 + cellUnit;
			if( i + 1 < a.T ) {
				const unsigned long long word = ( static_cast<unsigned long long>( i + 1 ) << 32 ) | __float_as_uint( h );
				__hip_atomic_store( a.Exchange + ( i & 1 ) * stepSize + cellInStep, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
			}
			a.HOut[pos * stepSize + cellInStep] = h;
			if( a.COut != nullptr ) {
				a.COut[pos * stepSize + cellInStep] = cState;
			}
		}
		// The loader wavefronts start asking for step i's values only now that this workgroup has published its own
		// (the workgroups run in lockstep, so the others are about as far): a round of loads issued earlier would
		// come back incomplete and cost a whole round trip.
		__syncthreads();
	}
}

// The same recurrence laid out by XCDs, for a device of 8 XCDs x 32 compute units: the workgroups that exchange values
// sit on one XCD and talk through that XCD's L2 with plain stores and loads that pass the L1 ( a third of the latency of
// a device-coherent store and load ), and the product takes its operand straight from the exchange: no staging of the
// previous output in LDS, one barrier per step instead of three.
//   workgroup  = 4 sequences x 32 hidden units ( 128 gate columns ); H / 64 product wavefronts + 2 cell wavefronts.
//                What a step has to move grows with the sequences a workgroup holds ( every workgroup reads the whole
//                previous output of its sequences: 4 x H tagged words ), and all of an XCD's workgroups ask the same L2
//                for it at the same time: with 16 sequences per workgroup those loads alone took a microsecond.
//   product    : v_mfma_f32_4x4x1_16b_f32, sixteen 4 x 4 rank-1 updates per instruction, with the A operand of one of
//                the sixteen blocks broadcast to all: A = h[ 4 sequences ][ k ], B = Wrec[ k ][ 64 columns ], so four
//                sequences fill the instruction. Wavefront m reduces over k = 64m .. 64m+63 for all 128 columns; its
//                64 x 128 weights never leave its registers ( 128 per lane ). Lane ( b, i ) loads the tagged word
//                h[ i ][ 64m + 16q + b ], q = 0..3: one register feeds sixteen instructions ( block b's value is
//                broadcast by instruction b ), four 64-bit loads per lane and step.
//                A wavefront waits with a light load ( one word of every store instruction that publishes into its k
//                range ) and then asks for everything; what it uses is checked word by word. ( Waiting with the full
//                request instead, 2 KB per wavefront and round, saves a round trip on paper and cost 15 %: 128 steps
//                266 -> 308 us. The waiting loads of 128 workgroups per XCD stand in the way of the stores they wait for. )
//   cells      : 128 cells, two wavefronts. Every load and store is a buffer access issued on every path ( a lane or
//                step with nothing to move gets an offset beyond the range, which the hardware drops ), so the compiler
//                can count what is in flight and wait for the gate loads alone; the wavefronts that publish never wait
//                for a load of the exchange. The sums of the product wavefronts meet in LDS ( two buffers, by step
//                parity ), one barrier, and the cell wavefronts finish the step while the product wavefronts already wait
//                for the next one.
//   placement  : the launch has 8 x 32 workgroups. The dispatcher deals a launch's workgroups out to the XCDs in turn,
//                so every XCD receives 32; which XCD comes first is not known, so a workgroup asks where it runs and
//                takes the next role of that XCD ( a counter per XCD ). XCDs without sequences have nothing to do:
//                their workgroups leave at once ( the partner of a pair of launches uses them ).
//   step 0     : the initial output ( or zero ) is published like a step's output before the loop, so every step is
//                the same code. Step i reads buffer ( i+1 )&1 with tag i+1 and publishes into buffer i&1 with tag i+2:
//                by the time a workgroup can publish step i, every workgroup of its sequences has published step i-1,
//                i.e. has the values of step i-2, which this store overwrites, in registers.
// set when a one-launch LSTM gave up ( for one, the device may not deal workgroups out as the layout by XCDs assumes ):
// the process goes on without that layout
static int xcdLayoutFailed = 0;
constexpr int RowsKernelRows = 4;
constexpr int RowsKernelUnits = 32;
// f( integral_constant<int, 0> ) ... f( integral_constant<int, N-1> ), for arguments that have to be constants
template<int N, class F>
__device__ __forceinline__ void staticFor( F&& f )
{
	if constexpr( N > 0 ) {
		staticFor<N - 1>( f );
		f( std::integral_constant<int, N - 1>() );
	}
}
template<int PW>
__global__ __launch_bounds__( 64 * ( PW + 2 ) )
void lstmRowsKernel( const CLstmSeqArgs a )
{
	__shared__ __attribute__( ( aligned( 16 ) ) ) float sumsLds[2][PW][RowsKernelRows][132];
	__shared__ int giveUp;
	__shared__ int role;
	constexpr int H = 64 * PW;
	constexpr int UnitGroups = H / RowsKernelUnits;
	const int B = a.B;
	const int tid = threadIdx.x;
	const int wave = tid >> 6;
	const int lane = tid & 63;
	unsigned xcd = 0;
	asm volatile( "s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"( xcd ) );
	const int slot = ( static_cast<int>( xcd & 7 ) - a.XcdBase ) & 7;
	if( slot >= a.RowBlocks ) {
		return;
	}
	if( tid == 0 ) {
		role = static_cast<int>( __hip_atomic_fetch_add( a.XcdTable + ( xcd & 7 ), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT ) );
		giveUp = 0;
	}
	__syncthreads();
	const int ticket = role;
	const int unit0 = ( ticket % UnitGroups ) * RowsKernelUnits;
	const int row0 = ( slot * ( 32 / UnitGroups ) + ticket / UnitGroups ) * RowsKernelRows;
	if( ticket >= 32 || row0 >= B ) {
		return; // ( more workgroups on this XCD than the dealing in turn gives it, or no sequences left for this role )
	}
	// ( 32-bit products on purpose: the scalar unit has no 64-bit multiply, and a 64-bit product would put every address
	// derived from it, buffer descriptors included, into vector registers; the host checks that T * B * 4H fits 31 bits )
	const unsigned stepSize = static_cast<unsigned>( B ) * static_cast<unsigned>( H );
	const unsigned stepBytes = stepSize * 4u;
	const bool product = wave < PW;
	const __amdgpu_buffer_rsrc_t exchange = __builtin_amdgcn_make_buffer_rsrc( a.ExchangeLocal, 0, stepBytes * 4u, 0x00020000 );

	// ---- cell wavefronts: the cell of this lane
	const int cellId = ( wave - PW ) * 64 + lane;
	const int cellRow = ( cellId / RowsKernelUnits ) & ( RowsKernelRows - 1 );
	const int cellUnit = cellId % RowsKernelUnits;
	const int cellB = row0 + cellRow;
	const bool cellActive = !product && cellB < B;
	const unsigned cellInStep = static_cast<unsigned>( cellB ) * H + unit0 + cellUnit;
	float cState = ( cellActive && a.C0 != nullptr ) ? a.C0[cellInStep] : 0.f;
	float gNext[4] = { 0.f, 0.f, 0.f, 0.f };
	const unsigned gateOffset = cellActive ? ( static_cast<unsigned>( cellB ) * 4u * H + unit0 + cellUnit ) * 4u : OutOfRange;
	auto requestGates = [&]( int step ) {
		const int p = a.Reverse ? a.T - 1 - step : step;
		const __amdgpu_buffer_rsrc_t gates = __builtin_amdgcn_make_buffer_rsrc(
			const_cast<float*>( a.Gates + static_cast<size_t>( step < a.T ? static_cast<unsigned>( p ) * ( stepSize * 4u ) : 0u ) ), 0,
			step < a.T ? stepBytes * 4u : 0u, 0x00020000 );
#pragma unroll
		for( int q = 0; q < 4; ++q ) {
			gNext[q] = __uint_as_float( __builtin_amdgcn_raw_buffer_load_b32( gates, gateOffset, q * H * 4, 0 ) );
		}
	};
	auto publish = [&]( float h, unsigned tag, unsigned parity ) {
		// one 64-bit store that this XCD's L2 holds: value and "it has been written" arrive in the same word
		const u32x2 word = { __float_as_uint( h ), tag };
		__builtin_amdgcn_raw_buffer_store_b64( word, exchange, cellActive ? ( parity * stepSize + cellInStep ) * 8u : OutOfRange, 0, 0 );
	};
	float h0 = 0.f;
	if( cellActive && a.H0 != nullptr ) {
		h0 = a.H0[cellInStep];
	}
	requestGates( 0 );
	publish( h0, 1u, 1u );
	// ( the compiler's count of what may be in flight at the top of the loop is the worse of the two ways there: the two
	// output stores that follow a step's publication follow the first one too, beyond every range )
	__builtin_amdgcn_raw_buffer_store_b32( 0u, exchange, OutOfRange, 0, 0 );
	__builtin_amdgcn_raw_buffer_store_b32( 0u, exchange, OutOfRange, 0, 0 );

	// ---- product wavefronts
	// lane ( b, j ) of the B operand: column 4b + j of a 64-column half = gate j of unit 16 * half + b
	// lane ( b, i ) of the A operand: sequence i of the workgroup, k = 16q + b of the wavefront's 64
	const int lb = lane >> 2;
	const int li = lane & 3;
	float weights[2][64];
	if( product ) {
#pragma unroll
		for( int half = 0; half < 2; ++half ) {
			const float* from = a.Wrec + ( static_cast<size_t>( li ) * H + unit0 + half * 16 + lb ) * H + wave * 64;
#pragma unroll
			for( int k4 = 0; k4 < 16; ++k4 ) {
				const float4 v = *reinterpret_cast<const float4*>( from + k4 * 4 );
				weights[half][k4 * 4] = v.x; weights[half][k4 * 4 + 1] = v.y; weights[half][k4 * 4 + 2] = v.z; weights[half][k4 * 4 + 3] = v.w;
			}
		}
	}
	const bool rowValid = row0 + li < B;
	const unsigned laneWords = rowValid ? ( static_cast<unsigned>( row0 + li ) * H + wave * 64 + lb ) * 8u : OutOfRange;
	const unsigned rowMask = rowValid ? 0xffffffffu : 0u;
	// The light load: the wavefront's 64 k are two producers of 32 units, each with two cell wavefronts of two sequences:
	// lane l < 4 looks at producer l / 2, sequence 2 * ( l % 2 ).
	unsigned lightWords = OutOfRange;
	if( lane < 4 && row0 + 2 * ( lane & 1 ) < B ) {
		lightWords = ( static_cast<unsigned>( row0 + 2 * ( lane & 1 ) ) * H + wave * 64 + ( lane >> 1 ) * RowsKernelUnits ) * 8u;
	}
	const unsigned lightMask = lightWords != OutOfRange ? 0xffffffffu : 0u;

	for( int counter = 0; counter < a.T; ++counter ) {
		// ( the counter of a loop that lanes can leave at different times, as the compiler sees the give-up exit, lives in a
		// vector register; buffer descriptors derived from it would be rebuilt lane by lane )
		const int i = __builtin_amdgcn_readfirstlane( counter );
		const int pos = a.Reverse ? a.T - 1 - i : i;
		if( product ) {
			const unsigned tag = static_cast<unsigned>( i + 1 );
			const unsigned parityBytes = static_cast<unsigned>( ( i + 1 ) & 1 ) * stepBytes * 2u;
			// ( ACCS accumulators per half take the instructions in turn, so that one does not wait for the one before it;
			// the widest shape has no registers to spare for a second one )
			constexpr int ACCS = PW < 8 ? 2 : 1;
			f32x4v acc[2][ACCS];
#pragma unroll
			for( int half = 0; half < 2; ++half ) {
#pragma unroll
				for( int e = 0; e < ACCS; ++e ) {
					acc[half][e] = f32x4v{ 0.f, 0.f, 0.f, 0.f };
				}
			}
			unsigned spins = 0;
			while( true ) {
				asm volatile( "" ::: "memory" ); // ( every round asks the memory again )
				const u32x2 first = __builtin_amdgcn_raw_buffer_load_b64( exchange, lightWords, parityBytes, 2 );
				if( __builtin_amdgcn_ballot_w64( ( ( first.y ^ tag ) & lightMask ) != 0 ) == 0 || ++spins > a.MaxSpins ) {
					break; // ( at the spin limit the rounds below fail and give up )
				}
			}
			u32x2 word[4];
			auto arrived = [&]( int q ) {
				return __builtin_amdgcn_ballot_w64( ( ( word[q].y ^ tag ) & rowMask ) != 0 ) == 0;
			};
			auto multiply = [&]( int q ) {
				const float h = __uint_as_float( word[q].x );
				staticFor<16>( [&]( auto blockOf ) {
					constexpr int b = decltype( blockOf )::value;
					// cbsz 4: the A operand of block `b` goes to all sixteen blocks ( the block is part of the instruction )
					acc[0][b % ACCS] = __builtin_amdgcn_mfma_f32_4x4x1f32( h, weights[0][q * 16 + b], acc[0][b % ACCS], 4, b, 0 );
					acc[1][b % ACCS] = __builtin_amdgcn_mfma_f32_4x4x1f32( h, weights[1][q * 16 + b], acc[1][b % ACCS], 4, b, 0 );
				} );
			};
			// All four loads are asked for at once ( aux 2: past the L1, into this XCD's L2 ) and a quarter is multiplied
			// as soon as its load has come back, always in order: the sum does not depend on what arrived when.
			asm volatile( "" ::: "memory" );
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				word[q] = __builtin_amdgcn_raw_buffer_load_b64( exchange, laneWords, parityBytes + q * 128, 2 );
			}
			int good = 0;
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				if( good == q && arrived( q ) ) {
					multiply( q );
					good = q + 1;
				}
			}
			bool gone = false;
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				if( q < good || gone ) {
					continue;
				}
				// this quarter was not there yet: its load again until it is
				while( true ) {
					if( ++spins > a.MaxSpins || ( ( spins & 15 ) == 0
						&& __hip_atomic_load( a.Abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT ) != 0 ) )
					{
						__hip_atomic_store( a.Abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
						if( lane == 0 ) {
							// the abort word lives in the caller's workspace, which the caller is free to recycle: the host
							// learns of the give-up through this word of pinned host memory that belongs to the launch stream
							__hip_atomic_store( a.GaveUp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM );
						}
						giveUp = 1; // read by the whole workgroup after the barrier
						gone = true;
						break;
					}
					asm volatile( "" ::: "memory" );
					word[q] = __builtin_amdgcn_raw_buffer_load_b64( exchange, laneWords, parityBytes + q * 128, 2 );
					if( arrived( q ) ) {
						break;
					}
				}
				if( !gone ) {
					multiply( q );
				}
			}
			// accumulator register r of lane ( b, j ) is ( sequence r, column 4b + j ) of the half
#pragma unroll
			for( int half = 0; half < 2; ++half ) {
#pragma unroll
				for( int r = 0; r < 4; ++r ) {
					sumsLds[i & 1][wave][r][half * 64 + lane] = ACCS == 2 ? acc[half][0][r] + acc[half][ACCS - 1][r] : acc[half][0][r];
				}
			}
		}
		__syncthreads();
		if( giveUp != 0 ) {
			return; // uniform: every thread reads the same LDS word after the barrier
		}
		if( !product ) {
			float g[4];
#pragma unroll
			for( int q = 0; q < 4; ++q ) {
				g[q] = gNext[q];
			}
#pragma unroll
			for( int wv = 0; wv < PW; ++wv ) {
				const float4 part = *reinterpret_cast<const float4*>( &sumsLds[i & 1][wv][cellRow][cellUnit * 4] );
				g[0] += part.x; g[1] += part.y; g[2] += part.z; g[3] += part.w;
			}
			requestGates( i + 1 );
			const float m = seqTanh( g[0] );
			const float f = seqSigmoid( g[1] );
			const float in = seqSigmoid( g[2] );
			const float o = seqSigmoid( g[3] );
			cState = f * cState + in * m;
			const float h = o * seqTanh( cState );
			// ( the last step publishes too: nobody reads it, and the next launch starts from cleared buffers )
			publish( h, static_cast<unsigned>( i + 2 ), static_cast<unsigned>( i & 1 ) );
			const unsigned outOffset = cellActive ? cellInStep * 4u : OutOfRange;
			const size_t outAt = static_cast<size_t>( static_cast<unsigned>( pos ) * stepSize );
			const __amdgpu_buffer_rsrc_t hOut = __builtin_amdgcn_make_buffer_rsrc( a.HOut + outAt, 0, stepBytes, 0x00020000 );
			const __amdgpu_buffer_rsrc_t cOut = __builtin_amdgcn_make_buffer_rsrc(
				a.COut != nullptr ? a.COut + outAt : a.HOut, 0, a.COut != nullptr ? stepBytes : 0u, 0x00020000 );
			__builtin_amdgcn_raw_buffer_store_b32( __float_as_uint( h ), hOut, outOffset, 0, 0 );
			__builtin_amdgcn_raw_buffer_store_b32( __float_as_uint( cState ), cOut, outOffset, 0, 0 );
		}
	}
}

__global__ __launch_bounds__( 256 ) void clearWordsKernel( unsigned long long* words, long long count )
{
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < count; i += gridDim.x * 256LL ) {
		words[i] = 0;
	}
}

// Pooling gradients as gathers. Max: the gradient of an output element goes to the input element its stored index names
// (always inside the window, as the forward pass wrote it). Mean: every window spreads its gradient, times 1 / fh / fw.
// One kernel for both: every input element ( VECW channels of a pixel ) walks the windows that cover it, in the order
// the reference's loop adds them. MAX: a window contributes where its stored index names this element.
template<int VECW, bool MAX>
__global__ __launch_bounds__( 256 )
void poolingBackwardKernel( const nhPoolingDesc d, const float* resultDiff, const int* maxIndices, float* sourceDiff,
	long long totalItems )
{
	const float scale = 1.f / d.filterHeight / d.filterWidth;
	const int cg = d.channels / VECW;
	// ( an item's place from 32-bit divisions where the count allows it: four 64-bit ones were most of this kernel's instructions )
	const bool narrow = totalItems <= 0x7fffffffLL;
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < totalItems; item += static_cast<long long>( gridDim.x ) * 256 ) {
		int c, wi, hi;
		long long n;
		if( narrow ) {
			unsigned t = static_cast<unsigned>( item );
			c = static_cast<int>( t % static_cast<unsigned>( cg ) ) * VECW; t /= static_cast<unsigned>( cg );
			wi = static_cast<int>( t % static_cast<unsigned>( d.width ) ); t /= static_cast<unsigned>( d.width );
			hi = static_cast<int>( t % static_cast<unsigned>( d.height ) );
			n = t / static_cast<unsigned>( d.height );
		} else {
			long long t = item;
			c = static_cast<int>( t % cg ) * VECW; t /= cg;
			wi = static_cast<int>( t % d.width ); t /= d.width;
			hi = static_cast<int>( t % d.height );
			n = t / d.height;
		}
		// windows ho with ho * s <= hi < ho * s + fh
		const int hoFirst = hi >= d.filterHeight ? ( hi - d.filterHeight ) / d.strideHeight + 1 : 0;
		const int hoLast = min( hi / d.strideHeight, d.resultHeight - 1 );
		const int woFirst = wi >= d.filterWidth ? ( wi - d.filterWidth ) / d.strideWidth + 1 : 0;
		const int woLast = min( wi / d.strideWidth, d.resultWidth - 1 );
		const int own = ( hi * d.width + wi ) * d.channels + c; // index inside the object, as the forward pass stores it
		float sum[VECW];
#pragma unroll
		for( int e = 0; e < VECW; ++e ) {
			sum[e] = 0.f;
		}
		for( int ho = hoFirst; ho <= hoLast; ++ho ) {
			for( int wo = woFirst; wo <= woLast; ++wo ) {
				const long long at = ( ( n * d.resultHeight + ho ) * d.resultWidth + wo ) * d.channels + c;
				float g[VECW];
				int index[VECW];
				if( VECW == 4 ) {
					const float4 v = *reinterpret_cast<const float4*>( resultDiff + at );
					g[0] = v.x; g[1] = v.y; g[2] = v.z; g[3] = v.w;
					if( MAX ) {
						const int4 k = *reinterpret_cast<const int4*>( maxIndices + at );
						index[0] = k.x; index[1] = k.y; index[2] = k.z; index[3] = k.w;
					}
				} else {
					g[0] = resultDiff[at];
					if( MAX ) {
						index[0] = maxIndices[at];
					}
				}
#pragma unroll
				for( int e = 0; e < VECW; ++e ) {
					if( !MAX || index[e] == own + e ) {
						sum[e] += g[e];
					}
				}
			}
		}
		float* out = sourceDiff + item * VECW;
		if( VECW == 4 ) {
			*reinterpret_cast<float4*>( out ) = MAX ? make_float4( sum[0], sum[1], sum[2], sum[3] )
				: make_float4( sum[0] * scale, sum[1] * scale, sum[2] * scale, sum[3] * scale );
		} else {
			out[0] = MAX ? sum[0] : sum[0] * scale;
		}
	}
}

// Gradient of the channelwise convolution by its input: every input pixel gathers, tap by tap, the output pixels whose
// window holds it: ( hi + pad - kh ) / stride where that division is exact and in range.
template<int VECW>
__global__ __launch_bounds__( 256 )
void channelwiseConvBackwardKernel( const nhConvDesc d, const float* outputDiff, const float* filter, float* inputDiff,
	long long totalItems )
{
	typedef CChanVec<VECW> V;
	typedef typename V::Type T;
	const int cg = d.channels / VECW;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < totalItems; item += step ) {
		long long t = item;
		const int c = static_cast<int>( t % cg ) * VECW; t /= cg;
		const int wi = static_cast<int>( t % d.width ); t /= d.width;
		const int hi = static_cast<int>( t % d.height );
		const long long n = t / d.height;
		const float* image = outputDiff + n * d.resultHeight * d.resultWidth * d.channels + c;
		T acc = V::zero();
		for( int kh = 0; kh < d.filterHeight; ++kh ) {
			const int hs = hi + d.paddingHeight - kh;
			if( hs < 0 || hs % d.strideHeight != 0 || hs / d.strideHeight >= d.resultHeight ) {
				continue;
			}
			const float* row = image + static_cast<long long>( hs / d.strideHeight ) * d.resultWidth * d.channels;
			for( int kw = 0; kw < d.filterWidth; ++kw ) {
				const int ws = wi + d.paddingWidth - kw;
				if( ws < 0 || ws % d.strideWidth != 0 || ws / d.strideWidth >= d.resultWidth ) {
					continue;
				}
				acc = V::fma( V::load( row + ( ws / d.strideWidth ) * d.channels ),
					V::load( filter + ( kh * d.filterWidth + kw ) * d.channels + c ), acc );
			}
		}
		V::store( inputDiff + item * VECW, acc );
	}
}

// The 3x3, stride 2 case of the gradient by the input, 4 channels per thread. With a = hi + padH and b = wi + padW an
// input pixel lies in the window rows kh of a's parity: a = 2r meets output row r through tap row 0 and output row r - 1
// through tap row 2, a = 2r + 1 meets output row r through tap row 1; the same along the width. A thread owns a strip
// of 8 columns of b that starts at an even b and pairsPerItem row pairs ( 2r, 2r + 1 ): the strip reads 5 columns of the
// output gradient, and walking down it needs output row r - 1 and r for the pair r, so every row of the output
// gradient is loaded once per strip ( a ring of three rows in registers: the row of the next pair is requested before
// the current pair is computed and stored ) and which taps meet which pixel is known at compile time. Out-of-range
// output pixels are out-of-range buffer offsets ( they read as zero ); input pixels outside the image are not stored.
__global__ __launch_bounds__( 256 )
void channelwiseBackward3x3Stride2Kernel( const nhConvDesc d, const float* outputDiff, const float* filter, float* inputDiff,
	int wGroups, int rowChunks, int pairsPerItem, int pairs, int totalItems )
{
	const int item = xcdSwizzle( blockIdx.x, gridDim.x ) * 256 + threadIdx.x;
	if( item >= totalItems ) {
		return;
	}
	const int cg = d.channels / 4;
	int t = item;
	const int c = ( t % cg ) * 4; t /= cg;
	const int b0 = ( t % wGroups ) * 8; t /= wGroups;
	const int r0 = ( t % rowChunks ) * pairsPerItem;
	const int n = t / rowChunks;
	const int rEnd = min( r0 + pairsPerItem, pairs );

	const __amdgpu_buffer_rsrc_t diff = makeBuffer( outputDiff );
	const unsigned rowBytes = static_cast<unsigned>( d.resultWidth ) * d.channels * 4;
	const unsigned imageBytes = n * d.resultHeight * rowBytes;
	unsigned colOff[5];
#pragma unroll
	for( int j = 0; j < 5; ++j ) {
		const int wo = b0 / 2 - 1 + j;
		colOff[j] = wo >= 0 && wo < d.resultWidth ? static_cast<unsigned>( wo * d.channels + c ) * 4 : OutOfRange;
	}
	float4 f[9];
#pragma unroll
	for( int k = 0; k < 9; ++k ) {
		f[k] = *reinterpret_cast<const float4*>( filter + k * d.channels + c );
	}
	float4 ring[3][5];
	auto loadRow = [&]( float4* row, int ho ) {
		const bool valid = ho >= 0 && ho < d.resultHeight && ho < rEnd;
		const unsigned rowOff = imageBytes + static_cast<unsigned>( ho ) * rowBytes;
#pragma unroll
		for( int j = 0; j < 5; ++j ) {
			// a valid row offset is below 2 GiB, so adding an out-of-range column stays out of range
			row[j] = bufferLoad4( diff, valid ? rowOff + colOff[j] : OutOfRange );
		}
	};
	loadRow( ring[0], r0 - 1 );
	loadRow( ring[1], r0 );
	const long long inRow = static_cast<long long>( d.width ) * d.channels;
	float* const image = inputDiff + static_cast<long long>( n ) * d.height * inRow + c;
	const int wi0 = b0 - d.paddingWidth;
	for( int rBase = r0; rBase < rEnd; rBase += 3 ) {
#pragma unroll
		for( int k = 0; k < 3; ++k ) {
			const int r = rBase + k;
			if( r < rEnd ) {
				const float4* prev = ring[k % 3];
				const float4* cur = ring[( k + 1 ) % 3];
				loadRow( ring[( k + 2 ) % 3], r + 1 );
#pragma unroll
				for( int odd = 0; odd < 2; ++odd ) {
					const int hi = 2 * r + odd - d.paddingHeight;
					if( hi < 0 || hi >= d.height ) {
						continue;
					}
					float* out = image + hi * inRow + static_cast<long long>( wi0 ) * d.channels;
#pragma unroll
					for( int m = 0; m < 4; ++m ) {
						float4 even, uneven;
						if( odd == 0 ) {
							even = CChanVec<4>::mul( cur[m + 1], f[0] );
							even = CChanVec<4>::fma( cur[m], f[2], even );
							even = CChanVec<4>::fma( prev[m + 1], f[6], even );
							even = CChanVec<4>::fma( prev[m], f[8], even );
							uneven = CChanVec<4>::mul( cur[m + 1], f[1] );
							uneven = CChanVec<4>::fma( prev[m + 1], f[7], uneven );
						} else {
							even = CChanVec<4>::mul( cur[m + 1], f[3] );
							even = CChanVec<4>::fma( cur[m], f[5], even );
							uneven = CChanVec<4>::mul( cur[m + 1], f[4] );
						}
						const int wi = wi0 + 2 * m;
						if( wi >= 0 && wi < d.width ) {
							*reinterpret_cast<float4*>( out + ( 2 * m ) * d.channels ) = even;
						}
						if( wi + 1 >= 0 && wi + 1 < d.width ) {
							*reinterpret_cast<float4*>( out + ( 2 * m + 1 ) * d.channels ) = uneven;
						}
					}
				}
			}
		}
	}
}

template<int VECW> struct CChanAtomic;
template<> struct CChanAtomic<4> {
	static __device__ __forceinline__ void add( float* p, float4 v )
	{
		unsafeAtomicAdd( p, v.x ); unsafeAtomicAdd( p + 1, v.y ); unsafeAtomicAdd( p + 2, v.z ); unsafeAtomicAdd( p + 3, v.w );
	}
	static __device__ __forceinline__ float4 sum( float4 a, float4 b ) { return make_float4( a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w ); }
};
template<> struct CChanAtomic<1> {
	static __device__ __forceinline__ void add( float* p, float v ) { unsafeAtomicAdd( p, v ); }
	static __device__ __forceinline__ float sum( float a, float b ) { return a + b; }
};

// The 3x3 case of the gradient by the filter, on the forward pass's strips: a thread owns 4 channels of a strip WPT
// output pixels wide and rowsPerItem output rows tall, slides down it with the three input rows of the window in
// registers ( every input row loaded once per strip ) and keeps the nine tap sums and the free-term sum of its strip in
// registers. The threads of a workgroup then meet per channel in an LDS table ( LDS atomics ), and the workgroup leaves
// with one global atomic add per table entry: a few hundred adds per address over the whole launch.
//
// PARTIALS ( the form that is launched wherever the stream has scratch memory ): a workgroup has a whole number of threads
// per channel group ( blockDim = cg * threads per group ), a thread keeps its channel group for all its strips and its
// sums in registers until the end, the threads of a group then meet in LDS through plain stores and one pass of
// adds, and the workgroup leaves its 40 x cg sums in a row of its own in scratch memory; sumLearnPartialsKernel adds the
// rows up in workgroup order. No atomic anywhere: LDS float atomics cost several hundred cycles per wave instruction
// on this part ( 40 of them per strip were a third of the launch at 14 x 14 x 384 ), a few hundred global adds per
// address another third, and the sums now come out the same on every run.
template<int STRIDE, int WPT, bool PARTIALS>
__global__ __launch_bounds__( 256 )
void channelwiseLearn3x3Kernel( const nhConvDesc d, const float* input, const float* outputDiff, float* filterDiff,
	float* freeTermDiff, int wGroups, int rowChunks, int rowsPerItem, int totalItems, float* partials )
{
	constexpr int NC = ( WPT - 1 ) * STRIDE + 3;
	constexpr int Keep = 3 - STRIDE;
	constexpr int Sums = 10; // nine taps and the free term
	__shared__ float table[Sums * 4 * 256];
	const int cg = d.channels / 4; // at most 256: the table has a column per channel group
	const int tableWidth = PARTIALS ? static_cast<int>( blockDim.x ) : cg;
	if( !PARTIALS ) {
		for( int idx = threadIdx.x; idx < Sums * 4 * tableWidth; idx += blockDim.x ) {
			table[idx] = 0.f;
		}
		__syncthreads();
	}
	float4 kept[Sums];
#pragma unroll
	for( int k = 0; k < Sums; ++k ) {
		kept[k] = make_float4( 0.f, 0.f, 0.f, 0.f );
	}
	// a few hundred workgroups walk the strips grid-stride and collect in their table: the global adds at the end are what
	// limits this kernel when thousands of workgroups bring their own
	// ( PARTIALS: items are counted group-first too, and blockDim is a multiple of cg: item % cg stays what it is )
	for( int item = blockIdx.x * blockDim.x + threadIdx.x; item < totalItems; item += gridDim.x * blockDim.x ) {
		int t = item;
		const int group = t % cg;
		const int c = group * 4; t /= cg;
		const int wo0 = ( t % wGroups ) * WPT; t /= wGroups;
		const int ho0 = ( t % rowChunks ) * rowsPerItem;
		const int n = t / rowChunks;
		const int hoEnd = min( ho0 + rowsPerItem, d.resultHeight );

		const __amdgpu_buffer_rsrc_t image = makeBuffer( input );
		const unsigned rowBytes = static_cast<unsigned>( d.width ) * d.channels * 4;
		const unsigned imageBytes = n * d.height * rowBytes;
		unsigned colOff[NC];
		const int wi0 = wo0 * STRIDE - d.paddingWidth;
#pragma unroll
		for( int j = 0; j < NC; ++j ) {
			const int wi = wi0 + j;
			colOff[j] = wi >= 0 && wi < d.width ? static_cast<unsigned>( wi * d.channels + c ) * 4 : OutOfRange;
		}
		float4 rows[3][NC];
		auto loadRow = [&]( float4* row, int hi ) {
			const bool valid = hi >= 0 && hi < d.height;
			const unsigned rowOff = imageBytes + static_cast<unsigned>( hi ) * rowBytes;
#pragma unroll
			for( int j = 0; j < NC; ++j ) {
				row[j] = bufferLoad4( image, valid ? rowOff + colOff[j] : OutOfRange );
			}
		};
		float4 sums[Sums];
#pragma unroll
		for( int k = 0; k < Sums; ++k ) {
			sums[k] = make_float4( 0.f, 0.f, 0.f, 0.f );
		}
		int hi = ho0 * STRIDE - d.paddingHeight;
#pragma unroll
		for( int r = 0; r < Keep; ++r ) {
			loadRow( rows[r], hi + r );
		}
		const float* diff = outputDiff + ( ( static_cast<long long>( n ) * d.resultHeight + ho0 ) * d.resultWidth + wo0 ) * d.channels + c;
		const long long diffRow = static_cast<long long>( d.resultWidth ) * d.channels;
		for( int ho = ho0; ho < hoEnd; ++ho ) {
#pragma unroll
			for( int r = Keep; r < 3; ++r ) {
				loadRow( rows[r], hi + r );
			}
#pragma unroll
			for( int j = 0; j < WPT; ++j ) {
				const float4 g = wo0 + j < d.resultWidth ? *reinterpret_cast<const float4*>( diff + j * d.channels )
					: make_float4( 0.f, 0.f, 0.f, 0.f );
#pragma unroll
				for( int kh = 0; kh < 3; ++kh ) {
#pragma unroll
					for( int kw = 0; kw < 3; ++kw ) {
						sums[kh * 3 + kw] = CChanVec<4>::fma( rows[kh][j * STRIDE + kw], g, sums[kh * 3 + kw] );
					}
				}
				sums[9].x += g.x; sums[9].y += g.y; sums[9].z += g.z; sums[9].w += g.w;
			}
#pragma unroll
			for( int r = 0; r < Keep; ++r ) {
#pragma unroll
				for( int j = 0; j < NC; ++j ) {
					rows[r][j] = rows[r + STRIDE][j];
				}
			}
			hi += STRIDE;
			diff += diffRow;
		}
		if( PARTIALS ) {
#pragma unroll
			for( int k = 0; k < Sums; ++k ) {
				kept[k].x += sums[k].x; kept[k].y += sums[k].y; kept[k].z += sums[k].z; kept[k].w += sums[k].w;
			}
		} else {
#pragma unroll
			for( int k = 0; k < Sums; ++k ) {
				atomicAdd( &table[( k * 4 + 0 ) * tableWidth + group], sums[k].x );
				atomicAdd( &table[( k * 4 + 1 ) * tableWidth + group], sums[k].y );
				atomicAdd( &table[( k * 4 + 2 ) * tableWidth + group], sums[k].z );
				atomicAdd( &table[( k * 4 + 3 ) * tableWidth + group], sums[k].w );
			}
		}
	}
	if( PARTIALS ) {
		// thread tid = sub * cg + group: every thread its column, then the threads below cg add their group's columns up
#pragma unroll
		for( int k = 0; k < Sums; ++k ) {
			table[( k * 4 + 0 ) * tableWidth + threadIdx.x] = kept[k].x;
			table[( k * 4 + 1 ) * tableWidth + threadIdx.x] = kept[k].y;
			table[( k * 4 + 2 ) * tableWidth + threadIdx.x] = kept[k].z;
			table[( k * 4 + 3 ) * tableWidth + threadIdx.x] = kept[k].w;
		}
		__syncthreads();
		float* const mine = partials + static_cast<long long>( blockIdx.x ) * ( Sums * 4 * cg );
		for( int idx = threadIdx.x; idx < Sums * 4 * cg; idx += blockDim.x ) {
			const int k4 = idx / cg;
			const int group = idx - k4 * cg;
			float v = 0.f;
			for( int at = group; at < tableWidth; at += cg ) {
				v += table[k4 * tableWidth + at];
			}
			mine[idx] = v;
		}
		return;
	}
	__syncthreads();
	for( int idx = threadIdx.x; idx < Sums * 4 * tableWidth; idx += blockDim.x ) {
		const int k4 = idx / tableWidth;
		const int group = idx - k4 * tableWidth;
		const int channel = group * 4 + ( k4 & 3 );
		const float v = table[idx];
		if( k4 < 36 ) {
			unsafeAtomicAdd( filterDiff + ( k4 >> 2 ) * d.channels + channel, v );
		} else if( freeTermDiff != nullptr ) {
			unsafeAtomicAdd( freeTermDiff + channel, v );
		}
	}
}

// Entry k4 * cg + group of every workgroup's row: tap k4 / 4 ( 9: the free term ) of channel 4 group + k4 % 4. A workgroup
// adds up 16 entries: 16 threads per entry take every 16th row with eight sums of their own in flight, then meet in LDS.
__global__ __launch_bounds__( 256 )
void sumLearnPartialsKernel( const float* partials, int rows, int cg, int channels, float* filterDiff, float* freeTermDiff )
{
	__shared__ float meet[16][17];
	const int entries = 40 * cg; // ( a multiple of 8 )
	const int column = threadIdx.x & 15, lane = threadIdx.x >> 4;
	const int idx = blockIdx.x * 16 + column;
	float sums[8] = { 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f };
	if( idx < entries ) {
		int r = lane;
		for( ; r + 7 * 16 < rows; r += 8 * 16 ) {
#pragma unroll
			for( int u = 0; u < 8; ++u ) {
				sums[u] += partials[static_cast<long long>( r + u * 16 ) * entries + idx];
			}
		}
		for( int u = 0; r < rows; r += 16, ++u ) {
			sums[u & 7] += partials[static_cast<long long>( r ) * entries + idx];
		}
	}
	meet[lane][column] = ( ( sums[0] + sums[1] ) + ( sums[2] + sums[3] ) ) + ( ( sums[4] + sums[5] ) + ( sums[6] + sums[7] ) );
	__syncthreads();
	if( lane == 0 && idx < entries ) {
		float v = 0.f;
#pragma unroll
		for( int l = 0; l < 16; ++l ) {
			v += meet[l][column];
		}
		const int k4 = idx / cg;
		const int channel = ( idx - k4 * cg ) * 4 + ( k4 & 3 );
		if( k4 < 36 ) {
			filterDiff[( k4 >> 2 ) * channels + channel] += v;
		} else if( freeTermDiff != nullptr ) {
			freeTermDiff[channel] += v;
		}
	}
}

// Gradient of the channelwise convolution by its filter (and free term): sums over every output pixel of the batch.
// A workgroup owns a block of GROUPS channel groups and a slice of the output pixels; its 256 / GROUPS pixel lanes keep
// the TAPS + 1 sums of their channel group in registers, meet in LDS and leave with one atomic add per sum.
// TAPS == 0: any filter size, one tap per pass over the slice.
template<int VECW, int TAPS>
__global__ __launch_bounds__( 256 )
void channelwiseConvLearnKernel( const nhConvDesc d, const float* input, const float* outputDiff, float* filterDiff,
	float* freeTermDiff, int groups, int groupBlocks, long long pixelsPerSlice )
{
	typedef CChanVec<VECW> V;
	typedef CChanAtomic<VECW> At;
	typedef typename V::Type T;
	constexpr int Sums = ( TAPS > 0 ? TAPS : 1 ) + 1;
	__shared__ T meet[256];
	const int lanes = 256 / groups;
	const int group = threadIdx.x % groups;
	const int lane = threadIdx.x / groups;
	const int cgTotal = d.channels / VECW;
	const int cgIndex = ( blockIdx.x % groupBlocks ) * groups + group;
	const bool active = cgIndex < cgTotal && lane < lanes;
	const int c = cgIndex * VECW;
	const long long slice = blockIdx.x / groupBlocks;
	const long long pixels = static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth;
	const long long first = slice * pixelsPerSlice;
	const long long last = min( first + pixelsPerSlice, pixels );
	const int taps = d.filterHeight * d.filterWidth;
	const int passes = TAPS > 0 ? 1 : taps;
	for( int pass = 0; pass < passes; ++pass ) {
		T sums[Sums];
#pragma unroll
		for( int i = 0; i < Sums; ++i ) {
			sums[i] = V::zero();
		}
		if( active ) {
			for( long long pixel = first + lane; pixel < last; pixel += lanes ) {
				const int wo = static_cast<int>( pixel % d.resultWidth );
				const long long t = pixel / d.resultWidth;
				const int ho = static_cast<int>( t % d.resultHeight );
				const long long n = t / d.resultHeight;
				const T g = V::load( outputDiff + pixel * d.channels + c );
				sums[Sums - 1] = At::sum( sums[Sums - 1], g );
				const float* image = input + n * d.height * d.width * d.channels + c;
				const int hi0 = ho * d.strideHeight - d.paddingHeight;
				const int wi0 = wo * d.strideWidth - d.paddingWidth;
				if( TAPS > 0 ) {
#pragma unroll
					for( int tap = 0; tap < ( TAPS > 0 ? TAPS : 1 ); ++tap ) {
						const int hi = hi0 + tap / 3, wi = wi0 + tap % 3; // TAPS == 9: the 3x3 filter
						if( hi >= 0 && hi < d.height && wi >= 0 && wi < d.width ) {
							sums[tap] = V::fma( V::load( image + ( static_cast<long long>( hi ) * d.width + wi ) * d.channels ), g, sums[tap] );
						}
					}
				} else {
					const int hi = hi0 + pass / d.filterWidth, wi = wi0 + pass % d.filterWidth;
					if( hi >= 0 && hi < d.height && wi >= 0 && wi < d.width ) {
						sums[0] = V::fma( V::load( image + ( static_cast<long long>( hi ) * d.width + wi ) * d.channels ), g, sums[0] );
					}
				}
			}
		}
		// the lanes of a channel group meet: lane 0 adds up and leaves
#pragma unroll
		for( int i = 0; i < Sums; ++i ) {
			__syncthreads();
			meet[threadIdx.x] = sums[i];
			__syncthreads();
			if( active && lane == 0 ) {
				T total = meet[group];
				for( int l = 1; l < lanes; ++l ) {
					total = At::sum( total, meet[l * groups + group] );
				}
				if( i < Sums - 1 ) {
					At::add( filterDiff + ( ( TAPS > 0 ? i : pass ) ) * d.channels + c, total );
				} else if( freeTermDiff != nullptr && pass == 0 ) {
					At::add( freeTermDiff + c, total );
				}
			}
		}
	}
}

// out[b][pixel][c] = act( in[b][pixel][c] * scale[b][c] ): the squeeze-and-excite gate of a MobileNetV3 block
template<int VECW>
__global__ __launch_bounds__( 256 )
void scaleChannelsKernel( const float* in, const float* scale, float* out, int pixelsPerImage, int channels, long long totalItems,
	const CFusedActivation actAsGiven )
{
	const CFusedActivation act = withParam( actAsGiven );
	typedef CChanVec<VECW> V;
	const int cg = channels / VECW;
	const long long perImage = static_cast<long long>( pixelsPerImage ) * cg;
	for( long long item = blockIdx.x * 256LL + threadIdx.x; item < totalItems; item += static_cast<long long>( gridDim.x ) * 256 ) {
		const int c = static_cast<int>( item % cg ) * VECW;
		const long long b = item / perImage;
		const typename V::Type v = V::fma( V::load( in + item * VECW ), V::load( scale + b * channels + c ), V::zero() );
		V::store( out + item * VECW, V::activate( v, act ) );
	}
}

// to[i0..i7] = from[the same index with 0 where from's dimension is 1]; dimension 7 is the additional width
struct CBroadcastShape {
	int ToDims[8];
	int FromStrides[8]; // 0 along broadcast dimensions
};

__global__ __launch_bounds__( 256 )
void broadcastCopyKernel( unsigned* to, const unsigned* from, const CBroadcastShape shape, long long total )
{
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		long long rest = i;
		long long source = 0;
#pragma unroll
		for( int d = 7; d >= 0; --d ) {
			const int index = static_cast<int>( rest % shape.ToDims[d] );
			rest /= shape.ToDims[d];
			source += static_cast<long long>( index ) * shape.FromStrides[d];
		}
		to[i] = from[source];
	}
}

// Dropout with the mask of the reference's CPU engine: the counter-based generator of src/CPU/CpuRandom.h (ten rounds of
// Philox 4x32 on the counter { n, 0, seed ^ 0xBADFACE, seed ^ 0xBADBEEF }, key { seed, seed ^ 0xBADF00D }), four mask
// values per counter value n, kept where the 32-bit value is <= threshold. Being counter-based it needs no state: every
// thread computes the word of its own mask element.
__device__ __forceinline__ unsigned dropoutWord( unsigned generation, int lane, unsigned seed )
{
	unsigned c0 = generation, c1 = 0, c2 = seed ^ 0xBADFACEu, c3 = seed ^ 0xBADBEEFu;
	unsigned k0 = seed, k1 = seed ^ 0xBADF00Du;
#pragma unroll
	for( int round = 0; round < 10; ++round ) {
		const unsigned long long first = 0xD2511F53ull * c0;
		const unsigned long long second = 0xCD9E8D57ull * c2;
		const unsigned n0 = static_cast<unsigned>( second >> 32 ) ^ c1 ^ k0;
		const unsigned n1 = static_cast<unsigned>( second );
		const unsigned n2 = static_cast<unsigned>( first >> 32 ) ^ c3 ^ k1;
		const unsigned n3 = static_cast<unsigned>( first );
		c0 = n0; c1 = n1; c2 = n2; c3 = n3;
		k0 += 0x9E3779B9u;
		k1 += 0xBB67AE85u;
	}
	return lane == 0 ? c0 : ( lane == 1 ? c1 : ( lane == 2 ? c2 : c3 ) );
}

// Mask layout (src/CPU/CpuMathEngineDnnDropout.cpp:33-96). Plain: one mask of batchWidth * objectSize values, shared by
// the batchLength outer slices. Spatial: one value per ( object of the batch width, channel ), shared by every pixel and
// by the outer slices; the generator runs on from object to object, ceil( channels / 4 ) counter values each.
__global__ __launch_bounds__( 256 )
void dropoutKernel( const float* in, float* out, long long total, int maskSize, int objectSize, int channels, int batchWidth,
	int spatial, unsigned seed, unsigned threshold, float value )
{
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		unsigned generation;
		int lane;
		if( spatial ) {
			const int c = static_cast<int>( i % channels );
			const int object = static_cast<int>( ( i / objectSize ) % batchWidth );
			generation = static_cast<unsigned>( object ) * ( ( channels + 3 ) / 4 ) + c / 4;
			lane = c & 3;
		} else {
			const int m = static_cast<int>( i % maskSize );
			generation = m / 4;
			lane = m & 3;
		}
		out[i] = dropoutWord( generation, lane, seed ) <= threshold ? in[i] * value : in[i] * 0.f;
	}
}

// VectorFillBernoulli with the same generator ( src/CPU/CpuMathEngineVectorMath.cpp:267-284 ): element i takes word i % 4 of
// counter value i / 4.
__global__ __launch_bounds__( 256 )
void fillBernoulliKernel( float* result, int n, unsigned seed, unsigned threshold, float value )
{
	const int i = blockIdx.x * 256 + threadIdx.x;
	if( i < n ) {
		result[i] = dropoutWord( static_cast<unsigned>( i ) / 4, i & 3, seed ) <= threshold ? value : 0.f;
	}
}

__global__ void addTwoVectorsKernel( const float* a, const float* b, float* out, int n )
{
	const int i = blockIdx.x * 256 + threadIdx.x;
	if( i < n ) {
		out[i] = ( a != nullptr ? a[i] : 0.f ) + ( b != nullptr ? b[i] : 0.f );
	}
}

} // namespace nh

using namespace nh;

extern "C" int nhInitPooling( nhPoolingDesc* d );

// ---- bookkeeping of the one-launch LSTM ------------------------------------------------------------------------
// Per ( device, stream ): one word of pinned host memory that a launch on that stream sets when its bounded wait
// trips. The synchronising entry points read the word of THEIR stream once it has drained, so a give-up is reported to
// whoever waits for the stream it happened on, once, and to nobody else; no copy, no other stream is touched.
// Per device: the event of the last one-launch LSTM. The kernel needs all its workgroups resident together; two such
// grids from different streams could each hold half of the device and starve one another until their waits expire.
// A launch on another stream is therefore ordered behind the previous one through that event ( a wait on the device,
// the host does not block ).
namespace nh {

struct CSequenceStream {
	unsigned* GaveUp = nullptr; // pinned host memory, device-visible
	bool Launched = false;      // a one-launch LSTM was issued since the word was last looked at
};

// `Last` is the one-launch LSTM issued last on the device ( not counting partners ), `Older` the one in front of it. Each
// may have a partner that runs beside it on a side stream, with a completion event of its own. A launch is ordered
// behind Last and Last's partner; a partner behind Older and Older's partner. Generation counts the launches that are
// not partners: a second nhLstm call may only become the partner of the launch it follows on its stream while that
// launch is still the device's last one, i.e. while no other stream, thread or engine has issued one in between ( such
// a launch waits for Last only: it would run beside the partner, and it may be a whole-device grid ).
struct CSequenceDevice {
	hipEvent_t LastDone = nullptr, LastPartnerDone = nullptr;
	hipEvent_t OlderDone = nullptr, OlderPartnerDone = nullptr;
	bool Any = false, AnyLastPartner = false, AnyOlder = false, AnyOlderPartner = false;
	hipStream_t LastStream = nullptr;
	unsigned long long Generation = 0;
};

// Two one-launch LSTMs side by side ( nhStreamOverlapLstm ): the two directions of a bidirectional layer read the same
// input and write different outputs, arrive as two nhLstm calls one behind the other, and each keeps its cell state for
// itself; in stream order the second waits for the first and the device is half idle. On a stream that has asked for it
// a one-launch LSTM takes a grid of at most half the compute units, and a second nhLstm that follows it directly ( nothing
// else was enqueued through this library in between ) and touches none of its memory runs on a side stream: the side
// stream waits for what was in front of the first, the main stream waits for the side stream right behind the first, so
// whatever is enqueued later, through this library or not, is ordered behind both.
struct CByteRange {
	const char* Lo = nullptr;
	const char* Hi = nullptr;
};

struct CLstmOverlap {
	bool Enabled = false;
	hipStream_t Side = nullptr;
	hipEvent_t Before = nullptr;   // recorded on the main stream in front of a one-launch LSTM
	hipEvent_t SideDone = nullptr; // recorded on the side stream behind its LSTM
	bool LastWasLstm = false;      // that LSTM was the last thing enqueued on the main stream
	unsigned long long Generation = 0; // ... and this was the device's launch count right behind it
	CByteRange Written[3];         // what it writes: results, workspace
	CByteRange Read[4];            // what it reads: input, initial states ( the weights are constant )
};

static std::mutex sequenceLock;
static std::map<std::pair<int, hipStream_t>, CSequenceStream>& sequenceStreams()
{
	static std::map<std::pair<int, hipStream_t>, CSequenceStream> streams;
	return streams;
}
static std::map<int, CSequenceDevice>& sequenceDevices()
{
	static std::map<int, CSequenceDevice> devices;
	return devices;
}
static std::map<std::pair<int, hipStream_t>, CLstmOverlap>& lstmOverlaps()
{
	static std::map<std::pair<int, hipStream_t>, CLstmOverlap> overlaps;
	return overlaps;
}

int overlapLstmStreams = 0;
int lstmPartnersAwaited = 0;

// ( under sequenceLock ) the stream's last launch is / is no longer a one-launch LSTM that a partner may join; the count
// of such streams is what every entry point looks at before it takes the lock
static void setLastWasLstm( CLstmOverlap& o, bool value )
{
	if( o.LastWasLstm != value ) {
		o.LastWasLstm = value;
		if( value ) {
			__atomic_fetch_add( &lstmPartnersAwaited, 1, __ATOMIC_RELAXED );
		} else {
			__atomic_fetch_sub( &lstmPartnersAwaited, 1, __ATOMIC_RELAXED );
		}
	}
}

// something is being enqueued on `stream` through this library: a one-launch LSTM on it has no partner any more
void noteStreamUse( hipStream_t stream )
{
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return;
	}
	std::lock_guard<std::mutex> guard( sequenceLock );
	auto found = lstmOverlaps().find( std::make_pair( device, stream ) );
	if( found != lstmOverlaps().end() ) {
		setLastWasLstm( found->second, false );
	}
}

static bool rangesMeet( const CByteRange& a, const CByteRange& b )
{
	return a.Lo != nullptr && b.Lo != nullptr && a.Lo < b.Hi && b.Lo < a.Hi;
}

// Called by the synchronising entry points once `stream` has drained: a one-launch LSTM of this stream whose bounded
// wait tripped has produced garbage, and that must not pass silently.
int checkSequenceGiveUps( hipStream_t stream )
{
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return NH_OK;
	}
	std::lock_guard<std::mutex> guard( sequenceLock );
	auto& streams = sequenceStreams();
	bool gaveUp = false;
	// the stream's own launches, and those of its side stream ( the main stream has waited for them )
	hipStream_t both[2] = { stream, nullptr };
	auto overlap = lstmOverlaps().find( std::make_pair( device, stream ) );
	if( overlap != lstmOverlaps().end() ) {
		both[1] = overlap->second.Side;
	}
	for( int i = 0; i < 2; ++i ) {
		if( i == 1 && both[1] == nullptr ) {
			break;
		}
		auto found = streams.find( std::make_pair( device, both[i] ) );
		if( found == streams.end() || !found->second.Launched ) {
			continue;
		}
		found->second.Launched = false;
		volatile unsigned* word = found->second.GaveUp;
		if( *word != 0 ) {
			*word = 0;
			gaveUp = true;
			if( getenv( "NH_LSTM_SPIN_LIMIT" ) == nullptr ) { // ( not when a test forces the give-up through the spin limit )
				__atomic_store_n( &xcdLayoutFailed, 1, __ATOMIC_RELAXED ); // ( whichever layout it was: the plain one asks less )
			}
		}
	}
	if( !gaveUp ) {
		return NH_OK;
	}
	setLastError( "nhLstm: a one-launch LSTM on this stream gave up waiting for the previous step (its grid was not "
		"resident as a whole, or the spin limit is too low): its output is invalid" );
	return NH_ERR_HIP;
}

// the stream is going away ( it has been drained )
void releaseSequenceStream( hipStream_t stream )
{
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return;
	}
	std::lock_guard<std::mutex> guard( sequenceLock );
	auto& streams = sequenceStreams();
	auto found = streams.find( std::make_pair( device, stream ) );
	if( found != streams.end() ) {
		( void )hipHostFree( found->second.GaveUp );
		streams.erase( found );
	}
	auto dev = sequenceDevices().find( device );
	if( dev != sequenceDevices().end() && dev->second.LastStream == stream ) {
		// drained: nothing of it is in flight, nor anything it had waited for
		dev->second.Any = dev->second.AnyLastPartner = false;
		dev->second.AnyOlder = dev->second.AnyOlderPartner = false;
	}
	auto overlap = lstmOverlaps().find( std::make_pair( device, stream ) );
	if( overlap != lstmOverlaps().end() ) {
		CLstmOverlap& o = overlap->second;
		if( o.Side != nullptr ) {
			auto side = streams.find( std::make_pair( device, o.Side ) );
			if( side != streams.end() ) {
				( void )hipHostFree( side->second.GaveUp );
				streams.erase( side );
			}
			releaseSliceScratch( o.Side, true );
			( void )hipStreamDestroy( o.Side );
			( void )hipEventDestroy( o.Before );
			( void )hipEventDestroy( o.SideDone );
		}
		if( o.Enabled ) {
			__atomic_fetch_sub( &overlapLstmStreams, 1, __ATOMIC_RELAXED );
		}
		setLastWasLstm( o, false );
		lstmOverlaps().erase( overlap );
	}
}

} // namespace nh

// ---- whole-sequence LSTM launch ------------------------------------------------------------------------------

// The shapes of the one-launch kernels: Rows sequences x ( 4 * Blocks ) hidden units per workgroup of Waves wavefronts.
// ByXcd: lstmRowsKernel ( the layout by XCDs ), otherwise lstmSequenceKernel.
struct CLstmSeqShape {
	int Rows, Blocks, Waves;
	bool ByXcd;
	const void* Kernel;
	void ( *Launch )( hipStream_t, unsigned, size_t, const CLstmSeqArgs& );
};

template<int RB, int CB, int W>
static void launchSeqShape( hipStream_t stream, unsigned groups, size_t lds, const CLstmSeqArgs& a )
{
	hipLaunchKernelGGL( ( lstmSequenceKernel<RB, CB, W> ), dim3( groups ), dim3( 64 * W ), lds, stream, a );
}

template<int PW>
static void launchRowsShape( hipStream_t stream, unsigned groups, size_t, const CLstmSeqArgs& a )
{
	hipLaunchKernelGGL( ( lstmRowsKernel<PW> ), dim3( groups ), dim3( 64 * ( PW + 2 ) ), 0, stream, a );
}

#define NH_SEQ_SHAPE( RB, CB, W ) { RB, CB, W, false, reinterpret_cast<const void*>( &lstmSequenceKernel<RB, CB, W> ), &launchSeqShape<RB, CB, W> }
#define NH_ROWS_SHAPE( PW ) { RowsKernelRows, RowsKernelUnits / SeqUnits, PW + 2, true, reinterpret_cast<const void*>( &lstmRowsKernel<PW> ), &launchRowsShape<PW> }
// in order of preference (measured at 64 sequences x 256 units, 128 steps: 433 / 445 / 515 us for the first three
// lstmSequenceKernel shapes; a v_mfma_f32_16x16x4_f32 issues every 64 clocks, so the narrow workgroup has the shortest
// product phase)
static const CLstmSeqShape lstmSeqShapes[] = {
	NH_ROWS_SHAPE( 1 ), NH_ROWS_SHAPE( 2 ), NH_ROWS_SHAPE( 4 ), NH_ROWS_SHAPE( 8 ),
	NH_SEQ_SHAPE( 16, 1, 8 ), NH_SEQ_SHAPE( 16, 2, 8 ), NH_SEQ_SHAPE( 16, 4, 8 ), NH_SEQ_SHAPE( 16, 2, 16 ), NH_SEQ_SHAPE( 16, 4, 16 ),
	NH_SEQ_SHAPE( 32, 2, 16 ) };
constexpr size_t LdsLimit = 160 * 1024 - 256; // dynamic part; the kernel also has a static word

static size_t lstmSequenceLds( int H, const CLstmSeqShape& shape )
{
	if( shape.ByXcd ) {
		return 0; // ( its LDS is static )
	}
	const size_t cols = 16 * static_cast<size_t>( shape.Blocks );
	return ( ( cols + shape.Rows ) * ( H + 4 ) + 4 + static_cast<size_t>( shape.Waves ) * shape.Rows * ( cols + 4 ) ) * sizeof( float );
}

// Can the shape's kernel run this size at all ( the grid aside )?
static bool lstmShapeTakes( int H, const CLstmSeqShape& shape )
{
	if( shape.ByXcd ) {
		return H == 64 * ( shape.Waves - 2 ); // one product wavefront per 64 k
	}
	if( H % ( SeqUnits * shape.Blocks ) != 0 || lstmSequenceLds( H, shape ) > LdsLimit ) {
		return false;
	}
	const int batch = 16; // lstmSequenceKernel's Batch: its loaders cover the tile in one batch
	return static_cast<long long>( shape.Rows ) * H <= static_cast<long long>( batch ) * ( shape.Waves / 2 ) * 64;
}

// The first shape whose grid fits the device; null = none does.
static const CLstmSeqShape* lstmSequenceShape( int H, int B, bool halfDevice = false )
{
	static int computeUnits = 0; // the engine drives one device per process
	static bool ldsRaised = false;
	if( computeUnits == 0 ) {
		int device = 0, count = 0;
		if( hipGetDevice( &device ) != hipSuccess
			|| hipDeviceGetAttribute( &count, hipDeviceAttributeMultiprocessorCount, device ) != hipSuccess || count <= 0 )
		{
			( void )hipGetLastError();
			return nullptr;
		}
		computeUnits = count;
	}
	if( !ldsRaised ) {
		// beyond 64 KB of dynamic LDS a kernel has to ask
		for( const CLstmSeqShape& shape : lstmSeqShapes ) {
			if( shape.ByXcd ) {
				continue;
			}
			const hipError_t err = hipFuncSetAttribute( shape.Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>( LdsLimit ) );
			if( err != hipSuccess ) {
				setLastError( "lstm: hipFuncSetAttribute failed: %s", hipGetErrorString( err ) );
				( void )hipGetLastError();
				return nullptr;
			}
		}
		ldsRaised = true;
	}
	for( const CLstmSeqShape& shape : lstmSeqShapes ) {
		const size_t lds = lstmSequenceLds( H, shape );
		if( shape.ByXcd || !lstmShapeTakes( H, shape ) ) {
			continue;
		}
		int perUnit = 0;
		const hipError_t err = hipOccupancyMaxActiveBlocksPerMultiprocessor( &perUnit, shape.Kernel, 64 * shape.Waves, lds );
		if( err != hipSuccess ) {
			setLastError( "lstm: occupancy query failed: %s", hipGetErrorString( err ) );
			( void )hipGetLastError();
			continue;
		}
		// one workgroup per compute unit is what the dispatcher certainly places side by side on an otherwise idle
		// device; the occupancy figure only confirms that one fits
		const long long groups = static_cast<long long>( H / ( SeqUnits * shape.Blocks ) ) * ceilDiv( B, shape.Rows );
		if( perUnit >= 1 && groups <= ( halfDevice ? computeUnits / 2 : computeUnits ) ) {
			return &shape;
		}
	}
	// ( no shape of half the device: the whole one, and no partner beside it )
	return halfDevice ? lstmSequenceShape( H, B, false ) : nullptr;
}

// How many XCDs the layout by XCDs needs for B sequences of H units: an XCD's 32 workgroups hold 4 sequences x 32 units each.
static int lstmXcdsNeeded( int H, int B )
{
	const int rowsPerXcd = RowsKernelRows * ( 32 / ( H / RowsKernelUnits ) );
	return ceilDiv( B, rowsPerXcd );
}

// The shape of the layout by XCDs ( lstmRowsKernel ) if the device has 8 XCDs of 32 compute units and the sequences fit
// the XCDs the launch may use ( all eight, or four when two launches share the device ); null: the plain layout.
static const CLstmSeqShape* lstmXcdShape( int H, int B, bool halfDevice )
{
	static const bool enabled = []() {
		const char* env = getenv( "NH_LSTM_XCD_LAYOUT" ); // "0" switches the layout off ( measurements )
		return env == nullptr || env[0] != '0';
	}();
	int device = 0, units = 0;
	if( !enabled || __atomic_load_n( &xcdLayoutFailed, __ATOMIC_RELAXED ) != 0 || hipGetDevice( &device ) != hipSuccess
		|| hipDeviceGetAttribute( &units, hipDeviceAttributeMultiprocessorCount, device ) != hipSuccess || units != 256 )
	{
		( void )hipGetLastError();
		return nullptr;
	}
	for( const CLstmSeqShape& shape : lstmSeqShapes ) {
		if( !shape.ByXcd || !lstmShapeTakes( H, shape ) ) {
			continue;
		}
		int perUnit = 0;
		if( lstmXcdsNeeded( H, B ) > ( halfDevice ? 4 : 8 )
			|| hipOccupancyMaxActiveBlocksPerMultiprocessor( &perUnit, shape.Kernel, 64 * shape.Waves, 0 ) != hipSuccess || perUnit < 1 )
		{
			( void )hipGetLastError();
			return nullptr;
		}
		return &shape;
	}
	return nullptr;
}

static bool lstmSequenceFits( int H, int B, const float* wRec, const float* c0, const float* h0, const float* hOut )
{
	( void )c0;
	return H % 16 == 0 && isAligned16( wRec ) && isAligned16( hOut ) && ( h0 == nullptr || isAligned16( h0 ) )
		&& lstmSequenceShape( H, B ) != nullptr;
}

// Rounds of loads a wavefront makes for one step's values before it gives up (a round is a trip to the device-level
// coherence point: about a microsecond).
// NH_LSTM_SPIN_LIMIT overrides it; tests use a tiny value to drive the give-up path from the host.
static unsigned lstmSpinLimit()
{
	const char* env = getenv( "NH_LSTM_SPIN_LIMIT" );
	if( env != nullptr && *env != 0 ) {
		return static_cast<unsigned>( strtoul( env, nullptr, 10 ) );
	}
	return 4u << 20;
}

// false: the one-launch path cannot be taken for this stream right now ( it is being captured into a graph, whose
// replays nothing here could order ); the caller runs the launch-per-step kernels instead
static bool lstmSequenceAllowed( hipStream_t stream )
{
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	return capture == hipStreamCaptureStatusNone;
}

// halfDevice: a grid of at most half the compute units if there is such a shape ( *tookHalf says whether ).
// partnerOf: not null = this launch, on a side stream, wants to run beside the launch that made the device's count
// *partnerOf; it does if that launch is still the device's last one and has no partner yet ( *ranBeside ), otherwise it
// is ordered like any other launch. *generation receives the device's count behind a launch that is not a partner.
static int launchLstmSequence( hipStream_t stream, CLstmSeqArgs a, bool halfDevice = false, const unsigned long long* partnerOf = nullptr,
	bool* tookHalf = nullptr, unsigned long long* generation = nullptr, bool* ranBeside = nullptr )
{
	const CLstmSeqShape* xcdShape = lstmXcdShape( a.H, a.B, halfDevice );
	const CLstmSeqShape* shape = xcdShape != nullptr ? xcdShape : lstmSequenceShape( a.H, a.B, halfDevice );
	NH_REQUIRE( shape != nullptr );
	int device = 0;
	NH_HIP( hipGetDevice( &device ) );
	int computeUnits = 0;
	NH_HIP( hipDeviceGetAttribute( &computeUnits, hipDeviceAttributeMultiprocessorCount, device ) );
	const long long shapeGroups = static_cast<long long>( a.H / ( SeqUnits * shape->Blocks ) ) * ceilDiv( a.B, shape->Rows );
	// ( in the layout by XCDs a launch holds as many XCDs as it has blocks of sequences )
	const bool isHalf = xcdShape != nullptr ? lstmXcdsNeeded( a.H, a.B ) <= 4 : shapeGroups <= computeUnits / 2;
	a.XcdLayout = xcdShape != nullptr ? 1 : 0;
	a.RowBlocks = xcdShape != nullptr ? lstmXcdsNeeded( a.H, a.B ) : ceilDiv( a.B, shape->Rows ); // ( by XCDs: the XCDs in use )
	if( tookHalf != nullptr ) {
		*tookHalf = isHalf;
	}
	std::lock_guard<std::mutex> guard( sequenceLock );
	CSequenceStream& own = sequenceStreams()[std::make_pair( device, stream )];
	if( own.GaveUp == nullptr ) {
		void* word = nullptr;
		NH_HIP( hipHostMalloc( &word, 64, hipHostMallocDefault ) );
		own.GaveUp = static_cast<unsigned*>( word );
		*own.GaveUp = 0;
	}
	CSequenceDevice& dev = sequenceDevices()[device];
	if( dev.LastDone == nullptr ) {
		NH_HIP( hipEventCreateWithFlags( &dev.LastDone, hipEventDisableTiming ) );
		NH_HIP( hipEventCreateWithFlags( &dev.OlderDone, hipEventDisableTiming ) );
		NH_HIP( hipEventCreateWithFlags( &dev.LastPartnerDone, hipEventDisableTiming ) );
		NH_HIP( hipEventCreateWithFlags( &dev.OlderPartnerDone, hipEventDisableTiming ) );
	}
	const bool partner = partnerOf != nullptr && isHalf && dev.Any && dev.Generation == *partnerOf && !dev.AnyLastPartner;
	if( ranBeside != nullptr ) {
		*ranBeside = partner;
	}
	if( partner ) {
		// beside the one issued last, behind the one in front of that and its partner
		if( dev.AnyOlder ) {
			NH_HIP( hipStreamWaitEvent( stream, dev.OlderDone, 0 ) );
		}
		if( dev.AnyOlderPartner ) {
			NH_HIP( hipStreamWaitEvent( stream, dev.OlderPartnerDone, 0 ) );
		}
	} else {
		// behind the one-launch LSTM issued last and its partner, whichever streams they went to ( on the same stream
		// the wait is free )
		if( dev.Any ) {
			NH_HIP( hipStreamWaitEvent( stream, dev.LastDone, 0 ) );
		}
		if( dev.AnyLastPartner ) {
			NH_HIP( hipStreamWaitEvent( stream, dev.LastPartnerDone, 0 ) );
		}
	}
	a.GaveUp = own.GaveUp;
	own.Launched = true;
	// a partner takes the XCDs its partner leaves free
	a.XcdBase = partner ? 4 : 0;
	const unsigned groups = a.XcdLayout != 0 ? 256u
		: static_cast<unsigned>( ( a.H / ( SeqUnits * shape->Blocks ) ) * ceilDiv( a.B, shape->Rows ) );
	// the exchange buffers and the abort word that follows them
	// both sets of exchange buffers, the table of XCDs and the abort word that follow them
	const long long words = 4LL * a.B * a.H + LstmXcdTableWords / 2 + 1;
	hipLaunchKernelGGL( clearWordsKernel, dim3( static_cast<unsigned>( ( words + 1023 ) / 1024 ) ), dim3( 256 ), 0, stream, a.Exchange, words );
	shape->Launch( stream, groups, lstmSequenceLds( a.H, *shape ), a );
	NH_LAUNCH_CHECK();
	if( partner ) {
		NH_HIP( hipEventRecord( dev.LastPartnerDone, stream ) );
		dev.AnyLastPartner = true;
	} else {
		std::swap( dev.LastDone, dev.OlderDone );
		std::swap( dev.LastPartnerDone, dev.OlderPartnerDone );
		dev.AnyOlder = dev.Any;
		dev.AnyOlderPartner = dev.AnyLastPartner;
		NH_HIP( hipEventRecord( dev.LastDone, stream ) );
		dev.LastStream = stream;
		dev.Any = true;
		dev.AnyLastPartner = false;
		++dev.Generation;
		if( generation != nullptr ) {
			*generation = dev.Generation;
		}
	}
	return NH_OK;
}

static int checkPoolingDesc( const nhPoolingDesc* d )
{
	NH_REQUIRE( d != nullptr );
	nhPoolingDesc check = *d;
	const int rc = nhInitPooling( &check );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( check.resultHeight == d->resultHeight && check.resultWidth == d->resultWidth );
	NH_REQUIRE( static_cast<long long>( d->height ) * d->width * d->channels <= 0x7fffffffLL );
	return NH_OK;
}

// Splits resultHeight into row chunks, one per work item: as tall as possible (the taller the strip, the fewer
// halo rows are read twice) while the launch still has `wantedBlocks` workgroups, several rounds of the 256
// compute units at the kernel's occupancy.
static void chooseRowChunks( long long itemsPerChunk, int resultHeight, int minRows, int wantedBlocks, int* rowChunks, int* rowsPerItem )
{
	const long long blocksPerChunk = ( itemsPerChunk + 255 ) / 256;
	const long long wanted = ( wantedBlocks + blocksPerChunk - 1 ) / blocksPerChunk;
	const long long maxChunks = ( resultHeight + minRows - 1 ) / minRows;
	const int chunks = static_cast<int>( wanted < maxChunks ? wanted : maxChunks );
	const int rows = ( resultHeight + chunks - 1 ) / chunks;
	*rowsPerItem = rows;
	*rowChunks = ( resultHeight + rows - 1 ) / rows;
}

template<bool MEAN>
static int poolingImpl( nhStream s, const nhPoolingDesc* d, const float* source, float* result )
{
	const bool vec = d->channels % 4 == 0 && isAligned16( source ) && isAligned16( result );
	const long long perRow = static_cast<long long>( d->batch ) * d->resultWidth * ( vec ? d->channels / 4 : d->channels );
	if( perRow == 0 ) {
		return NH_OK;
	}
	int rowChunks = 1, rowsPerItem = 1;
	chooseRowChunks( perRow, d->resultHeight, d->filterHeight > d->strideHeight ? 4 : 1, 8192, &rowChunks, &rowsPerItem );
	const long long items = perRow * rowChunks;
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	const int square = d->filterHeight == d->filterWidth ? d->filterHeight : 0;
	const dim3 grid( static_cast<unsigned>( blocks ) );
	if( vec && square == 2 ) {
		hipLaunchKernelGGL( ( poolingKernel<4, MEAN, 2> ), grid, dim3( 256 ), 0, toStream( s ), *d, source, result, rowChunks, rowsPerItem, items );
	} else if( vec && square == 3 ) {
		hipLaunchKernelGGL( ( poolingKernel<4, MEAN, 3> ), grid, dim3( 256 ), 0, toStream( s ), *d, source, result, rowChunks, rowsPerItem, items );
	} else if( vec ) {
		hipLaunchKernelGGL( ( poolingKernel<4, MEAN, 0> ), grid, dim3( 256 ), 0, toStream( s ), *d, source, result, rowChunks, rowsPerItem, items );
	} else {
		hipLaunchKernelGGL( ( poolingKernel<1, MEAN, 0> ), grid, dim3( 256 ), 0, toStream( s ), *d, source, result, rowChunks, rowsPerItem, items );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// ---- strips of the 3x3 depthwise kernel ------------------------------------------------------------------------
// How wide and how tall the strips of a launch are decides three things at once: how many input rows are read twice
// ( every strip re-reads the two rows above its first output row ), how many bytes the device has in flight ( a wave asks
// for one row of its strip ahead; about 10 MB in flight saturate HBM ), and how evenly the waves fill the device ( waves
// beyond what is resident at once form a second, partly filled round ). Measured on the three large layers of a
// MobileNetV2 at batch 128 with 7 to 56 rows per strip: the estimate below picks strips within 2.5 % of the best of each
// ( 5.5 / 6.05 / 5.6 TB/s ). Strips of more than 30 rows were slower than it says on every shape, hence the last term.
static double stripTimeEstimate( const nhConvDesc& d, int stride, int wpt, int chunks, int residentWaves )
{
	const int rows = ceilDiv( d.resultHeight, chunks );
	const double waves = static_cast<double>( d.batch ) * ceilDiv( d.resultWidth, wpt ) * ( d.channels / 4 ) * chunks / 64.0;
	const int columns = ( wpt - 1 ) * stride + 3;
	const double rounds = ceil( waves / residentWaves );
	const double fill = waves / ( rounds * residentWaves );
	const double inFlight = ( waves < residentWaves ? waves : residentWaves ) * 64.0 * columns * stride * 16.0;
	const double haloRows = static_cast<double>( rows * stride + 2 ) / ( rows * stride );
	const double haloColumns = pow( static_cast<double>( columns ) / ( wpt * stride ), 0.1 ); // mostly served by the L1
	double time = static_cast<double>( d.height ) * d.width * haloRows * haloColumns
		+ static_cast<double>( d.resultHeight ) * d.resultWidth;
	if( inFlight < 10e6 ) {
		time *= 10e6 / inFlight;
	}
	if( rounds > 1 ) {
		time *= 1.0 + 0.5 * ( 1.0 / fill - 1.0 );
	}
	if( rows > 30 ) {
		time /= 0.85;
	}
	return time;
}

static int residentWavesFor( const void* kernel )
{
	static std::mutex lock;
	static std::map<std::pair<int, const void*>, int> known;
	int device = 0;
	( void )hipGetDevice( &device );
	std::lock_guard<std::mutex> guard( lock );
	int& waves = known[std::make_pair( device, kernel )];
	if( waves == 0 ) {
		int perUnit = 0, units = 0;
		if( hipOccupancyMaxActiveBlocksPerMultiprocessor( &perUnit, kernel, 64, 0 ) != hipSuccess
			|| hipDeviceGetAttribute( &units, hipDeviceAttributeMultiprocessorCount, device ) != hipSuccess || perUnit <= 0 || units <= 0 )
		{
			( void )hipGetLastError();
			perUnit = 4;
			units = 256;
		}
		waves = perUnit * units;
	}
	return waves;
}

template<int STRIDE, int WPT, bool STREAM>
static int channelwise3x3Launch( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act, bool flipTaps, int rowChunks )
{
	const int wGroups = ceilDiv( d->resultWidth, WPT );
	const long long perRow = static_cast<long long>( d->batch ) * wGroups * ( d->channels / 4 );
	const int rowsPerItem = ceilDiv( d->resultHeight, rowChunks );
	rowChunks = ceilDiv( d->resultHeight, rowsPerItem );
	const long long items = perRow * rowChunks;
	// workgroups of one wave: the strips need nothing from one another, and single waves spread most evenly
	const unsigned resultBytes = static_cast<unsigned>( static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->channels * 4 );
	const dim3 grid( static_cast<unsigned>( ( items + 63 ) / 64 ) );
	const int flipArg = flipTaps ? 1 : 0;
	auto launch = [&]( auto actOf ) {
		constexpr int Act = decltype( actOf )::value;
		hipLaunchKernelGGL( ( channelwiseConv3x3Kernel<STRIDE, WPT, 1, STREAM, Act> ), grid, dim3( 64 ), 0, toStream( s ), *d, source, filter,
			freeTerm, result, wGroups, rowChunks, rowsPerItem, static_cast<int>( items ), act, flipArg, resultBytes );
	};
	if( act.Type == NH_ACT_RELU ) {
		launch( std::integral_constant<int, NH_ACT_RELU>() );
	} else if( act.Type == NH_ACT_HSWISH ) {
		launch( std::integral_constant<int, NH_ACT_HSWISH>() );
	} else {
		launch( std::integral_constant<int, NH_ACT_NONE>() );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

template<int STRIDE, int WPT>
static int channelwise3x3Impl( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act, bool flipTaps = false )
{
	const long long sourceBytes = static_cast<long long>( d->batch ) * d->height * d->width * d->channels * 4;
	if( sourceBytes < ( 64LL << 20 ) ) {
		// served by the caches: what counts is how many waves work at once, not what is read twice
		const long long perRow = static_cast<long long>( d->batch ) * ceilDiv( d->resultWidth, WPT ) * ( d->channels / 4 );
		int rowChunks = 1, rowsPerItem = 1;
		chooseRowChunks( perRow, d->resultHeight, 4, 3072, &rowChunks, &rowsPerItem );
		return channelwise3x3Launch<STRIDE, WPT, false>( s, d, source, filter, freeTerm, result, act, flipTaps, rowChunks );
	}
	// Strips twice as wide halve the columns read twice but need twice the registers: measured, they pay at stride 2
	// ( 9 columns for 4 output pixels instead of 5 for 2 ) and lose at stride 1.
	constexpr int Widths = STRIDE == 2 ? 2 : 1;
	const int resident[2] = {
		residentWavesFor( reinterpret_cast<const void*>( &channelwiseConv3x3Kernel<STRIDE, WPT, 1, true, NH_ACT_NONE> ) ),
		residentWavesFor( reinterpret_cast<const void*>( &channelwiseConv3x3Kernel<STRIDE, WPT * 2, 1, true, NH_ACT_NONE> ) ) };
	bool wide = false;
	int chunks = 1;
	double best = -1;
	const int mostChunks = ceilDiv( d->resultHeight, 4 );
	for( int w = 0; w < Widths; ++w ) {
		for( int c = 1; c <= mostChunks; ++c ) {
			if( c > 1 && ceilDiv( d->resultHeight, c ) == ceilDiv( d->resultHeight, c - 1 ) ) {
				continue; // the same strip height
			}
			const double time = stripTimeEstimate( *d, STRIDE, w == 0 ? WPT : WPT * 2, c, resident[w] );
			if( best < 0 || time < best ) {
				best = time;
				wide = w != 0;
				chunks = c;
			}
		}
	}
	if( wide ) {
		return channelwise3x3Launch<STRIDE, WPT * 2, true>( s, d, source, filter, freeTerm, result, act, flipTaps, chunks );
	}
	return channelwise3x3Launch<STRIDE, WPT, true>( s, d, source, filter, freeTerm, result, act, flipTaps, chunks );
}

template<int STRIDE, int WPT>
static int channelwiseLearn3x3Impl( nhStream s, const nhConvDesc* d, const float* input, const float* outputDiff,
	float* filterDiff, float* freeTermDiff )
{
	const int wGroups = ceilDiv( d->resultWidth, WPT );
	const long long perRow = static_cast<long long>( d->batch ) * wGroups * ( d->channels / 4 );
	int rowChunks = 1, rowsPerItem = 1;
	// tall strips ( few row chunks ): every chunk re-reads two halo rows and ends with 40 LDS adds per thread
	chooseRowChunks( perRow, d->resultHeight, 4, 256, &rowChunks, &rowsPerItem );
	const int cg = d->channels / 4;
	// with scratch memory: a row of 40 x cg sums per workgroup, added up by a second launch. 512 workgroups, two per compute
	// unit ( every row of a strip is a round trip to memory, so one per unit leaves the memory system idle; measured at
	// 128 / 256 / 384 / 512 / 768 / 1024: 14 x 14 x 384 36 / 26 / 27 / 26 / 31 / 36 us, 56 x 56 x 144 145 / 87 / 104 / 88 / 88 / 95,
	// 112 x 112 x 96 stride 2 191 / 159 / 157 / 140 / 148 / 141; with LDS and global adds instead 64 / 114 / 177 )
	{
		const int threads = cg * ( 256 / cg ); // ( cg <= 256 )
		const long long cap = 512;
		int chunks = 1, rows = 1;
		chooseRowChunks( perRow, d->resultHeight, 4, static_cast<int>( cap ), &chunks, &rows );
		const long long items = perRow * chunks;
		const long long blocks = ( items + threads - 1 ) / threads < cap ? ( items + threads - 1 ) / threads : cap;
		float* partials = nullptr;
		unsigned* counter = nullptr;
		if( streamMeetingPlace( toStream( s ), static_cast<size_t>( blocks ) * 40 * cg, &partials, &counter ) ) {
			hipLaunchKernelGGL( ( channelwiseLearn3x3Kernel<STRIDE, WPT, true> ), dim3( static_cast<unsigned>( blocks ) ), dim3( threads ), 0,
				toStream( s ), *d, input, outputDiff, filterDiff, freeTermDiff, wGroups, chunks, rows, static_cast<int>( items ), partials );
			NH_LAUNCH_CHECK();
			hipLaunchKernelGGL( sumLearnPartialsKernel, dim3( ceilDiv( 40 * cg, 16 ) ), dim3( 256 ), 0, toStream( s ),
				partials, static_cast<int>( blocks ), cg, d->channels, filterDiff, freeTermDiff );
			NH_LAUNCH_CHECK();
			return NH_OK;
		}
	}
	// without ( a stream that is being captured ): LDS adds, then global adds. One workgroup per compute unit: measured
	// best of 64..2048 ( more workgroups bring more global adds, fewer leave compute units idle )
	const long long items = perRow * rowChunks;
	const long long cap = 256;
	const long long blocks = ( items + 255 ) / 256 < cap ? ( items + 255 ) / 256 : cap;
	hipLaunchKernelGGL( ( channelwiseLearn3x3Kernel<STRIDE, WPT, false> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0,
		toStream( s ), *d, input, outputDiff, filterDiff, freeTermDiff, wGroups, rowChunks, rowsPerItem, static_cast<int>( items ), nullptr );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

template<bool MAX>
static int poolingBackwardImpl( nhStream s, const nhPoolingDesc* d, const float* resultDiff, const int* maxIndices,
	float* sourceDiff )
{
	const long long total = static_cast<long long>( d->batch ) * d->height * d->width * d->channels;
	if( total == 0 ) {
		return NH_OK;
	}
	const bool vec = d->channels % 4 == 0 && isAligned16( resultDiff ) && isAligned16( sourceDiff )
		&& ( !MAX || isAligned16( maxIndices ) );
	const long long items = vec ? total / 4 : total;
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( ( poolingBackwardKernel<4, MAX> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, resultDiff, maxIndices, sourceDiff, items );
	} else {
		hipLaunchKernelGGL( ( poolingBackwardKernel<1, MAX> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, resultDiff, maxIndices, sourceDiff, items );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// Expand 1x1 (+act) -> depthwise 3x3, padding 1 (+act) in one launch, the expanded tensor never in memory: for the blocks
// of a MobileNetV2 whose expanded tensor is several times the size of the last-level cache (16 -> 96 channels at
// 112 x 112, 24 -> 144 at 56 x 56, 32 -> 192 at 28 x 28, batch 128) writing it and reading it back is most of the block's
// time. Every wavefront works alone, no barrier anywhere: it owns a patch of PH x PW <= 64 input pixels ( 8 x 8 at
// stride 1 for 6 x 6 output pixels, 7 x 9 at stride 2 for 3 x 4 ), holds them as the operand of two 32 x 32 MFMA blocks
// in registers for the whole launch ( each lane its pixel's channels, fetched with 128-bit buffer loads; pixels
// outside the image are out-of-range offsets ) and walks the expanded channels 32 at a time: multiply by that chunk of
// the expand filter ( its rows straight from memory into the other operand ), add the free term, activate, put zeros
// where the pixel lies outside the image ( the depthwise convolution pads the expanded tensor, not the input ), write
// the 64 x 32 values to the wave's own LDS tile, and sum the nine taps of every output from there, four channels per lane,
// eight lanes per pixel = one 128-byte store per pixel and chunk. A wave's LDS operations complete in order, so the
// tile needs no synchronisation beyond the wave. The patches overlap by two pixels, i.e. the expand product is computed
// 1.8 times ( the matrix pipe is idle otherwise: the reduction is 16 to 32 long ).
namespace nh {

// ( declared in common.h: what a stream that puts calls aside does with a padded image that waited )
int launchPadding( hipStream_t stream, const CPendingPadding& p )
{
	const bool vec = p.Channels % 4 == 0 && isAligned16( p.From ) && isAligned16( p.To );
	const long long items = p.Batch * p.ToHeight * p.ToWidth * ( vec ? p.Channels / 4 : p.Channels );
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( resizeImageKernel<4>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			p.From, p.To, p.Height, p.Width, p.Channels, p.ToHeight, p.ToWidth, p.DeltaLeft, p.DeltaTop, p.Padding, p.DefaultValue, items );
	} else {
		hipLaunchKernelGGL( resizeImageKernel<1>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			p.From, p.To, p.Height, p.Width, p.Channels, p.ToHeight, p.ToWidth, p.DeltaLeft, p.DeltaTop, p.Padding, p.DefaultValue, items );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

bool launchPaddingWithPooling( hipStream_t stream, const CPendingPadding& p, const nhPoolingDesc& d, float* result, int* rc )
{
	if( p.Padding != NH_PAD_CONSTANT || p.Channels % 4 != 0 || !isAligned16( p.From ) || !isAligned16( p.To ) || !isAligned16( result )
		|| d.batch != p.Batch || d.height != p.ToHeight || d.width != p.ToWidth || d.channels != p.Channels
		|| d.filterHeight != 3 || d.filterWidth != 3 || d.strideHeight < 1 || d.strideHeight > 3 || d.strideWidth < 1 || d.strideWidth > 3
		|| d.resultHeight < 1 || d.resultWidth < 1 ) {
		return false;
	}
	// ( the pooled image may lie anywhere but over the two images of the padding )
	const float* padEnd = p.To + p.Batch * p.ToHeight * p.ToWidth * p.Channels;
	const float* fromEnd = p.From + p.Batch * p.Height * p.Width * p.Channels;
	const float* resultEnd = result + static_cast<long long>( d.batch ) * d.resultHeight * d.resultWidth * d.channels;
	if( ( result < padEnd && p.To < resultEnd ) || ( result < fromEnd && p.From < resultEnd ) ) {
		return false;
	}
	const long long perRow = static_cast<long long>( d.batch ) * d.resultWidth * ( d.channels / 4 );
	int rowChunks = 1, rowsPerItem = 1;
	chooseRowChunks( perRow, d.resultHeight, 4, 8192, &rowChunks, &rowsPerItem );
	CPadPoolArgs a;
	a.From = p.From; a.Padded = p.To; a.Result = result;
	a.Height = p.Height; a.Width = p.Width; a.Channels = p.Channels; a.ToHeight = p.ToHeight; a.ToWidth = p.ToWidth;
	a.DeltaTop = p.DeltaTop; a.DeltaLeft = p.DeltaLeft; a.DefaultValue = p.DefaultValue;
	a.StrideHeight = d.strideHeight; a.StrideWidth = d.strideWidth; a.ResultHeight = d.resultHeight; a.ResultWidth = d.resultWidth;
	a.RowChunks = rowChunks; a.RowsPerItem = rowsPerItem;
	a.TotalItems = perRow * rowChunks;
	long long blocks = ( a.TotalItems + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	hipLaunchKernelGGL( padMaxPool3x3Kernel, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream, a );
	const hipError_t launched = hipGetLastError();
	if( launched != hipSuccess ) {
		setLastError( hipGetErrorString( launched ) );
		*rc = NH_ERR_HIP;
	} else {
		*rc = NH_OK;
	}
	return true;
}


typedef float expandAcc __attribute__( ( ext_vector_type( 16 ) ) );

// CLIPPED: both activations are ReLU with an upper threshold ( ReLU6, what MobileNetV2 uses ): two instructions per value
template<bool CLIPPED>
__device__ __forceinline__ float activateExpanded( float v, const CFusedActivation& a )
{
	if( CLIPPED ) {
		// the median of ( v, 0, threshold ) in one instruction; with a NaN among its operands the instruction returns the
		// smallest of the others, so NaN becomes 0, as in VectorReLU
		return __builtin_amdgcn_fmed3f( v, 0.f, a.Param );
	}
	return applyActivation( v, a );
}

// ( four workgroups per compute unit where the registers allow it without spills: 16 input channels )
template<int STRIDE, int KIN, bool CLIPPED>
__global__ __launch_bounds__( 256, KIN <= 16 ? 4 : 2 )
void expandDepthwiseKernel( const nhSeparableBlockDesc d, int outH, int outW, const float* input, const float* expandFilter,
	const float* expandBias, const float* dwFilter, const float* dwBias, float* result, int tilesX, int tilesY, int totalTiles,
	const CFusedActivation expandAct, const CFusedActivation dwAct, unsigned resultBytes )
{
	constexpr int PH = STRIDE == 1 ? 8 : 7, PW = STRIDE == 1 ? 8 : 9;
	constexpr int OH = ( PH - 3 ) / STRIDE + 1, OW = ( PW - 3 ) / STRIDE + 1;
	constexpr int PitchE = 36;
	constexpr int KG = KIN / 8;
	static_assert( PH * PW <= 64 && KIN % 8 == 0, "one pixel per accumulator row of two blocks, whole groups of 8 k" );
	__shared__ __attribute__( ( aligned( 16 ) ) ) float ldsE[4][64 * PitchE];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
	int t = xcdSwizzle( blockIdx.x, gridDim.x ) * 4 + wave;
	if( t >= totalTiles ) {
		return;
	}
	const int tx = t % tilesX; t /= tilesX;
	const int ty = t % tilesY;
	const int n = t / tilesY;
	const int cexp = d.expandedChannels;
	const int hy0 = ty * OH * STRIDE - 1, wx0 = tx * OW * STRIDE - 1;
	auto insideImage = [&]( int p ) -> bool {
		const int py = p / PW, px = p - py * PW;
		const int hy = hy0 + py, wx = wx0 + px;
		return p < PH * PW && hy >= 0 && hy < d.height && wx >= 0 && wx < d.width;
	};
	// the patch as MFMA operand: lane ( l32, half ) holds k = 8 g + 4 half .. + 3 of pixel 32 b + l32
	const __amdgpu_buffer_rsrc_t image = makeBuffer( input + static_cast<long long>( n ) * d.height * d.width * KIN );
	float4 a[2][KG];
	unsigned insideBits[2];
#pragma unroll
	for( int b = 0; b < 2; ++b ) {
		const int p = b * 32 + l32;
		const int py = p / PW, px = p - py * PW;
		const unsigned base = insideImage( p ) ? static_cast<unsigned>( ( ( hy0 + py ) * d.width + wx0 + px ) * KIN + half * 4 ) * 4u : OutOfRange;
#pragma unroll
		for( int g = 0; g < KG; ++g ) {
			// a valid offset is below 2 GiB, so adding to an out-of-range one stays out of range
			a[b][g] = bufferLoad4( image, base + g * 32u );
		}
		// bit r: accumulator register r of this lane in block b is a pixel of the image
		insideBits[b] = 0;
#pragma unroll
		for( int r = 0; r < 16; ++r ) {
			insideBits[b] |= insideImage( b * 32 + ( r >> 2 ) * 8 + half * 4 + ( r & 3 ) ) ? ( 1u << r ) : 0u;
		}
	}
	// ( rows beyond PH x PW are never read by a window, so "inside" only matters for the patch's own pixels )
	const bool wholePatchInside = hy0 >= 0 && wx0 >= 0 && hy0 + PH <= d.height && wx0 + PW <= d.width;
	float* const tile = ldsE[wave];
	const int q4 = ( lane & 7 ) * 4;
	// lane ( q, o ) sums 4 channels of the output pixels 8 pass + o: where their windows begin in the tile and where they go
	constexpr int Passes = ( OH * OW + 7 ) / 8;
	int windowAt[Passes];
	unsigned storeAt[Passes]; // byte offset in result, without the chunk's channels; out of range: no such pixel
#pragma unroll
	for( int pass = 0; pass < Passes; ++pass ) {
		const int op = pass * 8 + ( lane >> 3 );
		const int oy = op / OW, ox = op - oy * OW;
		const int gy = ty * OH + oy, gx = tx * OW + ox;
		// ( lanes beyond the patch's outputs compute on the window at the origin; what they compute goes nowhere )
		windowAt[pass] = ( op < OH * OW ? ( oy * STRIDE * PW + ox * STRIDE ) * PitchE : 0 ) + q4;
		storeAt[pass] = ( op < OH * OW && gy < outH && gx < outW )
			? static_cast<unsigned>( ( ( n * outH + gy ) * outW + gx ) * cexp + q4 ) * 4u : OutOfRange;
	}
	// Every load and store of the chunk loop is a buffer access issued on every path ( what has nothing to move gets an
	// offset beyond the range: reads zeros, drops stores ), so that the compiler can count what is in flight: behind a
	// branch it waits for everything, and a pass of outputs then began by waiting for the stores of the pass before it
	// ( five round trips to memory per chunk, two thirds of the kernel's time ). A chunk's offset travels as the access's
	// scalar offset, which the range check does not see: the lane's part says whether the lane has a row / a quad at all.
	const __amdgpu_buffer_rsrc_t wBuffer = makeBuffer( expandFilter );
	const __amdgpu_buffer_rsrc_t expandBiasBuffer = __builtin_amdgcn_make_buffer_rsrc(
		const_cast<float*>( expandBias != nullptr ? expandBias : expandFilter ), 0, expandBias != nullptr ? BufferBytes : 0u, 0x00020000 );
	const __amdgpu_buffer_rsrc_t fBuffer = makeBuffer( dwFilter );
	const __amdgpu_buffer_rsrc_t dwBiasBuffer = __builtin_amdgcn_make_buffer_rsrc(
		const_cast<float*>( dwBias != nullptr ? dwBias : dwFilter ), 0, dwBias != nullptr ? BufferBytes : 0u, 0x00020000 );
	const __amdgpu_buffer_rsrc_t outBuffer = __builtin_amdgcn_make_buffer_rsrc( result, 0, resultBytes, 0x00020000 );
	// a chunk's rows of the expand filter ( lane = channel c0 + l32 ) and its free term are requested one chunk ahead
	float4 wNext[KG];
	float biasNext = 0.f;
	auto requestChunk = [&]( int c0 ) {
		const bool rowOk = c0 + l32 < cexp;
		const unsigned at = rowOk ? static_cast<unsigned>( l32 * KIN + half * 4 ) * 4u : OutOfRange;
#pragma unroll
		for( int g = 0; g < KG; ++g ) {
			wNext[g] = bufferLoad4( wBuffer, at + g * 32u, static_cast<unsigned>( c0 ) * ( KIN * 4u ) );
		}
		biasNext = __uint_as_float( __builtin_amdgcn_raw_buffer_load_b32( expandBiasBuffer, rowOk ? l32 * 4u : OutOfRange, c0 * 4, 0 ) );
	};
	requestChunk( 0 );
	// ( the compiler's count of what may be in flight at the top of the loop is the worse of the two ways there: what
	// follows a chunk's request in an iteration, ten loads' and Passes stores' worth, follows the first request too )
#pragma unroll
	for( int k = 0; k < 10 + Passes; ++k ) {
		bufferStore4( outBuffer, OutOfRange + 16u * k, make_float4( 0.f, 0.f, 0.f, 0.f ) ); // ( distinct, or they are merged into one )
	}
	for( int c0 = 0; c0 < cexp; c0 += 32 ) {
		float4 w[KG];
#pragma unroll
		for( int g = 0; g < KG; ++g ) {
			w[g] = wNext[g]; // ( rows beyond the last channel were read as zeros )
		}
		const float bias = biasNext;
		requestChunk( c0 + 32 );
		const bool quadOk = c0 + q4 < cexp;
		const unsigned quadAt = quadOk ? q4 * 4u : OutOfRange;
		float4 f[9];
#pragma unroll
		for( int k = 0; k < 9; ++k ) {
			f[k] = bufferLoad4( fBuffer, quadAt, static_cast<unsigned>( k * cexp + c0 ) * 4u );
		}
		const float4 bias4 = bufferLoad4( dwBiasBuffer, quadAt, static_cast<unsigned>( c0 ) * 4u );
#pragma unroll
		for( int b = 0; b < 2; ++b ) {
			// the accumulator starts as the free term: every register of a lane belongs to the lane's channel
			expandAcc acc;
#pragma unroll
			for( int r = 0; r < 16; ++r ) {
				acc[r] = bias;
			}
#pragma unroll
			for( int g = 0; g < KG; ++g ) {
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[b][g].x, w[g].x, acc, 0, 0, 0 );
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[b][g].y, w[g].y, acc, 0, 0, 0 );
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[b][g].z, w[g].z, acc, 0, 0, 0 );
				acc = __builtin_amdgcn_mfma_f32_32x32x2f32( a[b][g].w, w[g].w, acc, 0, 0, 0 );
			}
			if( wholePatchInside ) {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					tile[( b * 32 + ( r >> 2 ) * 8 + half * 4 + ( r & 3 ) ) * PitchE + l32] = activateExpanded<CLIPPED>( acc[r], expandAct );
				}
			} else {
#pragma unroll
				for( int r = 0; r < 16; ++r ) {
					const float v = activateExpanded<CLIPPED>( acc[r], expandAct );
					tile[( b * 32 + ( r >> 2 ) * 8 + half * 4 + ( r & 3 ) ) * PitchE + l32] = ( ( insideBits[b] >> r ) & 1u ) != 0 ? v : 0.f;
				}
			}
		}
		// the wave's own writes, read back by other lanes of the same wave: ordered by the LDS, kept in order by the fence
		__builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
		__builtin_amdgcn_wave_barrier();
		__builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );
#pragma unroll
		for( int pass = 0; pass < Passes; ++pass ) {
			const float* e = tile + windowAt[pass];
			float4 acc = CChanVec<4>::fma( *reinterpret_cast<const float4*>( e ), f[0], bias4 );
#pragma unroll
			for( int k = 1; k < 9; ++k ) {
				acc = CChanVec<4>::fma( *reinterpret_cast<const float4*>( e + ( ( k / 3 ) * PW + k % 3 ) * PitchE ), f[k], acc );
			}
			__builtin_amdgcn_raw_buffer_store_b128( u32x4{
				__float_as_uint( activateExpanded<CLIPPED>( acc.x, dwAct ) ), __float_as_uint( activateExpanded<CLIPPED>( acc.y, dwAct ) ),
				__float_as_uint( activateExpanded<CLIPPED>( acc.z, dwAct ) ), __float_as_uint( activateExpanded<CLIPPED>( acc.w, dwAct ) ) },
				outBuffer, quadOk ? storeAt[pass] : OutOfRange, c0 * 4, 0 );
		}
		__builtin_amdgcn_fence( __ATOMIC_RELEASE, "wavefront" );
		__builtin_amdgcn_wave_barrier();
		__builtin_amdgcn_fence( __ATOMIC_ACQUIRE, "wavefront" );
	}
}

} // namespace nh

// true ( and launched ) where the fused kernel is built for the block and the expanded tensor is too large for the caches
static bool tryExpandDepthwise( nhStream s, const nhSeparableBlockDesc* d, const nhConvDesc& dw, const float* input,
	const float* expandFilter, const float* expandBias, const float* dwFilter, const float* dwBias, float* reduced )
{
	const long long expandedBytes = static_cast<long long>( d->batch ) * d->height * d->width * d->expandedChannels * 4;
	const long long resultBytes = static_cast<long long>( d->batch ) * dw.resultHeight * dw.resultWidth * d->expandedChannels * 4;
	if( expandedBytes < ( 64LL << 20 ) || resultBytes >= 0x7fffff00LL || d->expandedChannels % 4 != 0 || !isAligned16( input ) || !isAligned16( expandFilter )
		|| !isAligned16( dwFilter ) || ( dwBias != nullptr && !isAligned16( dwBias ) ) || !isAligned16( reduced )
		|| ( d->inputChannels != 16 && d->inputChannels != 24 && d->inputChannels != 32 )
		|| static_cast<long long>( d->height ) * d->width * d->inputChannels * 4 >= 0x7fffffffLL )
	{
		return false;
	}
	const int oh = d->stride == 1 ? 6 : 3, ow = d->stride == 1 ? 6 : 4;
	const int tilesX = ceilDiv( dw.resultWidth, ow ), tilesY = ceilDiv( dw.resultHeight, oh );
	const long long tiles = static_cast<long long>( d->batch ) * tilesX * tilesY;
	if( tiles < 4096 || tiles > 0x7ffffff0LL ) {
		return false;
	}
	const unsigned groups = static_cast<unsigned>( ( tiles + 3 ) / 4 );
	const CFusedActivation expandAct = { d->expandActivation, d->expandParam };
	const CFusedActivation dwAct = { d->channelwiseActivation, d->channelwiseParam };
	const bool clipped = d->expandActivation == NH_ACT_RELU && d->expandParam > 0.f && d->channelwiseActivation == NH_ACT_RELU
		&& d->channelwiseParam > 0.f;
#define NH_EXPAND_DW( STRIDE, KIN, CLIPPED ) hipLaunchKernelGGL( ( expandDepthwiseKernel<STRIDE, KIN, CLIPPED> ), dim3( groups ), \
		dim3( 256 ), 0, toStream( s ), *d, dw.resultHeight, dw.resultWidth, input, expandFilter, expandBias, dwFilter, dwBias, reduced, \
		tilesX, tilesY, static_cast<int>( tiles ), expandAct, dwAct, static_cast<unsigned>( resultBytes ) )
#define NH_EXPAND_DW_K( STRIDE, CLIPPED ) if( d->inputChannels == 16 ) { NH_EXPAND_DW( STRIDE, 16, CLIPPED ); } \
	else if( d->inputChannels == 24 ) { NH_EXPAND_DW( STRIDE, 24, CLIPPED ); } else { NH_EXPAND_DW( STRIDE, 32, CLIPPED ); }
	if( d->stride == 1 ) {
		if( clipped ) { NH_EXPAND_DW_K( 1, true ) } else { NH_EXPAND_DW_K( 1, false ) }
	} else {
		if( clipped ) { NH_EXPAND_DW_K( 2, true ) } else { NH_EXPAND_DW_K( 2, false ) }
	}
#undef NH_EXPAND_DW_K
#undef NH_EXPAND_DW
	return true;
}

extern "C" {


int nhInitBlobChannelwiseConvolution( nhConvDesc* d )
{
	NH_REQUIRE( d != nullptr );
	NH_REQUIRE( d->batch >= 0 && d->height > 0 && d->width > 0 && d->channels > 0 );
	NH_REQUIRE( d->filterHeight > 0 && d->filterWidth > 0 && d->strideHeight > 0 && d->strideWidth > 0 );
	NH_REQUIRE( d->paddingHeight >= 0 && d->paddingWidth >= 0 );
	NH_REQUIRE( d->paddingHeight < d->filterHeight && d->paddingWidth < d->filterWidth );
	NH_REQUIRE( d->height + 2 * d->paddingHeight >= d->filterHeight && d->width + 2 * d->paddingWidth >= d->filterWidth );
	d->filterCount = d->channels;
	d->dilationHeight = 1;
	d->dilationWidth = 1;
	d->resultHeight = ( d->height + 2 * d->paddingHeight - d->filterHeight ) / d->strideHeight + 1;
	d->resultWidth = ( d->width + 2 * d->paddingWidth - d->filterWidth ) / d->strideWidth + 1;
	return NH_OK;
}

static int channelwiseConvolution( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act );

int nhBlobChannelwiseConvolution( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result )
{
	// ( on a stream that puts calls aside the convolution waits for the call behind it: a ReLU over its result in place
	// goes into the same launch )
	if( d != nullptr && source != nullptr && filter != nullptr && result != nullptr ) {
		nhConvDesc check = *d;
		if( nhInitBlobChannelwiseConvolution( &check ) == NH_OK && check.resultHeight == d->resultHeight && check.resultWidth == d->resultWidth
			&& deferConvolution( s, true, check, source, filter, freeTerm, result ) )
		{
			return NH_OK;
		}
	}
	const CFusedActivation none = { NH_ACT_NONE, 0.f };
	return channelwiseConvolution( s, d, source, filter, freeTerm, result, none );
}

static int channelwiseConvolution( nhStream s, const nhConvDesc* d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act )
{
	NH_REQUIRE( d != nullptr && source != nullptr && filter != nullptr && result != nullptr );
	nhConvDesc check = *d;
	const int rc = nhInitBlobChannelwiseConvolution( &check );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( check.resultHeight == d->resultHeight && check.resultWidth == d->resultWidth );
	if( d->batch == 0 ) {
		return NH_OK;
	}
	const bool vec = d->channels % 4 == 0 && isAligned16( source ) && isAligned16( filter ) && isAligned16( result )
		&& ( freeTerm == nullptr || isAligned16( freeTerm ) );
	// the strip kernel addresses the image with 32-bit byte offsets and counts work items in an int
	const long long sourceBytes = static_cast<long long>( d->batch ) * d->height * d->width * d->channels * 4;
	if( vec && d->filterHeight == 3 && d->filterWidth == 3 && d->strideHeight == d->strideWidth && d->strideHeight <= 2
		&& sourceBytes < 0x80000000LL
		&& static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->channels * 4 < 0x80000000LL )
	{
		return d->strideHeight == 1 ? channelwise3x3Impl<1, 4>( s, d, source, filter, freeTerm, result, act )
			: channelwise3x3Impl<2, 2>( s, d, source, filter, freeTerm, result, act );
	}
	constexpr int WPT = 4;
	const int wGroups = ceilDiv( d->resultWidth, WPT );
	const long long items = static_cast<long long>( d->batch ) * d->resultHeight * wGroups * ( vec ? d->channels / 4 : d->channels );
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( ( channelwiseConvKernel<4, WPT> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, source, filter, freeTerm, result, wGroups, items, act );
	} else {
		hipLaunchKernelGGL( ( channelwiseConvKernel<1, WPT> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, source, filter, freeTerm, result, wGroups, items, act );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

} // extern "C"

// a convolution that waited for its successor ( vector_ops.hip ), with the activation the successor turned out to be
int nh::launchDeferredConvolution( hipStream_t stream, bool channelwise, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act )
{
	if( channelwise ) {
		return channelwiseConvolution( reinterpret_cast<nhStream>( stream ), &d, source, filter, freeTerm, result, act );
	}
	return convImplicitGemm( stream, d, source, filter, freeTerm, result, act, nullptr );
}

extern "C" {

int nhInitPooling( nhPoolingDesc* d )
{
	NH_REQUIRE( d != nullptr );
	NH_REQUIRE( d->batch >= 0 && d->height > 0 && d->width > 0 && d->channels > 0 );
	NH_REQUIRE( d->filterHeight > 0 && d->filterWidth > 0 && d->strideHeight > 0 && d->strideWidth > 0 );
	NH_REQUIRE( d->filterHeight <= d->height && d->filterWidth <= d->width );
	d->resultHeight = ( d->height - d->filterHeight ) / d->strideHeight + 1;
	d->resultWidth = ( d->width - d->filterWidth ) / d->strideWidth + 1;
	return NH_OK;
}

int nhBlobMaxPooling( nhStream s, const nhPoolingDesc* d, const float* source, int* maxIndices, float* result )
{
	const int rc = checkPoolingDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( source != nullptr && result != nullptr );
	if( maxIndices == nullptr ) {
		int fused = NH_OK;
		if( __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0 && fusePendingPadding( s, *d, source, result, &fused ) ) {
			return fused; // ( the padded image that waited for this call went out with it )
		}
		return poolingImpl<false>( s, d, source, result );
	}
	const long long total = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->channels;
	if( total == 0 ) {
		return NH_OK;
	}
	const bool vec = d->channels % 4 == 0 && isAligned16( source ) && isAligned16( result ) && isAligned16( maxIndices );
	const long long items = vec ? total / 4 : total;
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	// ( the lookup reads image columns 0 .. filterWidth - 1: they exist, the filter fits the image )
	const bool square = vec && d->filterHeight == d->filterWidth && items <= 0x3fffffffLL;
	if( square && d->filterHeight == 3 ) {
		hipLaunchKernelGGL( maxPoolingIndexSquareKernel<3>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, source, maxIndices, result, static_cast<int>( items ) );
	} else if( square && d->filterHeight == 2 ) {
		hipLaunchKernelGGL( maxPoolingIndexSquareKernel<2>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, source, maxIndices, result, static_cast<int>( items ) );
	} else if( vec ) {
		hipLaunchKernelGGL( maxPoolingIndexKernel<4>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, source, maxIndices, result, items );
	} else {
		hipLaunchKernelGGL( maxPoolingIndexKernel<1>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, source, maxIndices, result, items );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhBlobMaxPoolingBackward( nhStream s, const nhPoolingDesc* d, const float* resultDiff, const int* maxIndices,
	float* sourceDiff )
{
	const int rc = checkPoolingDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( resultDiff != nullptr && maxIndices != nullptr && sourceDiff != nullptr );
	return poolingBackwardImpl<true>( s, d, resultDiff, maxIndices, sourceDiff );
}

int nhBlobMeanPoolingBackward( nhStream s, const nhPoolingDesc* d, const float* resultDiff, float* sourceDiff )
{
	const int rc = checkPoolingDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( resultDiff != nullptr && sourceDiff != nullptr );
	return poolingBackwardImpl<false>( s, d, resultDiff, nullptr, sourceDiff );
}

static int checkedChannelwiseDesc( const nhConvDesc* d )
{
	NH_REQUIRE( d != nullptr );
	nhConvDesc check = *d;
	const int rc = nhInitBlobChannelwiseConvolution( &check );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( check.resultHeight == d->resultHeight && check.resultWidth == d->resultWidth );
	return NH_OK;
}

int nhBlobChannelwiseConvolutionBackward( nhStream s, const nhConvDesc* d, const float* outputDiff, const float* filter,
	float* inputDiff )
{
	const int rc = checkedChannelwiseDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( outputDiff != nullptr && filter != nullptr && inputDiff != nullptr );
	if( d->batch == 0 ) {
		return NH_OK;
	}
	const bool vec = d->channels % 4 == 0 && isAligned16( outputDiff ) && isAligned16( filter ) && isAligned16( inputDiff );
	if( vec && d->filterHeight == 3 && d->filterWidth == 3 && d->strideHeight == 1 && d->strideWidth == 1
		&& d->dilationHeight == 1 && d->dilationWidth == 1 && d->paddingHeight <= 2 && d->paddingWidth <= 2
		&& static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->channels * 4 < 0x7fffffffLL
		&& static_cast<long long>( d->batch ) * d->height * d->width * d->channels * 4 < 0x7fffffffLL )
	{
		// Stride 1: the gradient by the input is the depthwise convolution of the output gradient with the filter turned
		// by 180 degrees and padding 2 - p: the forward pass's strip kernel ( every row of the gradient read once per strip ).
		nhConvDesc turned = *d;
		turned.height = d->resultHeight;
		turned.width = d->resultWidth;
		turned.paddingHeight = 2 - d->paddingHeight;
		turned.paddingWidth = 2 - d->paddingWidth;
		turned.resultHeight = d->height;
		turned.resultWidth = d->width;
		const CFusedActivation none = { NH_ACT_NONE, 0.f };
		return channelwise3x3Impl<1, 4>( s, &turned, outputDiff, filter, nullptr, inputDiff, none, true );
	}
	if( vec && d->filterHeight == 3 && d->filterWidth == 3 && d->strideHeight == 2 && d->strideWidth == 2
		&& static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->channels * 4 < 0x7fffffffLL
		&& static_cast<long long>( d->batch ) * d->height * d->width * ( d->channels / 4 ) < 0x7fffff00LL )
	{
		// strips of 8 columns of wi + padW and of 2 row pairs: measured on 128 x 112 x 112 x 96, strips of 2 / 3 / 6 / 12 / 29
		// pairs take 150 / 153 / 162 / 171 / 184 us although the short ones read every second row of the output gradient twice
		const int pairs = ( d->height + d->paddingHeight + 1 ) / 2;
		const int wGroups = ( d->width + d->paddingWidth + 7 ) / 8;
		const long long perChunk = static_cast<long long>( d->batch ) * wGroups * ( d->channels / 4 );
		const int pairsPerItem = 2;
		const int chunks = ( pairs + pairsPerItem - 1 ) / pairsPerItem;
		const int total = static_cast<int>( perChunk * chunks );
		hipLaunchKernelGGL( channelwiseBackward3x3Stride2Kernel, dim3( static_cast<unsigned>( ( total + 255 ) / 256 ) ), dim3( 256 ), 0,
			toStream( s ), *d, outputDiff, filter, inputDiff, wGroups, chunks, pairsPerItem, pairs, total );
		NH_LAUNCH_CHECK();
		return NH_OK;
	}
	const long long items = static_cast<long long>( d->batch ) * d->height * d->width * ( vec ? d->channels / 4 : d->channels );
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( channelwiseConvBackwardKernel<4>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, outputDiff, filter, inputDiff, items );
	} else {
		hipLaunchKernelGGL( channelwiseConvBackwardKernel<1>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			*d, outputDiff, filter, inputDiff, items );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhBlobChannelwiseConvolutionLearnAdd( nhStream s, const nhConvDesc* d, const float* input, const float* outputDiff,
	float* filterDiff, float* freeTermDiff )
{
	const int rc = checkedChannelwiseDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( input != nullptr && outputDiff != nullptr && filterDiff != nullptr );
	if( d->batch == 0 ) {
		return NH_OK;
	}
	const bool vec = d->channels % 4 == 0 && isAligned16( input ) && isAligned16( outputDiff );
	if( vec && d->filterHeight == 3 && d->filterWidth == 3 && d->strideHeight == d->strideWidth && d->strideHeight <= 2
		&& d->channels <= 1024
		&& static_cast<long long>( d->batch ) * d->height * d->width * d->channels * 4 < 0x80000000LL
		&& static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->channels < 0x7fffffffLL )
	{
		return d->strideHeight == 1 ? channelwiseLearn3x3Impl<1, 4>( s, d, input, outputDiff, filterDiff, freeTermDiff )
			: channelwiseLearn3x3Impl<2, 2>( s, d, input, outputDiff, filterDiff, freeTermDiff );
	}
	const int cg = vec ? d->channels / 4 : d->channels;
	// channel groups per workgroup: a power of two up to 64, so that a wave reads whole runs of channels
	int groups = 1;
	while( groups < cg && groups < 64 ) {
		groups *= 2;
	}
	const int groupBlocks = ceilDiv( cg, groups );
	const long long pixels = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth;
	// about 1024 workgroups ( measured best of 256..2048 ), each lane at least 8 pixels of its own
	const int lanes = 256 / groups;
	long long slices = 1024 / groupBlocks > 0 ? 1024 / groupBlocks : 1;
	const long long most = pixels / ( 8LL * lanes ) > 0 ? pixels / ( 8LL * lanes ) : 1;
	slices = slices < most ? slices : most;
	const long long pixelsPerSlice = ( pixels + slices - 1 ) / slices;
	slices = ( pixels + pixelsPerSlice - 1 ) / pixelsPerSlice;
	const dim3 grid( static_cast<unsigned>( slices * groupBlocks ) );
	const bool is3x3 = d->filterHeight == 3 && d->filterWidth == 3;
#define NH_LAUNCH_LEARN( VECW, TAPS ) hipLaunchKernelGGL( ( channelwiseConvLearnKernel<VECW, TAPS> ), grid, dim3( 256 ), 0, \
	toStream( s ), *d, input, outputDiff, filterDiff, freeTermDiff, groups, groupBlocks, pixelsPerSlice )
	if( vec ) {
		if( is3x3 ) { NH_LAUNCH_LEARN( 4, 9 ); } else { NH_LAUNCH_LEARN( 4, 0 ); }
	} else {
		if( is3x3 ) { NH_LAUNCH_LEARN( 1, 9 ); } else { NH_LAUNCH_LEARN( 1, 0 ); }
	}
#undef NH_LAUNCH_LEARN
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhBlobMeanPooling( nhStream s, const nhPoolingDesc* d, const float* source, float* result )
{
	const int rc = checkPoolingDesc( d );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( source != nullptr && result != nullptr );
	return poolingImpl<true>( s, d, source, result );
}

int nhBlobResizeImage( nhStream s, const nhBlobDesc* from, const float* fromData, int deltaLeft, int deltaRight,
	int deltaTop, int deltaBottom, int padding, float defaultValue, const nhBlobDesc* to, float* toData )
{
	NH_REQUIRE( from != nullptr && to != nullptr && fromData != nullptr && toData != nullptr );
	NH_REQUIRE( padding == NH_PAD_CONSTANT || padding == NH_PAD_EDGE || padding == NH_PAD_REFLECT );
	const int height = from->dims[3], width = from->dims[4];
	const int channels = from->dims[5] * from->dims[6];
	const long long batch = dimProduct( *from, 0, 3 );
	const int toHeight = height + deltaTop + deltaBottom;
	const int toWidth = width + deltaLeft + deltaRight;
	NH_REQUIRE( height > 0 && width > 0 && channels > 0 && toHeight > 0 && toWidth > 0 );
	NH_REQUIRE( to->dims[3] == toHeight && to->dims[4] == toWidth && to->dims[5] * to->dims[6] == channels );
	NH_REQUIRE( dimProduct( *to, 0, 3 ) == batch );
	if( batch == 0 ) {
		return NH_OK;
	}
	CPendingPadding p;
	p.From = fromData; p.To = toData; p.Batch = batch;
	p.Height = height; p.Width = width; p.Channels = channels; p.ToHeight = toHeight; p.ToWidth = toWidth;
	p.DeltaLeft = deltaLeft; p.DeltaTop = deltaTop; p.Padding = padding; p.DefaultValue = defaultValue;
	// ( on a stream that puts calls aside a border of constants waits for the pooling over the padded image )
	if( padding == NH_PAD_CONSTANT && deltaLeft >= 0 && deltaRight >= 0 && deltaTop >= 0 && deltaBottom >= 0 && channels % 4 == 0
		&& isAligned16( fromData ) && isAligned16( toData ) && deferPadding( s, p ) ) {
		return NH_OK;
	}
	return launchPadding( toStream( s ), p );
}

int nhBlobMergeByDim( nhStream s, int dim, const nhBlobDesc* from, const float* const* fromData, int fromCount,
	const nhBlobDesc* to, float* toData )
{
	NH_REQUIRE( from != nullptr && fromData != nullptr && to != nullptr && toData != nullptr );
	return splitMergeImpl<true>( s, dim, *to, toData, from, const_cast<float* const*>( fromData ), fromCount );
}

int nhBroadcastCopy( nhStream s, void* to, const void* from, const nhBlobDesc* toDesc, const nhBlobDesc* fromDesc,
	int additionalWidth )
{
	NH_REQUIRE( to != nullptr && from != nullptr && toDesc != nullptr && fromDesc != nullptr && additionalWidth >= 1 );
	CBroadcastShape shape;
	long long total = additionalWidth, stride = additionalWidth;
	shape.ToDims[7] = additionalWidth;
	shape.FromStrides[7] = 1;
	for( int d = 6; d >= 0; --d ) {
		NH_REQUIRE( toDesc->dims[d] >= 1 && ( fromDesc->dims[d] == 1 || fromDesc->dims[d] == toDesc->dims[d] ) );
		shape.ToDims[d] = toDesc->dims[d];
		shape.FromStrides[d] = fromDesc->dims[d] == toDesc->dims[d] ? static_cast<int>( stride ) : 0;
		stride *= fromDesc->dims[d];
		total *= toDesc->dims[d];
	}
	NH_REQUIRE( stride <= 0x7fffffffLL );
	long long blocks = ( total + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	hipLaunchKernelGGL( broadcastCopyKernel, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
		static_cast<unsigned*>( to ), static_cast<const unsigned*>( from ), shape, total );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhDropout( nhStream s, const nhBlobDesc* input, float rate, int isSpatial, int isBatchwise, int seed, const float* in,
	float* out )
{
	NH_REQUIRE( input != nullptr && rate >= 0.f && rate < 1.f );
	const long long objectCount = dimProduct( *input, 0, 3 );
	const long long objectSize = dimProduct( *input, 3, 7 );
	const long long total = objectCount * objectSize;
	if( total == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( in != nullptr && out != nullptr && total <= 0x7fffffffLL );
	const float forwardRate = 1.f - rate;
	if( forwardRate == 1.f ) {
		return nhVectorCopy( s, out, in, static_cast<int>( total ) );
	}
	// batchwise: every object is its own outer slice, the mask covers one object
	const long long batchLength = isBatchwise ? objectCount : input->dims[0];
	const int batchWidth = static_cast<int>( objectCount / batchLength );
	const int channels = input->dims[6];
	const long long maskSize = isSpatial ? static_cast<long long>( batchWidth ) * channels : batchWidth * objectSize;
	const unsigned threshold = static_cast<unsigned>( static_cast<double>( forwardRate ) * 4294967295.0 );
	long long blocks = ( total + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	hipLaunchKernelGGL( dropoutKernel, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
		in, out, total, static_cast<int>( maskSize ), static_cast<int>( objectSize ), channels, batchWidth, isSpatial ? 1 : 0,
		static_cast<unsigned>( seed ), threshold, 1.f / forwardRate );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhBlobSplitByDim( nhStream s, int dim, const nhBlobDesc* from, const float* fromData,
	const nhBlobDesc* to, float* const* toData, int toCount )
{
	NH_REQUIRE( from != nullptr && fromData != nullptr && to != nullptr && toData != nullptr );
	return splitMergeImpl<false>( s, dim, *from, const_cast<float*>( fromData ), to, toData, toCount );
}

int nhStreamOverlapLstm( nhStream s, int enable )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	NH_HIP( hipGetDevice( &device ) );
	std::lock_guard<std::mutex> guard( sequenceLock );
	CLstmOverlap& o = lstmOverlaps()[std::make_pair( device, stream )];
	if( enable != 0 && o.Side == nullptr ) {
		NH_HIP( hipStreamCreateWithFlags( &o.Side, hipStreamNonBlocking ) );
		NH_HIP( hipEventCreateWithFlags( &o.Before, hipEventDisableTiming ) );
		NH_HIP( hipEventCreateWithFlags( &o.SideDone, hipEventDisableTiming ) );
	}
	if( ( enable != 0 ) != o.Enabled ) {
		if( enable != 0 ) {
			__atomic_fetch_add( &overlapLstmStreams, 1, __ATOMIC_RELAXED );
		} else {
			__atomic_fetch_sub( &overlapLstmStreams, 1, __ATOMIC_RELAXED );
		}
		o.Enabled = enable != 0;
	}
	setLastWasLstm( o, false );
	return NH_OK;
}

// workspace layout: [ gates: T*B*4H ][ free term: 4H ][ state: B*H ][ tagged h exchange: 2*B*H 64-bit words ]
// [ the same for readers on the writer's XCD ][ table of XCDs: 256 words ][ abort word: 64 bits ]
int nhLstmWorkspaceSize( int hiddenSize, int objectSize, int sequenceLength, int sequenceCount, size_t* bytes )
{
	NH_REQUIRE( bytes != nullptr && hiddenSize > 0 && objectSize > 0 && sequenceLength >= 0 && sequenceCount >= 0 );
	const size_t gates = static_cast<size_t>( sequenceLength ) * sequenceCount * 4 * hiddenSize;
	*bytes = ( gates + 4 * static_cast<size_t>( hiddenSize ) + 9 * static_cast<size_t>( sequenceCount ) * hiddenSize + LstmXcdTableWords + 2 ) * sizeof( float );
	return NH_OK;
}

int nhLstm( nhStream s, int hiddenSize, int objectSize, const float* inputWeights, const float* inputFreeTerm,
	const float* recurrentWeights, const float* recurrentFreeTerm, int reverse, int sequenceLength,
	int sequenceCount, const float* inputStateBackLink, const float* inputMainBackLink, const float* input,
	float* outputStateBackLink, float* outputMainBackLink, void* workspace, size_t workspaceSize )
{
	size_t need = 0;
	const int rc0 = nhLstmWorkspaceSize( hiddenSize, objectSize, sequenceLength, sequenceCount, &need );
	if( rc0 != NH_OK ) {
		return rc0;
	}
	NH_REQUIRE( inputWeights != nullptr && recurrentWeights != nullptr && input != nullptr && outputMainBackLink != nullptr );
	NH_REQUIRE( workspace != nullptr && workspaceSize >= need && isAligned16( workspace ) );
	if( sequenceLength == 0 || sequenceCount == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( static_cast<long long>( sequenceLength ) * sequenceCount * 4 * hiddenSize <= 0x7fffffffLL );
	const int H = hiddenSize;
	const int B = sequenceCount;
	const int T = sequenceLength;
	// ( not through toStream: whether something was enqueued since the last nhLstm is what is asked here; small calls that
	// the stream has put aside are launched now and count as enqueued )
	const hipStream_t mainStream = reinterpret_cast<hipStream_t>( s );
	if( __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0 && flushTinyOps( mainStream ) ) {
		noteStreamUse( mainStream );
	}
	hipStream_t stream = mainStream;
	const bool sequencePath = T > 1 && lstmSequenceFits( H, B, recurrentWeights, inputStateBackLink, inputMainBackLink, outputMainBackLink )
		&& lstmSequenceAllowed( mainStream );
	// what this call writes and reads
	CByteRange written[3], read[4];
	{
		const size_t stateBytes = static_cast<size_t>( T ) * B * H * sizeof( float );
		const size_t oneState = static_cast<size_t>( B ) * H * sizeof( float );
		auto range = []( const void* p, size_t bytes ) {
			CByteRange r;
			if( p != nullptr ) {
				r.Lo = static_cast<const char*>( p );
				r.Hi = r.Lo + bytes;
			}
			return r;
		};
		written[0] = range( outputMainBackLink, stateBytes );
		written[1] = range( outputStateBackLink, stateBytes );
		written[2] = range( workspace, need );
		read[0] = range( input, static_cast<size_t>( T ) * B * objectSize * sizeof( float ) );
		read[1] = range( inputMainBackLink, oneState );
		read[2] = range( inputStateBackLink, oneState );
	}
	bool overlapEnabled = false;
	bool beside = false; // this call runs on the side stream, beside the one-launch LSTM issued just before
	CLstmOverlap pair;
	if( __atomic_load_n( &overlapLstmStreams, __ATOMIC_RELAXED ) != 0 ) {
		int device = 0;
		NH_HIP( hipGetDevice( &device ) );
		std::lock_guard<std::mutex> guard( sequenceLock );
		auto found = lstmOverlaps().find( std::make_pair( device, mainStream ) );
		if( found != lstmOverlaps().end() && found->second.Enabled ) {
			CLstmOverlap& o = found->second;
			overlapEnabled = true;
			beside = o.LastWasLstm && sequencePath && lstmSequenceShape( H, B, true ) != nullptr;
			if( beside ) {
				const long long groups = static_cast<long long>( H / ( SeqUnits * lstmSequenceShape( H, B, true )->Blocks ) )
					* ceilDiv( B, lstmSequenceShape( H, B, true )->Rows );
				int units = 0;
				beside = lstmXcdShape( H, B, true ) != nullptr
					|| ( hipDeviceGetAttribute( &units, hipDeviceAttributeMultiprocessorCount, device ) == hipSuccess && groups <= units / 2 );
			}
			for( int i = 0; beside && i < 3; ++i ) {
				for( int j = 0; j < 3; ++j ) {
					beside = beside && !rangesMeet( written[i], o.Written[j] ) && !rangesMeet( read[i], o.Written[j] )
						&& !rangesMeet( written[i], o.Read[j] );
				}
			}
			setLastWasLstm( o, false );
			pair = o;
		}
	}
	if( beside ) {
		stream = pair.Side;
		NH_HIP( hipStreamWaitEvent( stream, pair.Before, 0 ) ); // everything in front of the partner
	} else if( overlapEnabled && sequencePath ) {
		NH_HIP( hipEventRecord( pair.Before, mainStream ) ); // in case a partner follows
	}
	float* gates = static_cast<float*>( workspace );
	float* freeTerm = gates + static_cast<size_t>( T ) * B * 4 * H;
	float* stateScratch = freeTerm + 4 * H;

	const float* bias = nullptr;
	if( inputFreeTerm != nullptr || recurrentFreeTerm != nullptr ) {
		hipLaunchKernelGGL( addTwoVectorsKernel, dim3( ceilDiv( 4 * H, 256 ) ), dim3( 256 ), 0, stream,
			inputFreeTerm, recurrentFreeTerm, freeTerm, 4 * H );
		NH_LAUNCH_CHECK();
		bias = freeTerm;
	}
	// every step's input contribution in one product: gates[T*B x 4H] = x[T*B x In] * Win^T + free term
	int rc = matMulNT( stream, input, objectSize, inputWeights, objectSize, gates, 4 * H, T * B, 4 * H, objectSize,
		1, 0, 0, 0, bias, false );
	if( rc != NH_OK ) {
		return rc;
	}
	const int stepSize = B * H;
	if( sequencePath ) {
		CLstmSeqArgs a = {};
		a.Gates = gates; a.Wrec = recurrentWeights; a.H0 = inputMainBackLink; a.C0 = inputStateBackLink;
		a.HOut = outputMainBackLink; a.COut = outputStateBackLink;
		a.Exchange = reinterpret_cast<unsigned long long*>( stateScratch + static_cast<size_t>( B ) * H );
		a.ExchangeLocal = a.Exchange + 2 * static_cast<size_t>( B ) * H;
		a.XcdTable = reinterpret_cast<unsigned*>( a.ExchangeLocal + 2 * static_cast<size_t>( B ) * H );
		a.Abort = a.XcdTable + LstmXcdTableWords; // ( the last 8 bytes of the workspace )
		a.T = T; a.B = B; a.H = H; a.Reverse = reverse ? 1 : 0;
		a.MaxSpins = lstmSpinLimit();
		bool tookHalf = false, ranBeside = false;
		unsigned long long generation = 0;
		rc = launchLstmSequence( stream, a, overlapEnabled, beside ? &pair.Generation : nullptr, &tookHalf, &generation, &ranBeside );
		if( rc != NH_OK ) {
			return rc;
		}
		if( beside ) {
			// the main stream goes on behind both ( also where another stream's launch had come in between and this one
			// ran behind it instead of beside its partner: it is on the side stream all the same )
			NH_HIP( hipEventRecord( pair.SideDone, stream ) );
			NH_HIP( hipStreamWaitEvent( mainStream, pair.SideDone, 0 ) );
			return NH_OK;
		}
		if( overlapEnabled && tookHalf ) {
			int device = 0;
			NH_HIP( hipGetDevice( &device ) );
			std::lock_guard<std::mutex> guard( sequenceLock );
			auto found = lstmOverlaps().find( std::make_pair( device, mainStream ) );
			if( found != lstmOverlaps().end() ) {
				CLstmOverlap& o = found->second;
				setLastWasLstm( o, true );
				o.Generation = generation;
				for( int i = 0; i < 3; ++i ) {
					o.Written[i] = written[i];
					o.Read[i] = read[i];
				}
			}
		}
		return NH_OK;
	}
	// the one-launch step needs whole 32-k chunks and 8-unit blocks, 16-byte aligned rows and 32-bit byte offsets
	const bool fusedStep = H % 32 == 0 && isAligned16( recurrentWeights ) && isAligned16( outputMainBackLink )
		&& ( inputMainBackLink == nullptr || isAligned16( inputMainBackLink ) )
		&& static_cast<long long>( 4 ) * H * H * 4 < 0x80000000LL && static_cast<long long>( B ) * H * 4 < 0x80000000LL;
	for( int i = 0; i < T; ++i ) {
		const int pos = reverse ? T - 1 - i : i;
		const int prev = reverse ? pos + 1 : pos - 1;
		const float* hPrev = i == 0 ? inputMainBackLink : outputMainBackLink + static_cast<size_t>( prev ) * stepSize;
		const float* cPrev;
		float* cOut;
		if( outputStateBackLink != nullptr ) {
			cPrev = i == 0 ? inputStateBackLink : outputStateBackLink + static_cast<size_t>( prev ) * stepSize;
			cOut = outputStateBackLink + static_cast<size_t>( pos ) * stepSize;
		} else {
			cPrev = i == 0 ? inputStateBackLink : stateScratch;
			cOut = stateScratch;
		}
		float* g = gates + static_cast<size_t>( pos ) * B * 4 * H;
		if( fusedStep ) {
			hipLaunchKernelGGL( lstmStepKernel, dim3( H / LstmUnits, ceilDiv( B, LstmRows ) ), dim3( LstmThreads ), 0, stream,
				g, hPrev, recurrentWeights, cPrev, cOut, outputMainBackLink + static_cast<size_t>( pos ) * stepSize, B, H );
			NH_LAUNCH_CHECK();
			continue;
		}
		if( hPrev != nullptr ) {
			rc = matMulNT( stream, hPrev, H, recurrentWeights, H, g, 4 * H, B, 4 * H, H, 1, 0, 0, 0, nullptr, true );
			if( rc != NH_OK ) {
				return rc;
			}
		}
		hipLaunchKernelGGL( lstmGatesKernel, dim3( ceilDiv( stepSize, 256 ) ), dim3( 256 ), 0, stream,
			g, cPrev, cOut, outputMainBackLink + static_cast<size_t>( pos ) * stepSize, H, stepSize );
		NH_LAUNCH_CHECK();
	}
	return NH_OK;
}

// ---- the fused blocks of depthwise-separable networks -----------------------------------------------------------
// Every stage is one launch with its activation (and the residual sum) in the epilogue of the kernel that produces
// the values: expand 1x1 (+act) -> depthwise 3x3 (+act) -> down 1x1 (+input). Unfused, the same block costs two
// activation passes and one sum pass more over the six-fold expanded tensor.

static int checkSeparableDesc( const nhSeparableBlockDesc* d, bool withExpand, nhConvDesc* dw )
{
	NH_REQUIRE( d != nullptr );
	NH_REQUIRE( d->batch >= 0 && d->height > 0 && d->width > 0 && d->expandedChannels > 0 && d->outputChannels > 0 );
	NH_REQUIRE( !withExpand || d->inputChannels > 0 );
	NH_REQUIRE( d->stride == 1 || d->stride == 2 );
	const int blockInput = withExpand ? d->inputChannels : d->expandedChannels;
	NH_REQUIRE( d->residual == 0 || ( d->stride == 1 && blockInput == d->outputChannels ) );
	*dw = nhConvDesc();
	dw->batch = d->batch; dw->height = d->height; dw->width = d->width; dw->channels = d->expandedChannels;
	dw->filterCount = d->expandedChannels; dw->filterHeight = 3; dw->filterWidth = 3;
	dw->paddingHeight = 1; dw->paddingWidth = 1; dw->strideHeight = d->stride; dw->strideWidth = d->stride;
	return nhInitBlobChannelwiseConvolution( dw );
}

int nhMobileNetV2BlockWorkspaceSize( const nhSeparableBlockDesc* d, size_t* bytes )
{
	nhConvDesc dw;
	const int rc = checkSeparableDesc( d, true, &dw );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( bytes != nullptr );
	const size_t expanded = static_cast<size_t>( d->batch ) * d->height * d->width * d->expandedChannels;
	const size_t reduced = static_cast<size_t>( d->batch ) * dw.resultHeight * dw.resultWidth * d->expandedChannels;
	*bytes = ( ( expanded + 63 ) / 64 * 64 + reduced ) * sizeof( float );
	return NH_OK;
}

int nhMobileNetV2Block( nhStream s, const nhSeparableBlockDesc* d, const float* input, const float* expandFilter,
	const float* expandFreeTerm, const float* channelwiseFilter, const float* channelwiseFreeTerm,
	const float* downFilter, const float* downFreeTerm, float* output, void* workspace, size_t workspaceSize )
{
	nhConvDesc dw;
	int rc = checkSeparableDesc( d, true, &dw );
	if( rc != NH_OK ) {
		return rc;
	}
	size_t need = 0;
	rc = nhMobileNetV2BlockWorkspaceSize( d, &need );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( input != nullptr && expandFilter != nullptr && channelwiseFilter != nullptr && downFilter != nullptr && output != nullptr );
	NH_REQUIRE( workspace != nullptr && workspaceSize >= need && isAligned16( workspace ) );
	if( d->batch == 0 ) {
		return NH_OK;
	}
	const long long pixelsIn = static_cast<long long>( d->batch ) * d->height * d->width;
	const long long pixelsOut = static_cast<long long>( d->batch ) * dw.resultHeight * dw.resultWidth;
	NH_REQUIRE( pixelsIn <= 0x7fffffffLL && pixelsIn * d->expandedChannels <= 0x7fffffffLL );
	float* expanded = static_cast<float*>( workspace );
	float* reduced = expanded + ( static_cast<size_t>( pixelsIn ) * d->expandedChannels + 63 ) / 64 * 64;
	const CFusedActivation expandAct = { d->expandActivation, d->expandParam };
	const CFusedActivation channelwiseAct = { d->channelwiseActivation, d->channelwiseParam };
	const CFusedActivation none = { NH_ACT_NONE, 0.f };
	if( tryExpandDepthwise( s, d, dw, input, expandFilter, expandFreeTerm, channelwiseFilter, channelwiseFreeTerm, reduced ) ) {
		NH_LAUNCH_CHECK();
	} else {
		rc = matMulNTFused( toStream( s ), input, d->inputChannels, expandFilter, d->inputChannels, expanded, d->expandedChannels,
			static_cast<int>( pixelsIn ), d->expandedChannels, d->inputChannels, 1, 0, 0, 0, expandFreeTerm, false, expandAct, nullptr );
		if( rc != NH_OK ) {
			return rc;
		}
		rc = channelwiseConvolution( s, &dw, expanded, channelwiseFilter, channelwiseFreeTerm, reduced, channelwiseAct );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	return matMulNTFused( toStream( s ), reduced, d->expandedChannels, downFilter, d->expandedChannels, output, d->outputChannels,
		static_cast<int>( pixelsOut ), d->outputChannels, d->expandedChannels, 1, 0, 0, 0, downFreeTerm, false, none,
		d->residual != 0 ? input : nullptr );
}

// The two halves of a MobileNetV3 block, around its squeeze-and-excite branch: expand 1x1 (+act) -> depthwise (+act), and
// gate (+act) -> down 1x1 (+residual). The depthwise stage takes any channelwise descriptor (3x3 and 5x5 occur).
static int checkPreSE( const nhConvDesc* dw, int inputChannels )
{
	NH_REQUIRE( dw != nullptr && inputChannels > 0 );
	nhConvDesc check = *dw;
	const int rc = nhInitBlobChannelwiseConvolution( &check );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( check.resultHeight == dw->resultHeight && check.resultWidth == dw->resultWidth );
	const long long expanded = static_cast<long long>( dw->batch ) * dw->height * dw->width * dw->channels;
	NH_REQUIRE( expanded <= 0x7fffffffLL );
	return NH_OK;
}

int nhMobileNetV3PreSEBlockWorkspaceSize( const nhConvDesc* dw, size_t* bytes )
{
	const int rc = checkPreSE( dw, 1 );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( bytes != nullptr );
	*bytes = static_cast<size_t>( dw->batch ) * dw->height * dw->width * dw->channels * sizeof( float );
	return NH_OK;
}

int nhMobileNetV3PreSEBlock( nhStream s, const nhConvDesc* dw, int inputChannels, const float* input,
	const float* expandFilter, const float* expandFreeTerm, int expandActivation, float expandParam,
	const float* channelwiseFilter, const float* channelwiseFreeTerm, int channelwiseActivation, float channelwiseParam,
	float* output, void* workspace, size_t workspaceSize )
{
	const int rc = checkPreSE( dw, inputChannels );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( input != nullptr && expandFilter != nullptr && channelwiseFilter != nullptr && output != nullptr );
	const size_t need = static_cast<size_t>( dw->batch ) * dw->height * dw->width * dw->channels * sizeof( float );
	NH_REQUIRE( workspace != nullptr && workspaceSize >= need && isAligned16( workspace ) );
	if( dw->batch == 0 ) {
		return NH_OK;
	}
	float* expanded = static_cast<float*>( workspace );
	const CFusedActivation expandAct = { expandActivation, expandParam };
	const CFusedActivation channelwiseAct = { channelwiseActivation, channelwiseParam };
	if( dw->filterHeight == 3 && dw->filterWidth == 3 && dw->paddingHeight == 1 && dw->paddingWidth == 1
		&& dw->strideHeight == dw->strideWidth && ( dw->strideHeight == 1 || dw->strideHeight == 2 ) )
	{
		// the 3x3 case is the MobileNetV2 block's pair of stages: one launch where the expanded tensor would be large
		nhSeparableBlockDesc pair = {};
		pair.batch = dw->batch; pair.height = dw->height; pair.width = dw->width;
		pair.inputChannels = inputChannels; pair.expandedChannels = dw->channels; pair.outputChannels = dw->channels;
		pair.stride = dw->strideHeight;
		pair.expandActivation = expandActivation; pair.expandParam = expandParam;
		pair.channelwiseActivation = channelwiseActivation; pair.channelwiseParam = channelwiseParam;
		if( tryExpandDepthwise( s, &pair, *dw, input, expandFilter, expandFreeTerm, channelwiseFilter, channelwiseFreeTerm, output ) ) {
			NH_LAUNCH_CHECK();
			return NH_OK;
		}
	}
	const int pixels = dw->batch * dw->height * dw->width;
	const int rcExpand = matMulNTFused( toStream( s ), input, inputChannels, expandFilter, inputChannels, expanded, dw->channels,
		pixels, dw->channels, inputChannels, 1, 0, 0, 0, expandFreeTerm, false, expandAct, nullptr );
	if( rcExpand != NH_OK ) {
		return rcExpand;
	}
	return channelwiseConvolution( s, dw, expanded, channelwiseFilter, channelwiseFreeTerm, output, channelwiseAct );
}

int nhMobileNetV3PostSEBlock( nhStream s, int batch, int pixelsPerImage, int channels, int outputChannels,
	const float* channelwiseOutput, const float* squeezeAndExcite, const float* residual, int activation, float param,
	const float* downFilter, const float* downFreeTerm, float* output, void* workspace, size_t workspaceSize )
{
	NH_REQUIRE( batch >= 0 && pixelsPerImage > 0 && channels > 0 && outputChannels > 0 );
	const long long total = static_cast<long long>( batch ) * pixelsPerImage * channels;
	NH_REQUIRE( total <= 0x7fffffffLL );
	NH_REQUIRE( channelwiseOutput != nullptr && squeezeAndExcite != nullptr && downFilter != nullptr && output != nullptr );
	NH_REQUIRE( workspace != nullptr && workspaceSize >= static_cast<size_t>( total ) * sizeof( float ) && isAligned16( workspace ) );
	if( batch == 0 ) {
		return NH_OK;
	}
	float* gated = static_cast<float*>( workspace );
	const CFusedActivation act = { activation, param };
	const bool vec = channels % 4 == 0 && isAligned16( channelwiseOutput ) && isAligned16( squeezeAndExcite );
	const long long items = vec ? total / 4 : total;
	long long blocks = ( items + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( scaleChannelsKernel<4>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			channelwiseOutput, squeezeAndExcite, gated, pixelsPerImage, channels, items, act );
	} else {
		hipLaunchKernelGGL( scaleChannelsKernel<1>, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			channelwiseOutput, squeezeAndExcite, gated, pixelsPerImage, channels, items, act );
	}
	NH_LAUNCH_CHECK();
	const CFusedActivation none = { NH_ACT_NONE, 0.f };
	return matMulNTFused( toStream( s ), gated, channels, downFilter, channels, output, outputChannels,
		batch * pixelsPerImage, outputChannels, channels, 1, 0, 0, 0, downFreeTerm, false, none, residual );
}

int nhChannelwiseWith1x1WorkspaceSize( const nhSeparableBlockDesc* d, size_t* bytes )
{
	nhConvDesc dw;
	const int rc = checkSeparableDesc( d, false, &dw );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( bytes != nullptr );
	*bytes = static_cast<size_t>( d->batch ) * dw.resultHeight * dw.resultWidth * d->expandedChannels * sizeof( float );
	return NH_OK;
}

int nhChannelwiseWith1x1( nhStream s, const nhSeparableBlockDesc* d, const float* input, const float* channelwiseFilter,
	const float* channelwiseFreeTerm, const float* convFilter, const float* convFreeTerm, float* output,
	void* workspace, size_t workspaceSize )
{
	nhConvDesc dw;
	int rc = checkSeparableDesc( d, false, &dw );
	if( rc != NH_OK ) {
		return rc;
	}
	size_t need = 0;
	rc = nhChannelwiseWith1x1WorkspaceSize( d, &need );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( input != nullptr && channelwiseFilter != nullptr && convFilter != nullptr && output != nullptr );
	NH_REQUIRE( workspace != nullptr && workspaceSize >= need && isAligned16( workspace ) );
	if( d->batch == 0 ) {
		return NH_OK;
	}
	const long long pixelsOut = static_cast<long long>( d->batch ) * dw.resultHeight * dw.resultWidth;
	NH_REQUIRE( pixelsOut <= 0x7fffffffLL );
	float* reduced = static_cast<float*>( workspace );
	const CFusedActivation channelwiseAct = { d->channelwiseActivation, d->channelwiseParam };
	const CFusedActivation none = { NH_ACT_NONE, 0.f };
	rc = channelwiseConvolution( s, &dw, input, channelwiseFilter, channelwiseFreeTerm, reduced, channelwiseAct );
	if( rc != NH_OK ) {
		return rc;
	}
	return matMulNTFused( toStream( s ), reduced, d->expandedChannels, convFilter, d->expandedChannels, output, d->outputChannels,
		static_cast<int>( pixelsOut ), d->outputChannels, d->expandedChannels, 1, 0, 0, 0, convFreeTerm, false, none,
		d->residual != 0 ? input : nullptr );
}

} // extern "C"

extern "C" int nhVectorFillBernoulli( nhStream s, float* result, float p, int vectorSize, float value, int seed )
{
	NH_REQUIRE( vectorSize >= 0 );
	if( vectorSize == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( result != nullptr );
	const unsigned threshold = static_cast<unsigned>( static_cast<double>( p ) * 4294967295.0 );
	hipLaunchKernelGGL( fillBernoulliKernel, dim3( ceilDiv( vectorSize, 256 ) ), dim3( 256 ), 0, toStream( s ), result, vectorSize,
		static_cast<unsigned>( seed ), threshold, value );
	NH_LAUNCH_CHECK();
	return NH_OK;
}
