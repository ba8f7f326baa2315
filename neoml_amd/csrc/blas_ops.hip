// Bandwidth-bound matrix helpers of IBlasEngine: row/column broadcasts, row/column sums, softmax, arg-max,
// diagonal products and the blob transpose. Row reductions give one 64-lane wavefront to each row and reduce
// with cross-lane shuffles; element-wise broadcasts use 128-bit accesses when shapes and pointers allow it.
#include "common.h"
#include <float.h>

namespace nh {

// ---------------------------------------------------------------------------------------------------------
// Broadcast family: result[i] = f( matrix[matIndex( i )], vector[vecIndex( i )] )

enum TBroadcastOp { BO_Add, BO_Sub, BO_Mul, BO_Set };

template<int OP> __device__ __forceinline__ float broadcastApply( float m, float v )
{
	switch( OP ) {
		case BO_Add: return m + v;
		case BO_Sub: return m - v;
		case BO_Mul: return m * v;
		default: return v;
	}
}

// Row broadcast: element ( b, r, c ) pairs with vector[b * vecBatchStride + c];
// the matrix of batch b starts at b * matBatchStride (result is always dense).
template<int OP, bool VEC>
__global__ __launch_bounds__( 256 )
void rowBroadcastKernel( const float* matrix, float* result, const float* vector, int height, int width,
	long long total, int matBatchStride, int vecBatchStride )
{
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	const int hw = height * width;
	if( VEC ) {
		const long long total4 = total >> 2;
		for( long long i4 = blockIdx.x * 256LL + threadIdx.x; i4 < total4; i4 += step ) {
			const long long i = i4 << 2;
			const int b = static_cast<int>( i / hw );
			const int inMat = static_cast<int>( i - static_cast<long long>( b ) * hw );
			const int c = inMat % width;
			const float4 v = *reinterpret_cast<const float4*>( vector + static_cast<long long>( b ) * vecBatchStride + c );
			float4 m = make_float4( 0.f, 0.f, 0.f, 0.f );
			if( OP != BO_Set ) {
				m = *reinterpret_cast<const float4*>( matrix + static_cast<long long>( b ) * matBatchStride + inMat );
			}
			float4 r;
			r.x = broadcastApply<OP>( m.x, v.x );
			r.y = broadcastApply<OP>( m.y, v.y );
			r.z = broadcastApply<OP>( m.z, v.z );
			r.w = broadcastApply<OP>( m.w, v.w );
			*reinterpret_cast<float4*>( result + i ) = r;
		}
	} else {
		for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += step ) {
			const int b = static_cast<int>( i / hw );
			const int inMat = static_cast<int>( i - static_cast<long long>( b ) * hw );
			const int c = inMat % width;
			const float v = vector[static_cast<long long>( b ) * vecBatchStride + c];
			const float m = OP != BO_Set ? matrix[static_cast<long long>( b ) * matBatchStride + inMat] : 0.f;
			result[i] = broadcastApply<OP>( m, v );
		}
	}
}

template<int OP>
static int launchRowBroadcastOn( hipStream_t stream, const float* matrix, float* result, const float* vector, int batch,
	int height, int width, int matBatchStride, int vecBatchStride );

template<int OP>
static int launchRowBroadcast( nhStream s, const float* matrix, float* result, const float* vector, int batch,
	int height, int width, int matBatchStride, int vecBatchStride )
{
	return launchRowBroadcastOn<OP>( toStream( s ), matrix, result, vector, batch, height, width, matBatchStride, vecBatchStride );
}

template<int OP>
static int launchRowBroadcastOn( hipStream_t stream, const float* matrix, float* result, const float* vector, int batch,
	int height, int width, int matBatchStride, int vecBatchStride )
{
	const long long total = static_cast<long long>( batch ) * height * width;
	if( total == 0 ) {
		return NH_OK;
	}
	const bool vec = width % 4 == 0 && matBatchStride % 4 == 0 && vecBatchStride % 4 == 0 && isAligned16( result )
		&& isAligned16( vector ) && ( OP == BO_Set || isAligned16( matrix ) );
	const long long work = vec ? total / 4 : total;
	long long blocks = ( work + 1023 ) / 1024; // 4 items per thread
	blocks = blocks > 65536 ? 65536 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( ( rowBroadcastKernel<OP, true> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			matrix, result, vector, height, width, total, matBatchStride, vecBatchStride );
	} else {
		hipLaunchKernelGGL( ( rowBroadcastKernel<OP, false> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			matrix, result, vector, height, width, total, matBatchStride, vecBatchStride );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// Column broadcast: element ( r, c ) pairs with vector[r].
template<int OP, bool VEC>
__global__ __launch_bounds__( 256 )
void columnBroadcastKernel( const float* matrix, float* result, const float* vector, int width, long long total )
{
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	if( VEC ) {
		const long long total4 = total >> 2;
		for( long long i4 = blockIdx.x * 256LL + threadIdx.x; i4 < total4; i4 += step ) {
			const long long i = i4 << 2;
			const float v = vector[i / width];
			const float4 m = *reinterpret_cast<const float4*>( matrix + i );
			float4 r;
			r.x = broadcastApply<OP>( m.x, v );
			r.y = broadcastApply<OP>( m.y, v );
			r.z = broadcastApply<OP>( m.z, v );
			r.w = broadcastApply<OP>( m.w, v );
			*reinterpret_cast<float4*>( result + i ) = r;
		}
	} else {
		for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += step ) {
			result[i] = broadcastApply<OP>( matrix[i], vector[i / width] );
		}
	}
}

template<int OP>
static int launchColumnBroadcastOn( hipStream_t stream, const float* matrix, float* result, const float* vector, int height, int width );

template<int OP>
static int launchColumnBroadcast( nhStream s, const float* matrix, float* result, const float* vector, int height, int width )
{
	return launchColumnBroadcastOn<OP>( toStream( s ), matrix, result, vector, height, width );
}

template<int OP>
static int launchColumnBroadcastOn( hipStream_t stream, const float* matrix, float* result, const float* vector, int height, int width )
{
	const long long total = static_cast<long long>( height ) * width;
	if( total == 0 ) {
		return NH_OK;
	}
	const bool vec = width % 4 == 0 && isAligned16( result ) && isAligned16( matrix );
	const long long work = vec ? total / 4 : total;
	long long blocks = ( work + 1023 ) / 1024;
	blocks = blocks > 65536 ? 65536 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( ( columnBroadcastKernel<OP, true> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			matrix, result, vector, width, total );
	} else {
		hipLaunchKernelGGL( ( columnBroadcastKernel<OP, false> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, stream,
			matrix, result, vector, width, total );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// ---------------------------------------------------------------------------------------------------------
// Row reductions: one wavefront per row

constexpr int RowsPerBlock = 4; // 256 threads

// result[r] = sum_c matrix[r][c]
__global__ __launch_bounds__( 256 )
void sumColumnsKernel( float* result, const float* matrix, int height, int width, int vec )
{
	const int row = blockIdx.x * RowsPerBlock + ( threadIdx.x >> 6 );
	if( row >= height ) {
		return;
	}
	const int lane = threadIdx.x & 63;
	const float* p = matrix + static_cast<long long>( row ) * width;
	float s = 0.f;
	if( vec ) {
		const int w4 = width >> 2;
		for( int i = lane; i < w4; i += 64 ) {
			const float4 v = reinterpret_cast<const float4*>( p )[i];
			s += ( v.x + v.y ) + ( v.z + v.w );
		}
	} else {
		for( int i = lane; i < width; i += 64 ) {
			s += p[i];
		}
	}
	s = waveReduceSum( s );
	if( lane == 0 ) {
		result[row] = s;
	}
}

// result[b][c] (+)= sum_r matrix[b][r][c]; rows [rowBegin, rowEnd) of this slice, one thread per column.
// With several slices the partial sums meet in the result through atomic adds.
__global__ __launch_bounds__( 256 )
void sumRowsKernel( float* result, const float* matrix, int height, int width, int rowsPerSlice, int accumulate )
{
	const int c = blockIdx.x * 256 + threadIdx.x;
	if( c >= width ) {
		return;
	}
	const int b = blockIdx.y;
	const int rowBegin = blockIdx.z * rowsPerSlice;
	int rowEnd = rowBegin + rowsPerSlice;
	rowEnd = rowEnd > height ? height : rowEnd;
	const float* p = matrix + ( static_cast<long long>( b ) * height + rowBegin ) * width + c;
	float s = 0.f;
	for( int r = rowBegin; r < rowEnd; ++r ) {
		s += *p;
		p += width;
	}
	float* out = result + static_cast<long long>( b ) * width + c;
	if( gridDim.z > 1 ) {
		atomicAdd( out, s );
	} else if( accumulate ) {
		*out += s;
	} else {
		*out = s;
	}
}

// The same sums for a tall matrix of few columns (the free-term gradient of a convolution: one row per pixel of the
// batch). The 256 threads of a workgroup form 256 / groups row lanes of `groups` float4 columns, so that a wave reads
// whole rows back to back; every lane keeps four loads in flight, the lanes meet in LDS, one atomic add per column.
__global__ __launch_bounds__( 256 )
void sumTallRowsKernel( float* result, const float* matrix, int height, int width, int groups, int rowsPerSlice )
{
	__shared__ float4 meet[256];
	const int group = threadIdx.x % groups;
	const int lane = threadIdx.x / groups;
	const int lanes = 256 / groups;
	const int b = blockIdx.y;
	const int rowBegin = blockIdx.x * rowsPerSlice;
	const int rowEnd = min( rowBegin + rowsPerSlice, height );
	float4 sum[4];
#pragma unroll
	for( int j = 0; j < 4; ++j ) {
		sum[j] = make_float4( 0.f, 0.f, 0.f, 0.f );
	}
	if( group * 4 < width ) {
		const float* p = matrix + static_cast<long long>( b ) * height * width + group * 4;
		int r = rowBegin + lane;
		for( ; r + 3 * lanes < rowEnd; r += 4 * lanes ) {
			float4 v[4];
#pragma unroll
			for( int j = 0; j < 4; ++j ) {
				v[j] = *reinterpret_cast<const float4*>( p + static_cast<long long>( r + j * lanes ) * width );
			}
#pragma unroll
			for( int j = 0; j < 4; ++j ) {
				sum[j].x += v[j].x; sum[j].y += v[j].y; sum[j].z += v[j].z; sum[j].w += v[j].w;
			}
		}
		for( ; r < rowEnd; r += lanes ) {
			const float4 v = *reinterpret_cast<const float4*>( p + static_cast<long long>( r ) * width );
			sum[0].x += v.x; sum[0].y += v.y; sum[0].z += v.z; sum[0].w += v.w;
		}
	}
	meet[threadIdx.x] = make_float4( sum[0].x + sum[1].x + sum[2].x + sum[3].x, sum[0].y + sum[1].y + sum[2].y + sum[3].y,
		sum[0].z + sum[1].z + sum[2].z + sum[3].z, sum[0].w + sum[1].w + sum[2].w + sum[3].w );
	__syncthreads();
	// one thread per column adds up its lanes
	const int c = threadIdx.x;
	if( c < width ) {
		const float* column = reinterpret_cast<const float*>( meet ) + c;
		float total = 0.f;
		for( int l = 0; l < lanes; ++l ) {
			total += column[l * groups * 4];
		}
		atomicAdd( result + static_cast<long long>( b ) * width + c, total );
	}
}

// result[r] = <first[r], second[r]> (DIFF == false), or the softmax derivative expressed through the softmax's output:
// result[r][c] = first[r][c] * ( second[r][c] - <first[r], second[r]> ) with first = y, second = dE/dy
// (src/CPU/CpuMathEngineBlas.cpp:1161-1179). One row per wavefront.
template<bool DIFF>
__global__ __launch_bounds__( 256 )
void rowDotKernel( const float* first, const float* second, int height, int width, float* result )
{
	const int row = blockIdx.x * RowsPerBlock + ( threadIdx.x >> 6 );
	if( row >= height ) {
		return;
	}
	const int lane = threadIdx.x & 63;
	const float* a = first + static_cast<long long>( row ) * width;
	const float* b = second + static_cast<long long>( row ) * width;
	float dot = 0.f;
	for( int c = lane; c < width; c += 64 ) {
		dot += a[c] * b[c];
	}
	dot = waveReduceSum( dot );
	if( DIFF ) {
		float* out = result + static_cast<long long>( row ) * width;
		for( int c = lane; c < width; c += 64 ) {
			out[c] = a[c] * ( b[c] - dot );
		}
	} else if( lane == 0 ) {
		result[row] = dot;
	}
}

// result[j][c] += sum over b of first[b][j] * second[b][j][c]: one result matrix for the whole batch
// (src/CPU/x86/CpuX86MathEngineBlas.cpp:401-456)
__global__ __launch_bounds__( 256 )
void diagByMatrixAddKernel( int batchSize, const float* first, int firstSize, const float* second, int secondWidth, float* result )
{
	const long long total = static_cast<long long>( firstSize ) * secondWidth;
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		const int j = static_cast<int>( i / secondWidth );
		float sum = result[i];
		for( int b = 0; b < batchSize; ++b ) {
			sum += first[static_cast<long long>( b ) * firstSize + j] * second[b * total + i];
		}
		result[i] = sum;
	}
}

// Softmax / log-sum-exp of one row per wavefront. Rows of up to 64 * CACHE elements stay in registers between
// the three passes (max, sum of exp, scale); longer rows are read again from memory.
// The formula follows the reference: exp( x - max ) * ( 1 / sum ) (src/CPU/CpuMathEngineBlas.cpp:1131-1159).
template<int CACHE, bool LOGSUMEXP>
__global__ __launch_bounds__( 256 )
void softmaxRowsKernel( const float* matrix, int height, int width, float* result )
{
	const int row = blockIdx.x * RowsPerBlock + ( threadIdx.x >> 6 );
	if( row >= height ) {
		return;
	}
	const int lane = threadIdx.x & 63;
	const float* p = matrix + static_cast<long long>( row ) * width;
	float cache[CACHE > 0 ? CACHE : 1];
	float mx = -FLT_MAX;
	if( CACHE > 0 ) {
#pragma unroll
		for( int j = 0; j < CACHE; ++j ) {
			const int i = lane + j * 64;
			cache[j] = i < width ? p[i] : -FLT_MAX;
			mx = fmaxf( mx, cache[j] );
		}
	} else {
		for( int i = lane; i < width; i += 64 ) {
			mx = fmaxf( mx, p[i] );
		}
	}
	mx = waveReduceMax( mx );
	float sum = 0.f;
	if( CACHE > 0 ) {
#pragma unroll
		for( int j = 0; j < CACHE; ++j ) {
			const int i = lane + j * 64;
			cache[j] = i < width ? expf( cache[j] - mx ) : 0.f;
			sum += cache[j];
		}
	} else {
		for( int i = lane; i < width; i += 64 ) {
			sum += expf( p[i] - mx );
		}
	}
	sum = waveReduceSum( sum );
	if( LOGSUMEXP ) {
		if( lane == 0 ) {
			result[row] = mx + logf( sum );
		}
		return;
	}
	const float inv = 1.f / sum;
	float* q = result + static_cast<long long>( row ) * width;
	if( CACHE > 0 ) {
#pragma unroll
		for( int j = 0; j < CACHE; ++j ) {
			const int i = lane + j * 64;
			if( i < width ) {
				q[i] = cache[j] * inv;
			}
		}
	} else {
		for( int i = lane; i < width; i += 64 ) {
			q[i] = expf( p[i] - mx ) * inv;
		}
	}
}

// Maximum of a row and the index of its first occurrence
__global__ __launch_bounds__( 256 )
void findMaxInRowsKernel( const float* matrix, int height, int width, float* result, int* indices )
{
	const int row = blockIdx.x * RowsPerBlock + ( threadIdx.x >> 6 );
	if( row >= height ) {
		return;
	}
	const int lane = threadIdx.x & 63;
	const float* p = matrix + static_cast<long long>( row ) * width;
	float best = -FLT_MAX;
	int bestIdx = 0x7fffffff;
	for( int i = lane; i < width; i += 64 ) {
		const float v = p[i];
		if( bestIdx == 0x7fffffff || v > best ) {
			best = v;
			bestIdx = i;
		}
	}
	waveReduceArgMax( best, bestIdx );
	if( lane == 0 ) {
		result[row] = best;
		if( indices != nullptr ) {
			indices[row] = bestIdx;
		}
	}
}

// Maximum of every column of each [height x width] matrix of the batch; first row wins ties
__global__ __launch_bounds__( 256 )
void findMaxInColumnsKernel( const float* matrix, int height, int width, float* result, int* indices )
{
	const int c = blockIdx.x * 256 + threadIdx.x;
	if( c >= width ) {
		return;
	}
	const int b = blockIdx.y;
	const float* p = matrix + static_cast<long long>( b ) * height * width + c;
	float best = *p;
	int bestIdx = 0;
	for( int r = 1; r < height; ++r ) {
		p += width;
		const float v = *p;
		if( v > best ) {
			best = v;
			bestIdx = r;
		}
	}
	result[static_cast<long long>( b ) * width + c] = best;
	indices[static_cast<long long>( b ) * width + c] = bestIdx;
}

// ---------------------------------------------------------------------------------------------------------
// Transpose [b, h, m, w, c] -> [b, w, m, h, c]

// General form: one thread per group of VECW output elements (VECW divides c); reads are contiguous runs of c.
template<typename T, int VECW>
__global__ __launch_bounds__( 256 )
void transposeCellsKernel( const T* in, T* out, int height, int medium, int width, int channels, long long totalGroups )
{
	const int cg = channels / VECW;
	const long long step = static_cast<long long>( gridDim.x ) * 256;
	for( long long g = blockIdx.x * 256LL + threadIdx.x; g < totalGroups; g += step ) {
		long long t = g;
		const int ch = static_cast<int>( t % cg ) * VECW; t /= cg;
		const int j = static_cast<int>( t % height ); t /= height;
		const int m = static_cast<int>( t % medium ); t /= medium;
		const int i = static_cast<int>( t % width ); t /= width;
		const long long b = t;
		const long long src = ( ( ( b * height + j ) * medium + m ) * width + i ) * channels + ch;
		const long long dst = g * VECW;
		if( VECW == 4 ) {
			*reinterpret_cast<int4*>( out + dst ) = *reinterpret_cast<const int4*>( in + src );
		} else {
			out[dst] = in[src];
		}
	}
}

// Plain matrices (m == 1, c == 1): 64x64 tiles through LDS so that both the read and the write are coalesced.
template<typename T>
__global__ __launch_bounds__( 256 )
void transposePlainKernel( const T* in, T* out, int height, int width )
{
	__shared__ T tile[64][65];
	const long long base = static_cast<long long>( blockIdx.z ) * height * width;
	const int x0 = blockIdx.x * 64;
	const int y0 = blockIdx.y * 64;
	const int tx = threadIdx.x & 63;
	const int ty = threadIdx.x >> 6;
	for( int r = ty; r < 64; r += 4 ) {
		const int y = y0 + r;
		const int x = x0 + tx;
		if( y < height && x < width ) {
			tile[r][tx] = in[base + static_cast<long long>( y ) * width + x];
		}
	}
	__syncthreads();
	for( int r = ty; r < 64; r += 4 ) {
		const int x = x0 + r; // row of the result
		const int y = y0 + tx;
		if( x < width && y < height ) {
			out[base + static_cast<long long>( x ) * height + y] = tile[tx][r];
		}
	}
}

// The same with 128-bit accesses to memory ( both dimensions multiples of 4, 16-byte aligned ): a thread reads four
// neighbours of a row, leaves them in a column of the tile, and collects four neighbours of a result row from four rows of it.
template<typename T>
__global__ __launch_bounds__( 256 )
void transposePlainQuadKernel( const T* in, T* out, int height, int width )
{
	static_assert( sizeof( T ) == 4, "four elements are 128 bits" );
	__shared__ T tile[64][65];
	const long long base = static_cast<long long>( blockIdx.z ) * height * width;
	const int x0 = blockIdx.x * 64;
	const int y0 = blockIdx.y * 64;
	const int q4 = ( threadIdx.x & 15 ) * 4;
	const int r0 = threadIdx.x >> 4;
	int4 v[4];
#pragma unroll
	for( int k = 0; k < 4; ++k ) {
		const int y = y0 + r0 + 16 * k, x = x0 + q4;
		v[k] = make_int4( 0, 0, 0, 0 );
		if( y < height && x < width ) {
			v[k] = *reinterpret_cast<const int4*>( in + base + static_cast<long long>( y ) * width + x );
		}
	}
#pragma unroll
	for( int k = 0; k < 4; ++k ) {
		int* row = reinterpret_cast<int*>( &tile[r0 + 16 * k][q4] );
		row[0] = v[k].x; row[1] = v[k].y; row[2] = v[k].z; row[3] = v[k].w;
	}
	__syncthreads();
#pragma unroll
	for( int k = 0; k < 4; ++k ) {
		const int xr = r0 + 16 * k; // row of the result inside the tile
		const int x = x0 + xr, y = y0 + q4;
		if( x < width && y < height ) {
			int4 w;
			w.x = *reinterpret_cast<const int*>( &tile[q4 + 0][xr] );
			w.y = *reinterpret_cast<const int*>( &tile[q4 + 1][xr] );
			w.z = *reinterpret_cast<const int*>( &tile[q4 + 2][xr] );
			w.w = *reinterpret_cast<const int*>( &tile[q4 + 3][xr] );
			*reinterpret_cast<int4*>( out + base + static_cast<long long>( x ) * height + y ) = w;
		}
	}
}

template<typename T>
static int transposeImpl( nhStream s, int batchSize, const T* first, int height, int medium, int width, int channels,
	T* result, int resultBufferSize )
{
	if( batchSize < 0 || height < 0 || medium < 0 || width < 0 || channels < 0 ) {
		setLastError( "TransposeMatrix: negative dimension" );
		return NH_ERR_ARGUMENT;
	}
	// resultBufferSize is not looked at: the reference CPU engine ignores it too (src/CPU/CpuMathEngineBlas.cpp:152-163)
	( void )resultBufferSize;
	const long long total = static_cast<long long>( batchSize ) * height * medium * width * channels;
	if( total == 0 ) {
		return NH_OK;
	}
	if( first == result ) {
		setLastError( "TransposeMatrix: in-place transposition is not supported" );
		return NH_ERR_ARGUMENT;
	}
	if( height == 1 || width == 1 ) {
		// [b,1,m,w,c] -> [b,w,m,1,c] moves whole rows when m == 1 and is a (w x m) cell transpose otherwise
		if( medium == 1 ) {
			NH_HIP( hipMemcpyAsync( result, first, total * sizeof( T ), hipMemcpyDeviceToDevice, toStream( s ) ) );
			return NH_OK;
		}
	}
	if( medium == 1 && channels == 1 ) {
		const dim3 grid( ceilDiv( width, 64 ), ceilDiv( height, 64 ), batchSize );
		if( grid.y <= 65535 && grid.z <= 65535 && height % 4 == 0 && width % 4 == 0 && isAligned16( first ) && isAligned16( result ) ) {
			hipLaunchKernelGGL( transposePlainQuadKernel<T>, grid, dim3( 256 ), 0, toStream( s ), first, result, height, width );
			NH_LAUNCH_CHECK();
			return NH_OK;
		}
		if( grid.y <= 65535 && grid.z <= 65535 ) {
			hipLaunchKernelGGL( transposePlainKernel<T>, grid, dim3( 256 ), 0, toStream( s ), first, result, height, width );
			NH_LAUNCH_CHECK();
			return NH_OK;
		}
	}
	const bool vec = channels % 4 == 0 && isAligned16( first ) && isAligned16( result );
	const long long groups = vec ? total / 4 : total;
	long long blocks = ( groups + 255 ) / 256;
	blocks = blocks > 262144 ? 262144 : blocks;
	if( vec ) {
		hipLaunchKernelGGL( ( transposeCellsKernel<T, 4> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			first, result, height, medium, width, channels, groups );
	} else {
		hipLaunchKernelGGL( ( transposeCellsKernel<T, 1> ), dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
			first, result, height, medium, width, channels, groups );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

} // namespace nh

using namespace nh;

static int sumMatrixRowsImpl( nhStream s, int batchSize, float* result, const float* matrix, int matrixHeight,
	int matrixWidth, bool accumulate )
{
	if( batchSize == 0 || matrixWidth == 0 ) {
		return NH_OK;
	}
	if( matrixWidth % 4 == 0 && matrixWidth <= 256 && matrixHeight >= 2048 && batchSize <= 65535 && isAligned16( matrix ) ) {
		int groups = 1;
		while( groups * 4 < matrixWidth ) {
			groups *= 2;
		}
		const int lanes = 256 / groups;
		// about 256 workgroups ( every workgroup ends with one atomic add per column, all on the same few addresses: 784
		// workgroups took 25 us for 200 704 x 64, 256 take 14 us ), at least 16 rows per lane
		int slices = 256 / batchSize > 0 ? 256 / batchSize : 1;
		const int most = matrixHeight / ( 16 * lanes ) > 0 ? matrixHeight / ( 16 * lanes ) : 1;
		slices = slices < most ? slices : most;
		const int rowsPerSlice = ceilDiv( matrixHeight, slices );
		slices = ceilDiv( matrixHeight, rowsPerSlice );
		if( !accumulate ) {
			const int rc = nhVectorFill( s, result, 0.f, batchSize * matrixWidth );
			if( rc != NH_OK ) {
				return rc;
			}
		}
		hipLaunchKernelGGL( sumTallRowsKernel, dim3( slices, batchSize ), dim3( 256 ), 0, toStream( s ),
			result, matrix, matrixHeight, matrixWidth, groups, rowsPerSlice );
		NH_LAUNCH_CHECK();
		return NH_OK;
	}
	const int colBlocks = ceilDiv( matrixWidth, 256 );
	// split tall matrices over several workgroups until about 1024 of them exist
	int slices = 1;
	const long long base = static_cast<long long>( colBlocks ) * batchSize;
	if( base < 512 && matrixHeight >= 256 ) {
		slices = static_cast<int>( 1024 / base );
		const int maxSlices = matrixHeight / 64;
		slices = slices > maxSlices ? maxSlices : slices;
		slices = slices < 1 ? 1 : slices;
	}
	if( slices > 1 && !accumulate ) {
		const int rc = nhVectorFill( s, result, 0.f, batchSize * matrixWidth );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	const int rowsPerSlice = ceilDiv( matrixHeight, slices );
	slices = matrixHeight == 0 ? 1 : ceilDiv( matrixHeight, rowsPerSlice );
	if( batchSize > 65535 || slices > 65535 ) {
		setLastError( "SumMatrixRows: batch is too large" );
		return NH_ERR_ARGUMENT;
	}
	hipLaunchKernelGGL( sumRowsKernel, dim3( colBlocks, batchSize, slices ), dim3( 256 ), 0, toStream( s ),
		result, matrix, matrixHeight, matrixWidth, rowsPerSlice, accumulate ? 1 : 0 );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

template<bool LOGSUMEXP>
static int softmaxImpl( nhStream s, const float* matrix, int height, int width, float* result )
{
	if( height == 0 || width == 0 ) {
		return NH_OK;
	}
	const dim3 grid( ceilDiv( height, RowsPerBlock ) );
	if( width <= 64 ) {
		hipLaunchKernelGGL( ( softmaxRowsKernel<1, LOGSUMEXP> ), grid, dim3( 256 ), 0, toStream( s ), matrix, height, width, result );
	} else if( width <= 256 ) {
		hipLaunchKernelGGL( ( softmaxRowsKernel<4, LOGSUMEXP> ), grid, dim3( 256 ), 0, toStream( s ), matrix, height, width, result );
	} else if( width <= 1024 ) {
		hipLaunchKernelGGL( ( softmaxRowsKernel<16, LOGSUMEXP> ), grid, dim3( 256 ), 0, toStream( s ), matrix, height, width, result );
	} else {
		hipLaunchKernelGGL( ( softmaxRowsKernel<0, LOGSUMEXP> ), grid, dim3( 256 ), 0, toStream( s ), matrix, height, width, result );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// The launch of a call with a spread vector that a stream had put aside and nothing joined
static void launchSpreadAlone( hipStream_t stream, bool multiply, int spread, const float* matrix, const float* vector, float* result,
	int height, int width )
{
	// ( a launch that fails leaves its HIP error to the next launch check )
	if( spread == TS_PerRow ) {
		( void )( multiply ? launchColumnBroadcastOn<BO_Mul>( stream, matrix, result, vector, height, width )
			: launchColumnBroadcastOn<BO_Add>( stream, matrix, result, vector, height, width ) );
	} else {
		( void )( multiply ? launchRowBroadcastOn<BO_Mul>( stream, matrix, result, vector, 1, height, width, 0, 0 )
			: launchRowBroadcastOn<BO_Add>( stream, matrix, result, vector, 1, height, width, 0, 0 ) );
	}
}

extern "C" {


int nhSetVectorToMatrixRows( nhStream s, float* result, int matrixHeight, int matrixWidth, const float* vector )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth >= 0 );
	return launchRowBroadcast<BO_Set>( s, nullptr, result, vector, 1, matrixHeight, matrixWidth, 0, 0 );
}

int nhAddVectorToMatrixRows( nhStream s, int batchSize, const float* matrix, float* result,
	int matrixHeight, int matrixWidth, const float* vector )
{
	NH_REQUIRE( batchSize >= 0 && matrixHeight >= 0 && matrixWidth >= 0 );
	NH_REQUIRE( static_cast<long long>( matrixHeight ) * matrixWidth <= 0x7fffffffLL );
	int rc = NH_OK;
	if( batchSize == 1 && __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0
		&& fusePendingProduct( s, matrix, result, matrixHeight, matrixWidth, vector, &rc ) )
	{
		return rc; // ( the product that waited for this call took the vector with it )
	}
	if( batchSize == 1 && deferSpreadOp( s, false, TS_PerColumn, matrix, vector, result, matrixHeight, matrixWidth, &launchSpreadAlone ) ) {
		return NH_OK;
	}
	return launchRowBroadcast<BO_Add>( s, matrix, result, vector, batchSize, matrixHeight, matrixWidth,
		matrixHeight * matrixWidth, matrixWidth );
}

int nhAddVectorToMatrixColumns( nhStream s, const float* matrix, float* result, int matrixHeight, int matrixWidth,
	const float* vector )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth >= 0 );
	// ( on a stream that puts calls aside: one of a run of passes over the matrix, CObjectNormalizationLayer's four last calls )
	if( deferSpreadOp( s, false, TS_PerRow, matrix, vector, result, matrixHeight, matrixWidth, &launchSpreadAlone ) ) {
		return NH_OK;
	}
	return launchColumnBroadcast<BO_Add>( s, matrix, result, vector, matrixHeight, matrixWidth );
}

int nhSubVectorFromMatrixColumns( nhStream s, const float* matrix, float* result, int matrixHeight, int matrixWidth,
	const float* vector )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth >= 0 );
	return launchColumnBroadcast<BO_Sub>( s, matrix, result, vector, matrixHeight, matrixWidth );
}

int nhMultiplyDiagMatrixByMatrix( nhStream s, const float* first, int firstSize, const float* second,
	int secondWidth, float* result, int resultBufferSize )
{
	NH_REQUIRE( firstSize >= 0 && secondWidth >= 0 );
	NH_REQUIRE( static_cast<long long>( firstSize ) * secondWidth <= resultBufferSize );
	if( deferSpreadOp( s, true, TS_PerRow, second, first, result, firstSize, secondWidth, &launchSpreadAlone ) ) {
		return NH_OK;
	}
	return launchColumnBroadcast<BO_Mul>( s, second, result, first, firstSize, secondWidth );
}

int nhMultiplyDiagMatrixByMatrixAndAdd( nhStream s, int batchSize, const float* first, int firstSize, const float* second,
	int secondWidth, float* result )
{
	NH_REQUIRE( batchSize >= 0 && firstSize >= 0 && secondWidth >= 0 );
	const long long total = static_cast<long long>( firstSize ) * secondWidth;
	if( total == 0 || batchSize == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( first != nullptr && second != nullptr && result != nullptr );
	long long blocks = ( total + 255 ) / 256;
	blocks = blocks > 1048576 ? 1048576 : blocks;
	hipLaunchKernelGGL( diagByMatrixAddKernel, dim3( static_cast<unsigned>( blocks ) ), dim3( 256 ), 0, toStream( s ),
		batchSize, first, firstSize, second, secondWidth, result );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhRowMultiplyMatrixByMatrix( nhStream s, const float* first, const float* second, int height, int width, float* result )
{
	NH_REQUIRE( height >= 0 && width >= 0 );
	if( height == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( first != nullptr && second != nullptr && result != nullptr );
	hipLaunchKernelGGL( rowDotKernel<false>, dim3( ceilDiv( height, RowsPerBlock ) ), dim3( 256 ), 0, toStream( s ),
		first, second, height, width, result );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhMatrixSoftmaxDiffOpByRows( nhStream s, const float* first, const float* second, int height, int width, float* result )
{
	NH_REQUIRE( height >= 0 && width >= 0 );
	if( height == 0 || width == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( first != nullptr && second != nullptr && result != nullptr );
	hipLaunchKernelGGL( rowDotKernel<true>, dim3( ceilDiv( height, RowsPerBlock ) ), dim3( 256 ), 0, toStream( s ),
		first, second, height, width, result );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhBatchMultiplyMatrixByDiagMatrix( nhStream s, int batchSize, const float* first, int height, int width,
	int firstMatrixOffset, const float* second, int secondMatrixOffset, float* result, int resultBufferSize )
{
	NH_REQUIRE( batchSize >= 0 && height >= 0 && width >= 0 && firstMatrixOffset >= 0 && secondMatrixOffset >= 0 );
	NH_REQUIRE( static_cast<long long>( batchSize ) * height * width <= resultBufferSize );
	if( batchSize == 1 && deferSpreadOp( s, true, TS_PerColumn, first, second, result, height, width, &launchSpreadAlone ) ) {
		return NH_OK;
	}
	return launchRowBroadcast<BO_Mul>( s, first, result, second, batchSize, height, width, firstMatrixOffset, secondMatrixOffset );
}

int nhSumMatrixRows( nhStream s, int batchSize, float* result, const float* matrix, int matrixHeight, int matrixWidth )
{
	NH_REQUIRE( batchSize >= 0 && matrixHeight >= 0 && matrixWidth >= 0 );
	return sumMatrixRowsImpl( s, batchSize, result, matrix, matrixHeight, matrixWidth, false );
}

int nhSumMatrixRowsAdd( nhStream s, int batchSize, float* result, const float* matrix, int matrixHeight, int matrixWidth )
{
	NH_REQUIRE( batchSize >= 0 && matrixHeight >= 0 && matrixWidth >= 0 );
	return sumMatrixRowsImpl( s, batchSize, result, matrix, matrixHeight, matrixWidth, true );
}

int nhSumMatrixColumns( nhStream s, float* result, const float* matrix, int matrixHeight, int matrixWidth )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth >= 0 );
	if( matrixHeight == 0 ) {
		return NH_OK;
	}
	// ( on a stream that puts calls aside the sums wait for the small calls in place over them: one launch with those )
	if( matrixWidth > 0 && deferColumnSum( s, result, matrix, matrixHeight, matrixWidth ) ) {
		return NH_OK;
	}
	const int vec = ( matrixWidth % 4 == 0 && isAligned16( matrix ) ) ? 1 : 0;
	hipLaunchKernelGGL( sumColumnsKernel, dim3( ceilDiv( matrixHeight, RowsPerBlock ) ), dim3( 256 ), 0, toStream( s ),
		result, matrix, matrixHeight, matrixWidth, vec );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhMatrixSoftmaxByRows( nhStream s, const float* matrix, int height, int width, float* result )
{
	NH_REQUIRE( height >= 0 && width >= 0 );
	return softmaxImpl<false>( s, matrix, height, width, result );
}

int nhMatrixLogSumExpByRows( nhStream s, const float* matrix, int height, int width, float* result, int resultSize )
{
	NH_REQUIRE( height >= 0 && width >= 0 && resultSize >= height );
	return softmaxImpl<true>( s, matrix, height, width, result );
}

int nhFindMaxValueInRows( nhStream s, const float* matrix, int matrixHeight, int matrixWidth,
	float* result, int* columnIndices, int vectorSize )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth > 0 && vectorSize >= matrixHeight );
	if( matrixHeight == 0 ) {
		return NH_OK;
	}
	hipLaunchKernelGGL( findMaxInRowsKernel, dim3( ceilDiv( matrixHeight, RowsPerBlock ) ), dim3( 256 ), 0, toStream( s ),
		matrix, matrixHeight, matrixWidth, result, columnIndices );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhFindMaxValueInColumns( nhStream s, int batchSize, const float* matrix, int matrixHeight,
	int matrixWidth, float* result, int* rowIndices, int vectorSize )
{
	NH_REQUIRE( batchSize >= 0 && matrixHeight > 0 && matrixWidth >= 0 && rowIndices != nullptr );
	NH_REQUIRE( static_cast<long long>( batchSize ) * matrixWidth <= vectorSize && batchSize <= 65535 );
	if( batchSize == 0 || matrixWidth == 0 ) {
		return NH_OK;
	}
	hipLaunchKernelGGL( findMaxInColumnsKernel, dim3( ceilDiv( matrixWidth, 256 ), batchSize ), dim3( 256 ), 0, toStream( s ),
		matrix, matrixHeight, matrixWidth, result, rowIndices );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhTransposeMatrix( nhStream s, int batchSize, const float* first, int height, int medium, int width,
	int channels, float* result, int resultBufferSize )
{
	return transposeImpl<float>( s, batchSize, first, height, medium, width, channels, result, resultBufferSize );
}

int nhTransposeMatrixInt( nhStream s, int batchSize, const int* first, int height, int medium, int width,
	int channels, int* result, int resultBufferSize )
{
	return transposeImpl<int>( s, batchSize, first, height, medium, width, channels, result, resultBufferSize );
}

} // extern "C"
