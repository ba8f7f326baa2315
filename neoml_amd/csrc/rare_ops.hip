// Interface members that no network of the benchmark configurations calls: the recurrent parts of QRNN and IndRNN,
// BERT's light-weight convolution, local response normalization, products with a sparse (CSR) matrix, top-k, 3-D
// convolution and pooling, the decoder of run-length encoded images. Plain kernels, one thread per result element (or
// per independent recurrence), written for coverage of the interface; semantics are the reference CPU engine's, cited
// per kernel.
#include "common.h"
#include <float.h>

namespace nh {

static inline unsigned gridFor( long long total )
{
	const long long blocks = ( total + 255 ) / 256;
	return static_cast<unsigned>( blocks > 16384 ? 16384 : ( blocks < 1 ? 1 : blocks ) );
}

#define NH_FOR_EACH( i, total ) \
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < ( total ); i += static_cast<long long>( gridDim.x ) * 256 )

#define NH_LAUNCH( kernel, total, ... ) \
	do { \
		if( ( total ) > 0 ) { \
			hipLaunchKernelGGL( kernel, dim3( gridFor( total ) ), dim3( 256 ), 0, toStream( s ), __VA_ARGS__ ); \
			NH_LAUNCH_CHECK(); \
		} \
	} while( 0 )

// ---- QRNN poolings ( src/CPU/CpuMathEngineDnn.cpp:388-650 ) ------------------------------------------------------
// One thread owns one element of the object and walks the sequence: the recurrence is independent per element.

// h_t = f_t h_(t-1) + ( 1 - f_t ) z_t, or with an input gate h_t = f_t h_(t-1) + i_t z_t; without an initial state h_(-1) = 0
__global__ __launch_bounds__( 256 )
void qrnnPoolingKernel( int reverse, int length, int objectSize, const float* z, const float* f, const float* gate, const float* h0,
	float* result )
{
	NH_FOR_EACH( index, objectSize ) {
		float h = h0 != nullptr ? h0[index] : 0.f;
		for( int step = 0; step < length; ++step ) {
			const long long at = static_cast<long long>( reverse ? length - 1 - step : step ) * objectSize + index;
			const float fv = f[at];
			const float zv = z[at];
			h = fv * h + ( gate != nullptr ? gate[at] : 1.f - fv ) * zv;
			result[at] = h;
		}
	}
}

// The reference walks the sequence in the direction `reverse` names, reads the state "before" an element at the next
// position of that walk, and adds each element's recurrent share onto the gradient of that next position, in place.
__global__ __launch_bounds__( 256 )
void qrnnPoolingBackwardKernel( int reverse, int length, int objectSize, const float* z, const float* f, const float* gate,
	const float* h0, const float* out, float* outDiff, float* zDiff, float* fDiff, float* gateDiff )
{
	NH_FOR_EACH( index, objectSize ) {
		for( int step = 0; step < length; ++step ) {
			const long long at = static_cast<long long>( reverse ? length - 1 - step : step ) * objectSize + index;
			const long long before = at + ( reverse ? -objectSize : objectSize );
			const bool last = step == length - 1;
			const float d = outDiff[at];
			const float previous = last ? ( h0 != nullptr ? h0[index] : 0.f ) : out[before];
			if( gate != nullptr ) {
				zDiff[at] = d * gate[at];
				fDiff[at] = d * previous;
				gateDiff[at] = d * z[at];
			} else {
				zDiff[at] = d * ( 1.f - f[at] );
				fDiff[at] = d * ( previous - z[at] );
			}
			if( !last ) {
				outDiff[before] += d * f[at];
			}
		}
	}
}

// ---- IndRNN ( src/CPU/CpuMathEngineDnn.cpp:652-829 ) -------------------------------------------------------------

__device__ __forceinline__ float indRnnActivation( int relu, float x )
{
	if( relu ) {
		return x > 0.f ? x : 0.f;
	}
	// the two-sided form the reference uses: no overflow for large |x|
	if( x <= 0.f ) {
		const float e = __expf( x );
		return e / ( e + 1.f );
	}
	return 1.f / ( 1.f + __expf( -x ) );
}

__device__ __forceinline__ float indRnnActivationDiffOp( int relu, float out, float diff )
{
	return relu ? ( out > 0.f ? diff : 0.f ) : diff * out * ( 1.f - out );
}

// h_t = act( wx_t + u * mask * h_(t-1) ), per element of [batch x object]
__global__ __launch_bounds__( 256 )
void indRnnKernel( int reverse, int length, int batch, int objectSize, int relu, const float* wx, const float* mask, const float* u,
	float* h )
{
	const long long stepSize = static_cast<long long>( batch ) * objectSize;
	NH_FOR_EACH( index, stepSize ) {
		const float weight = u[index % objectSize] * ( mask != nullptr ? mask[index] : 1.f );
		float previous = 0.f;
		for( int step = 0; step < length; ++step ) {
			const long long at = static_cast<long long>( reverse ? length - 1 - step : step ) * stepSize + index;
			const float x = step == 0 ? wx[at] : wx[at] + weight * previous;
			previous = indRnnActivation( relu, x );
			h[at] = previous;
		}
	}
}

// Walks like the QRNN gradients: the gradient that reaches an element is its own plus what the element before it in the
// walk hands on ( activation derivative x u x mask ). learn != 0: sums the gradient by u instead of writing wxDiff.
__global__ __launch_bounds__( 256 )
void indRnnBackwardKernel( int reverse, int length, int batch, int objectSize, int relu, const float* mask, const float* u,
	const float* h, const float* hDiff, float* wxDiff, float* uDiff )
{
	const long long stepSize = static_cast<long long>( batch ) * objectSize;
	NH_FOR_EACH( index, stepSize ) {
		const int channel = static_cast<int>( index % objectSize );
		const float maskValue = mask != nullptr ? mask[index] : 1.f;
		const float weight = u[channel] * maskValue;
		float total = 0.f;
		float uSum = 0.f;
		for( int step = 0; step < length; ++step ) {
			const long long at = static_cast<long long>( reverse ? length - 1 - step : step ) * stepSize + index;
			total = step == 0 ? hDiff[at] : hDiff[at] + total;
			const float through = indRnnActivationDiffOp( relu, h[at], total );
			if( wxDiff != nullptr ) {
				wxDiff[at] = through;
			}
			if( step < length - 1 ) {
				const long long next = at + ( reverse ? -stepSize : stepSize );
				uSum += through * h[next] * maskValue;
			}
			total = through * weight;
		}
		if( uDiff != nullptr ) {
			atomicAdd( uDiff + channel, uSum );
		}
	}
}

// ---- BERT convolution ( src/CPU/CpuMathEngineDnn.cpp, BertConv / BertConvBackward ) --------------------------------
// output[seq][b][h] = sum_k data[seq - pad + k][b][h] * kernel[seq][b][k], b over batch x heads, pad = ( kernelSize - 1 ) / 2

__global__ __launch_bounds__( 256 )
void bertConvKernel( const float* data, const float* kernel, int seqLen, int lanes, int headSize, int kernelSize, float* output )
{
	const long long total = static_cast<long long>( seqLen ) * lanes * headSize;
	const int pad = ( kernelSize - 1 ) / 2;
	NH_FOR_EACH( i, total ) {
		const long long row = i / headSize; // seq * lanes + b
		const int seq = static_cast<int>( row / lanes );
		const long long inStep = static_cast<long long>( lanes ) * headSize;
		const long long inSeq = i - seq * inStep;
		float sum = 0.f;
		for( int k = 0; k < kernelSize; ++k ) {
			const int from = seq - pad + k;
			if( from >= 0 && from < seqLen ) {
				sum += data[from * inStep + inSeq] * kernel[row * kernelSize + k];
			}
		}
		output[i] = sum;
	}
}

__global__ __launch_bounds__( 256 )
void bertConvDataDiffKernel( const float* kernel, const float* outDiff, int seqLen, int lanes, int headSize, int kernelSize, float* dataDiff )
{
	const long long total = static_cast<long long>( seqLen ) * lanes * headSize;
	const int pad = ( kernelSize - 1 ) / 2;
	NH_FOR_EACH( i, total ) {
		const long long row = i / headSize;
		const int seq = static_cast<int>( row / lanes );
		const long long b = row - static_cast<long long>( seq ) * lanes;
		const long long inStep = static_cast<long long>( lanes ) * headSize;
		const long long inSeq = i - seq * inStep;
		float sum = 0.f;
		for( int k = 0; k < kernelSize; ++k ) {
			const int to = seq + pad - k; // the output position that read this element through tap k
			if( to >= 0 && to < seqLen ) {
				sum += outDiff[to * inStep + inSeq] * kernel[( static_cast<long long>( to ) * lanes + b ) * kernelSize + k];
			}
		}
		dataDiff[i] = sum;
	}
}

__global__ __launch_bounds__( 256 )
void bertConvKernelDiffKernel( const float* data, const float* outDiff, int seqLen, int lanes, int headSize, int kernelSize, float* kernelDiff )
{
	const long long total = static_cast<long long>( seqLen ) * lanes * kernelSize;
	const int pad = ( kernelSize - 1 ) / 2;
	NH_FOR_EACH( i, total ) {
		const long long row = i / kernelSize;
		const int k = static_cast<int>( i - row * kernelSize );
		const int seq = static_cast<int>( row / lanes );
		const long long b = row - static_cast<long long>( seq ) * lanes;
		const int from = seq - pad + k;
		float sum = 0.f;
		if( from >= 0 && from < seqLen ) {
			const float* d = data + ( static_cast<long long>( from ) * lanes + b ) * headSize;
			const float* o = outDiff + row * headSize;
			for( int h = 0; h < headSize; ++h ) {
				sum += d[h] * o[h];
			}
		}
		kernelDiff[i] = sum;
	}
}

// ---- local response normalization ( src/CPU/CpuMathEngineDnnLrn.cpp:33-98 ) -------------------------------------
// invSum = 1 / ( bias + alpha / window * sum of squares over the channel window ), output = invSum^beta * input

__global__ __launch_bounds__( 256 )
void lrnKernel( const float* input, long long total, int vectorSize, int windowSize, float bias, float scale, float beta,
	float* invSum, float* invSumBeta, float* output )
{
	NH_FOR_EACH( i, total ) {
		const long long vec = i / vectorSize;
		const int ch = static_cast<int>( i - vec * vectorSize );
		const int first = max( 0, ch - ( windowSize - 1 ) / 2 );
		const int last = min( vectorSize - 1, ch + windowSize / 2 );
		const float* row = input + vec * vectorSize;
		float sum = 0.f;
		for( int c = first; c <= last; ++c ) {
			sum += row[c] * row[c];
		}
		const float inv = 1.f / ( sum * scale + bias );
		const float powered = powf( inv, beta );
		if( invSum != nullptr ) {
			invSum[i] = inv;
		}
		if( invSumBeta != nullptr ) {
			invSumBeta[i] = powered;
		}
		output[i] = powered * row[ch];
	}
}

// inputDiff = invSumBeta * outputDiff + input * scale * sum over the mirrored window of ( output * outputDiff * invSum )
__global__ __launch_bounds__( 256 )
void lrnBackwardKernel( const float* input, const float* output, const float* outputDiff, const float* invSum, const float* invSumBeta,
	long long total, int vectorSize, int windowSize, float scale, float* inputDiff )
{
	NH_FOR_EACH( i, total ) {
		const long long vec = i / vectorSize;
		const int ch = static_cast<int>( i - vec * vectorSize );
		const int first = max( 0, ch - windowSize / 2 );
		const int last = min( vectorSize - 1, ch + ( windowSize - 1 ) / 2 );
		const long long base = vec * vectorSize;
		float sum = 0.f;
		for( int c = first; c <= last; ++c ) {
			sum += output[base + c] * outputDiff[base + c] * invSum[base + c];
		}
		inputDiff[i] = sum * scale * input[i] + invSumBeta[i] * outputDiff[i];
	}
}

// ---- products with a sparse matrix in CSR form ( src/CPU/x86/CpuX86MathEngineBlasMkl.cpp:196-400 ) ----------------

// result[fh x sh] = sparse[fh x fw] * dense[sh x fw]^T
__global__ __launch_bounds__( 256 )
void sparseByTransposedKernel( const int* rows, const int* columns, const float* values, const float* second, int firstHeight,
	int firstWidth, int secondHeight, float* result )
{
	NH_FOR_EACH( i, static_cast<long long>( firstHeight ) * secondHeight ) {
		const int row = static_cast<int>( i / secondHeight );
		const float* dense = second + ( i - static_cast<long long>( row ) * secondHeight ) * firstWidth;
		float sum = 0.f;
		for( int at = rows[row]; at < rows[row + 1]; ++at ) {
			sum += values[at] * dense[columns[at]];
		}
		result[i] = sum;
	}
}

// result[fh x sw] = sparse[fh x fw] * dense[fw x sw]
__global__ __launch_bounds__( 256 )
void sparseByMatrixKernel( const int* rows, const int* columns, const float* values, const float* second, int firstHeight,
	int secondWidth, float* result )
{
	NH_FOR_EACH( i, static_cast<long long>( firstHeight ) * secondWidth ) {
		const int row = static_cast<int>( i / secondWidth );
		const int col = static_cast<int>( i - static_cast<long long>( row ) * secondWidth );
		float sum = 0.f;
		for( int at = rows[row]; at < rows[row + 1]; ++at ) {
			sum += values[at] * second[static_cast<long long>( columns[at] ) * secondWidth + col];
		}
		result[i] = sum;
	}
}

// result[fw x sw] += sparse[fh x fw]^T * dense[fh x sw]: thread per ( sparse row, dense column ), scattered with atomics
__global__ __launch_bounds__( 256 )
void transposedSparseByMatrixKernel( const int* rows, const int* columns, const float* values, const float* second, int firstHeight,
	int secondWidth, float* result )
{
	NH_FOR_EACH( i, static_cast<long long>( firstHeight ) * secondWidth ) {
		const int row = static_cast<int>( i / secondWidth );
		const int col = static_cast<int>( i - static_cast<long long>( row ) * secondWidth );
		const float dense = second[i];
		for( int at = rows[row]; at < rows[row + 1]; ++at ) {
			atomicAdd( result + static_cast<long long>( columns[at] ) * secondWidth + col, values[at] * dense );
		}
	}
}

// result[fw x rw] += dense[fh x fw]^T * sparse[fh x rw]: thread per ( sparse row, dense column )
__global__ __launch_bounds__( 256 )
void transposedBySparseKernel( const float* first, const int* rows, const int* columns, const float* values, int firstHeight,
	int firstWidth, int resultWidth, float* result )
{
	NH_FOR_EACH( i, static_cast<long long>( firstHeight ) * firstWidth ) {
		const int row = static_cast<int>( i / firstWidth );
		const int col = static_cast<int>( i - static_cast<long long>( row ) * firstWidth );
		const float dense = first[i];
		for( int at = rows[row]; at < rows[row + 1]; ++at ) {
			atomicAdd( result + static_cast<long long>( col ) * resultWidth + columns[at], dense * values[at] );
		}
	}
}

// result[fw x rw] = dense[fh x fw]^T * sparse[rw x fh]^T: thread per result element, no atomics
__global__ __launch_bounds__( 256 )
void transposedByTransposedSparseKernel( const float* first, const int* rows, const int* columns, const float* values, int firstWidth,
	int resultWidth, float* result )
{
	NH_FOR_EACH( i, static_cast<long long>( firstWidth ) * resultWidth ) {
		const int col = static_cast<int>( i / resultWidth );
		const int row = static_cast<int>( i - static_cast<long long>( col ) * resultWidth );
		float sum = 0.f;
		for( int at = rows[row]; at < rows[row + 1]; ++at ) {
			sum += first[static_cast<long long>( columns[at] ) * firstWidth + col] * values[at];
		}
		result[i] = sum;
	}
}

__global__ __launch_bounds__( 256 )
void zeroKernel( float* data, long long total )
{
	NH_FOR_EACH( i, total ) {
		data[i] = 0.f;
	}
}

// ---- top-k ( src/CPU/CpuMathEngineVectorMath.cpp:384-450 ) ---------------------------------------------------------
// The k largest values in descending order with their positions; of equal values the one met first comes first.
// One wavefront: k rounds, each a reduction for the largest value not yet taken ( ties to the smaller index ).
__global__ __launch_bounds__( 64 )
void topKKernel( const float* first, int size, int k, float* result, int* indices )
{
	const int lane = threadIdx.x;
	float lastValue = 0.f;
	int lastIndex = -1;
	for( int round = 0; round < k && round < size; ++round ) {
		float best = 0.f;
		int bestIndex = -1;
		for( int i = lane; i < size; i += 64 ) {
			const float v = first[i];
			// not yet taken: smaller than the last one, or equal to it and behind it
			const bool open = round == 0 || v < lastValue || ( v == lastValue && i > lastIndex );
			if( open && ( bestIndex < 0 || v > best ) ) {
				best = v;
				bestIndex = i;
			}
		}
		for( int off = 32; off > 0; off >>= 1 ) {
			const float otherValue = __shfl_xor( best, off, 64 );
			const int otherIndex = __shfl_xor( bestIndex, off, 64 );
			if( otherIndex >= 0 && ( bestIndex < 0 || otherValue > best || ( otherValue == best && otherIndex < bestIndex ) ) ) {
				best = otherValue;
				bestIndex = otherIndex;
			}
		}
		if( bestIndex < 0 ) {
			break; // what is left does not compare ( NaN )
		}
		if( lane == 0 ) {
			result[round] = best;
			indices[round] = bestIndex;
		}
		lastValue = best;
		lastIndex = bestIndex;
	}
}

// the gradient of top-k: row i of the result is row indices[i] of the source ( for a single row: its element indices[i]
// kept in place, zeros elsewhere )
__global__ __launch_bounds__( 256 )
void topKDiffKernel( const float* sourceGrad, int height, int width, const int* indices, int k, float* resultGrad )
{
	NH_FOR_EACH( i, static_cast<long long>( k ) * width ) {
		const int row = static_cast<int>( i / width );
		const int col = static_cast<int>( i - static_cast<long long>( row ) * width );
		if( height == 1 ) {
			resultGrad[i] = col == indices[row] ? sourceGrad[col] : 0.f;
		} else {
			resultGrad[i] = sourceGrad[static_cast<long long>( indices[row] ) * width + col];
		}
	}
}

// ---- 3-D convolution and pooling ( blobs are N x H x W x D x C; src/CPU/CpuMathEngineDnn3dConv.cpp, CpuMathEngineDnnPooling.cpp ) --

struct CVolume {
	int N, H, W, D, C;
	__host__ __device__ long long size() const { return static_cast<long long>( N ) * H * W * D * C; }
};

__device__ __forceinline__ void unpack5( long long i, const CVolume& v, int& n, int& h, int& w, int& d, int& c )
{
	c = static_cast<int>( i % v.C ); i /= v.C;
	d = static_cast<int>( i % v.D ); i /= v.D;
	w = static_cast<int>( i % v.W ); i /= v.W;
	h = static_cast<int>( i % v.H );
	n = static_cast<int>( i / v.H );
}

// filter [Cout][fh][fw][fd][Cin]
__global__ __launch_bounds__( 256 )
void conv3dKernel( const nh3dDesc d, const float* source, const float* filter, const float* freeTerm, float* result )
{
	const CVolume out = { d.batch, d.resultHeight, d.resultWidth, d.resultDepth, d.filterCount };
	NH_FOR_EACH( i, out.size() ) {
		int n, ho, wo, zo, co;
		unpack5( i, out, n, ho, wo, zo, co );
		float sum = freeTerm != nullptr ? freeTerm[co] : 0.f;
		for( int fh = 0; fh < d.filterHeight; ++fh ) {
			const int hi = ho * d.strideHeight - d.paddingHeight + fh;
			if( hi < 0 || hi >= d.height ) {
				continue;
			}
			for( int fw = 0; fw < d.filterWidth; ++fw ) {
				const int wi = wo * d.strideWidth - d.paddingWidth + fw;
				if( wi < 0 || wi >= d.width ) {
					continue;
				}
				for( int fd = 0; fd < d.filterDepth; ++fd ) {
					const int zi = zo * d.strideDepth - d.paddingDepth + fd;
					if( zi < 0 || zi >= d.depth ) {
						continue;
					}
					const float* in = source + ( ( ( static_cast<long long>( n ) * d.height + hi ) * d.width + wi ) * d.depth + zi ) * d.channels;
					const float* f = filter + ( ( ( static_cast<long long>( co ) * d.filterHeight + fh ) * d.filterWidth + fw ) * d.filterDepth + fd ) * d.channels;
					for( int c = 0; c < d.channels; ++c ) {
						sum = fmaf( in[c], f[c], sum );
					}
				}
			}
		}
		result[i] = sum;
	}
}

// gradient by the input: gathers, per input element, the output positions whose windows hold it
__global__ __launch_bounds__( 256 )
void conv3dBackwardKernel( const nh3dDesc d, const float* outputDiff, const float* filter, const float* freeTerm, float* inputDiff )
{
	const CVolume in = { d.batch, d.height, d.width, d.depth, d.channels };
	NH_FOR_EACH( i, in.size() ) {
		int n, hi, wi, zi, c;
		unpack5( i, in, n, hi, wi, zi, c );
		float sum = freeTerm != nullptr ? freeTerm[c] : 0.f;
		for( int fh = 0; fh < d.filterHeight; ++fh ) {
			const int hs = hi + d.paddingHeight - fh;
			if( hs < 0 || hs % d.strideHeight != 0 || hs / d.strideHeight >= d.resultHeight ) {
				continue;
			}
			for( int fw = 0; fw < d.filterWidth; ++fw ) {
				const int ws = wi + d.paddingWidth - fw;
				if( ws < 0 || ws % d.strideWidth != 0 || ws / d.strideWidth >= d.resultWidth ) {
					continue;
				}
				for( int fd = 0; fd < d.filterDepth; ++fd ) {
					const int zs = zi + d.paddingDepth - fd;
					if( zs < 0 || zs % d.strideDepth != 0 || zs / d.strideDepth >= d.resultDepth ) {
						continue;
					}
					const float* o = outputDiff + ( ( ( static_cast<long long>( n ) * d.resultHeight + hs / d.strideHeight ) * d.resultWidth
						+ ws / d.strideWidth ) * d.resultDepth + zs / d.strideDepth ) * d.filterCount;
					const long long tap = ( ( static_cast<long long>( fh ) * d.filterWidth + fw ) * d.filterDepth + fd ) * d.channels + c;
					const long long filterStep = static_cast<long long>( d.filterHeight ) * d.filterWidth * d.filterDepth * d.channels;
					for( int co = 0; co < d.filterCount; ++co ) {
						sum = fmaf( o[co], filter[co * filterStep + tap], sum );
					}
				}
			}
		}
		inputDiff[i] = sum;
	}
}

// gradient by the filter: thread per filter element, sums over every output position
__global__ __launch_bounds__( 256 )
void conv3dLearnKernel( const nh3dDesc d, const float* input, const float* outputDiff, float* filterDiff )
{
	const CVolume flt = { d.filterCount, d.filterHeight, d.filterWidth, d.filterDepth, d.channels };
	NH_FOR_EACH( i, flt.size() ) {
		int co, fh, fw, fd, c;
		unpack5( i, flt, co, fh, fw, fd, c );
		float sum = 0.f;
		for( int n = 0; n < d.batch; ++n ) {
			for( int ho = 0; ho < d.resultHeight; ++ho ) {
				const int hi = ho * d.strideHeight - d.paddingHeight + fh;
				if( hi < 0 || hi >= d.height ) {
					continue;
				}
				for( int wo = 0; wo < d.resultWidth; ++wo ) {
					const int wi = wo * d.strideWidth - d.paddingWidth + fw;
					if( wi < 0 || wi >= d.width ) {
						continue;
					}
					for( int zo = 0; zo < d.resultDepth; ++zo ) {
						const int zi = zo * d.strideDepth - d.paddingDepth + fd;
						if( zi < 0 || zi >= d.depth ) {
							continue;
						}
						sum = fmaf( input[( ( ( static_cast<long long>( n ) * d.height + hi ) * d.width + wi ) * d.depth + zi ) * d.channels + c],
							outputDiff[( ( ( static_cast<long long>( n ) * d.resultHeight + ho ) * d.resultWidth + wo ) * d.resultDepth + zo ) * d.filterCount + co],
							sum );
					}
				}
			}
		}
		filterDiff[i] += sum;
	}
}

// target[c] += sum over rows of matrix[rows x columns]
__global__ __launch_bounds__( 256 )
void addColumnSumsKernel( const float* matrix, long long rows, int columns, float* target )
{
	NH_FOR_EACH( c, columns ) {
		float sum = 0.f;
		for( long long r = 0; r < rows; ++r ) {
			sum += matrix[r * columns + c];
		}
		target[c] += sum;
	}
}

// The index is the offset, inside the source object, of channel 0 of the winning position ( the gradient adds the
// channel ); the window is scanned rows first, then columns, then depth, a later equal value does not replace.
__global__ __launch_bounds__( 256 )
void maxPooling3dKernel( const nh3dDesc d, const float* source, int* indices, float* result )
{
	const CVolume out = { d.batch, d.resultHeight, d.resultWidth, d.resultDepth, d.channels };
	NH_FOR_EACH( i, out.size() ) {
		int n, ho, wo, zo, c;
		unpack5( i, out, n, ho, wo, zo, c );
		const float* object = source + static_cast<long long>( n ) * d.height * d.width * d.depth * d.channels;
		float best = 0.f;
		int bestAt = -1;
		for( int fh = 0; fh < d.filterHeight; ++fh ) {
			for( int fw = 0; fw < d.filterWidth; ++fw ) {
				for( int fd = 0; fd < d.filterDepth; ++fd ) {
					const int at = ( ( ( ho * d.strideHeight + fh ) * d.width + wo * d.strideWidth + fw ) * d.depth + zo * d.strideDepth + fd ) * d.channels;
					const float v = object[at + c];
					if( bestAt < 0 || v > best ) {
						best = v;
						bestAt = at;
					}
				}
			}
		}
		result[i] = best;
		if( indices != nullptr ) {
			indices[i] = bestAt;
		}
	}
}

__global__ __launch_bounds__( 256 )
void maxPooling3dBackwardKernel( const nh3dDesc d, const float* resultDiff, const int* indices, float* sourceDiff )
{
	const CVolume out = { d.batch, d.resultHeight, d.resultWidth, d.resultDepth, d.channels };
	const long long objectSize = static_cast<long long>( d.height ) * d.width * d.depth * d.channels;
	NH_FOR_EACH( i, out.size() ) {
		const long long n = i / ( static_cast<long long>( d.resultHeight ) * d.resultWidth * d.resultDepth * d.channels );
		const int c = static_cast<int>( i % d.channels );
		atomicAdd( sourceDiff + n * objectSize + indices[i] + c, resultDiff[i] );
	}
}

__global__ __launch_bounds__( 256 )
void meanPooling3dKernel( const nh3dDesc d, const float* source, float* result )
{
	const CVolume out = { d.batch, d.resultHeight, d.resultWidth, d.resultDepth, d.channels };
	const float scale = 1.f / ( d.filterHeight * d.filterWidth * d.filterDepth );
	NH_FOR_EACH( i, out.size() ) {
		int n, ho, wo, zo, c;
		unpack5( i, out, n, ho, wo, zo, c );
		const float* object = source + static_cast<long long>( n ) * d.height * d.width * d.depth * d.channels;
		float sum = 0.f;
		for( int fh = 0; fh < d.filterHeight; ++fh ) {
			for( int fw = 0; fw < d.filterWidth; ++fw ) {
				for( int fd = 0; fd < d.filterDepth; ++fd ) {
					sum += object[( ( ( ho * d.strideHeight + fh ) * d.width + wo * d.strideWidth + fw ) * d.depth + zo * d.strideDepth + fd ) * d.channels + c];
				}
			}
		}
		result[i] = sum * scale;
	}
}

// gathers, per source element, the windows that hold it ( elements that no window holds get zero )
__global__ __launch_bounds__( 256 )
void meanPooling3dBackwardKernel( const nh3dDesc d, const float* resultDiff, float* sourceDiff )
{
	const CVolume in = { d.batch, d.height, d.width, d.depth, d.channels };
	const float scale = 1.f / ( d.filterHeight * d.filterWidth * d.filterDepth );
	NH_FOR_EACH( i, in.size() ) {
		int n, hi, wi, zi, c;
		unpack5( i, in, n, hi, wi, zi, c );
		float sum = 0.f;
		for( int fh = 0; fh < d.filterHeight; ++fh ) {
			const int hs = hi - fh;
			if( hs < 0 || hs % d.strideHeight != 0 || hs / d.strideHeight >= d.resultHeight ) {
				continue;
			}
			for( int fw = 0; fw < d.filterWidth; ++fw ) {
				const int ws = wi - fw;
				if( ws < 0 || ws % d.strideWidth != 0 || ws / d.strideWidth >= d.resultWidth ) {
					continue;
				}
				for( int fd = 0; fd < d.filterDepth; ++fd ) {
					const int zs = zi - fd;
					if( zs < 0 || zs % d.strideDepth != 0 || zs / d.strideDepth >= d.resultDepth ) {
						continue;
					}
					sum += resultDiff[( ( ( static_cast<long long>( n ) * d.resultHeight + hs / d.strideHeight ) * d.resultWidth + ws / d.strideWidth )
						* d.resultDepth + zs / d.strideDepth ) * d.channels + c];
				}
			}
		}
		sourceDiff[i] = sum * scale;
	}
}

// ---- run-length encoded images ( include/NeoMathEngine/NeoMathEngine.h:664-686, src/CPU/CpuMathEngineDnnRleConv.cpp ) ----
// An image of height x width pixels sits in a slot of height x width 4-byte words: { strokes, height, width, stub } and
// then, line by line, the strokes { short start, short end ( first pixel behind the stroke ) } of a line, closed by the
// sentinel { SHRT_MAX, -1 }. The decoder writes stroke / non-stroke values; a thread decodes one line group by walking
// the strokes from the image's beginning ( lines are not addressable ), so one thread per image.
__global__ __launch_bounds__( 64 )
void rleDecodeKernel( const int* rle, int batch, int height, int width, float stroke, float nonStroke, float* dense )
{
	const int image = blockIdx.x * 64 + threadIdx.x;
	if( image >= batch ) {
		return;
	}
	const long long slot = static_cast<long long>( height ) * width;
	const int* words = rle + image * slot;
	float* out = dense + image * slot;
	for( long long i = 0; i < slot; ++i ) {
		out[i] = nonStroke;
	}
	long long at = 4;
	for( int line = 0; line < height && at < slot; ++line ) {
		for( ; at < slot; ++at ) {
			const int word = words[at];
			const int start = static_cast<short>( word & 0xffff );
			const int end = static_cast<short>( ( word >> 16 ) & 0xffff );
			if( end < 0 ) {
				++at; // the sentinel that closes the line
				break;
			}
			for( int x = max( start, 0 ); x < min( end, width ); ++x ) {
				out[static_cast<long long>( line ) * width + x] = stroke;
			}
		}
	}
}


// ---- CTC loss ( src/CPU/CpuMathEngineDnnCtc.cpp:202-403 ) ----------------------------------------------------------
// The lattice of a sequence: U = 2 * labelLen + 1 positions ( blank, label 0, blank, label 1, ..., blank ), T frames.
// logAlpha[t][u] / logBeta[t][u] are the reference's forward / backward variables in the log domain, computed by the same
// operations in the same order ( its log-sum-exp of two values, its "log zero" of -FLT_MAX / 4, its padding of frames beyond
// a sequence's length with a certain blank ), so that both engines agree to rounding. One workgroup walks one sequence of
// the batch: the frames one after the other, the positions side by side.

constexpr float CtcLogZero = -FLT_MAX / 4;

__device__ __forceinline__ float ctcExp( float x )
{
	return x < -87.33654474f ? 0.f : ( x > 88.f ? FLT_MAX : expf( x ) );
}

// ( x86/CpuX86MathEngineVectorMathMkl.cpp:155-213 )
__device__ __forceinline__ float ctcLogSumExp( float a, float b )
{
	const float e = ctcExp( -fabsf( a - b ) );
	return fmaxf( a, b ) + logf( fminf( 1.f + fmaxf( e, FLT_MIN ), FLT_MAX ) );
}

struct CCtcShape {
	int T, B, C, L, U, Blank, SkipBlanks;
};

__device__ __forceinline__ int ctcPaddedLabel( const CCtcShape& n, const int* labels, int b, int u )
{
	return ( u & 1 ) != 0 ? labels[( u >> 1 ) * n.B + b] : n.Blank;
}

// log( I{ u < U - 2 } * I{ label[u] != label[u + 2] } ): what a step over a blank adds
__device__ __forceinline__ float ctcSkipMask( const CCtcShape& n, const int* labels, int b, int u )
{
	return ( u < n.U - 2 && ctcPaddedLabel( n, labels, b, u ) != ctcPaddedLabel( n, labels, b, u + 2 ) ) ? 0.f : CtcLogZero;
}

// log-probability of class k in frame t; frames beyond the sequence's length emit a blank for certain
__device__ __forceinline__ float ctcEmission( const CCtcShape& n, const float* logProb, const int* resultLens, int t, int b, int k )
{
	if( resultLens != nullptr && t >= resultLens[b] ) {
		return k == n.Blank ? -FLT_MIN * 2 : CtcLogZero;
	}
	return logProb[( static_cast<long long>( t ) * n.B + b ) * n.C + k];
}

// the reference's column-wise log-sum-exp: maximum, sum of exp( x - maximum ) in ascending order, clamped log
__device__ float ctcLogSumExpOf( const float* values, int count )
{
	float top = values[0];
	for( int i = 1; i < count; ++i ) {
		top = values[i] > top ? values[i] : top;
	}
	float sum = 0.f;
	for( int i = 0; i < count; ++i ) {
		sum += ctcExp( values[i] - top );
	}
	return top + logf( fminf( fmaxf( sum, FLT_MIN ), FLT_MAX ) );
}

__global__ __launch_bounds__( 256 )
void ctcLatticeKernel( const CCtcShape n, const float* logProb, const int* labels, const int* labelLens, const int* resultLens,
	float* logAlpha, float* logBeta, float* total )
{
	extern __shared__ float lattice[]; // [3][U]
	float* previous = lattice;
	float* current = lattice + n.U;
	float* shifted = lattice + 2 * n.U;
	const int b = blockIdx.x;
	const int U = n.U;
	const long long frame = static_cast<long long>( U ) * n.B;

	// forward: a sequence begins with a blank or with its first label
	for( int u = threadIdx.x; u < U; u += 256 ) {
		const float v = ( u < 2 ? 0.f : CtcLogZero ) + ctcEmission( n, logProb, resultLens, 0, b, ctcPaddedLabel( n, labels, b, u ) );
		previous[u] = v;
		logAlpha[static_cast<long long>( u ) * n.B + b] = v;
	}
	__syncthreads();
	for( int t = 1; t < n.T; ++t ) {
		for( int u = threadIdx.x; u < U; u += 256 ) {
			float v = u == 0 ? previous[0] : ctcLogSumExp( previous[u - 1], previous[u] );
			if( n.SkipBlanks && u >= 2 ) {
				v = ctcLogSumExp( v, previous[u - 2] + ctcSkipMask( n, labels, b, u - 2 ) );
			}
			v += ctcEmission( n, logProb, resultLens, t, b, ctcPaddedLabel( n, labels, b, u ) );
			current[u] = v;
			logAlpha[t * frame + static_cast<long long>( u ) * n.B + b] = v;
		}
		__syncthreads();
		float* swap = previous;
		previous = current;
		current = swap;
	}

	// backward: a sequence ends with its last label or with the blank behind it ( with the blank only where frames
	// beyond its length follow: CpuMathEngineDnnCtc.cpp:350-376 )
	__syncthreads();
	{
		int endA = U - 1, endB = U - 2;
		if( labelLens != nullptr ) {
			endA = 2 * labelLens[b];
			endB = endA - 1 + ( ( resultLens != nullptr && resultLens[b] < n.T ) ? 1 : 0 );
		}
		for( int u = threadIdx.x; u < U; u += 256 ) {
			const float v = ( u == endA || u == endB ) ? 0.f : CtcLogZero;
			previous[u] = v;
			logBeta[( n.T - 1 ) * frame + static_cast<long long>( u ) * n.B + b] = v;
		}
	}
	__syncthreads();
	for( int t = n.T - 2; t >= 0; --t ) {
		for( int u = threadIdx.x; u < U; u += 256 ) {
			shifted[u] = previous[u] + ctcEmission( n, logProb, resultLens, t + 1, b, ctcPaddedLabel( n, labels, b, u ) );
		}
		__syncthreads();
		for( int u = threadIdx.x; u < U; u += 256 ) {
			float v = shifted[u];
			if( u < U - 1 ) {
				v = ctcLogSumExp( shifted[u], shifted[u + 1] );
				if( n.SkipBlanks && u < U - 2 ) {
					v = ctcLogSumExp( v, shifted[u + 2] + ctcSkipMask( n, labels, b, u ) );
				}
			}
			current[u] = v;
			logBeta[t * frame + static_cast<long long>( u ) * n.B + b] = v;
		}
		__syncthreads();
		float* swap = previous;
		previous = current;
		current = swap;
	}

	// log-probability of the labelling: over the positions of frame 0
	for( int u = threadIdx.x; u < U; u += 256 ) {
		shifted[u] = logAlpha[static_cast<long long>( u ) * n.B + b] + logBeta[static_cast<long long>( u ) * n.B + b];
	}
	__syncthreads();
	if( threadIdx.x == 0 ) {
		total[b] = ctcLogSumExpOf( shifted, U );
	}
}

// loss = - sum( weight * total ) / batch
__global__ void ctcLossKernel( const float* total, const float* weights, int batch, float* loss )
{
	if( blockIdx.x == 0 && threadIdx.x == 0 ) {
		float sum = 0.f;
		for( int b = 0; b < batch; ++b ) {
			sum += weights != nullptr ? weights[b] * total[b] : total[b];
		}
		*loss = -sum / batch;
	}
}

// gradient by the network's result ( before its softmax ): prob - exp( logsumexp over the positions of class k of
// ( logAlpha + logBeta ) - total ); one workgroup per ( frame, sequence )
__global__ __launch_bounds__( 256 )
void ctcGradientKernel( const CCtcShape n, const float* prob, const int* labels, const int* resultLens, const float* logAlpha,
	const float* logBeta, const float* total, float* gradient )
{
	extern __shared__ float both[]; // [U] + 1
	const int t = blockIdx.x / n.B;
	const int b = blockIdx.x - t * n.B;
	const long long frame = static_cast<long long>( n.U ) * n.B;
	float* out = gradient + ( static_cast<long long>( t ) * n.B + b ) * n.C;
	if( resultLens != nullptr && t >= resultLens[b] ) {
		for( int k = threadIdx.x; k < n.C; k += 256 ) {
			out[k] = 0.f;
		}
		return;
	}
	for( int u = threadIdx.x; u < n.U; u += 256 ) {
		const long long at = t * frame + static_cast<long long>( u ) * n.B + b;
		both[u] = logAlpha[at] + logBeta[at];
	}
	__syncthreads();
	if( threadIdx.x == 0 ) {
		// ( with skipped blanks the reference takes the total of the frame itself, for stability )
		both[n.U] = n.SkipBlanks ? ctcLogSumExpOf( both, n.U ) : total[b];
	}
	__syncthreads();
	const float all = both[n.U];
	const float* p = prob + ( static_cast<long long>( t ) * n.B + b ) * n.C;
	for( int k = threadIdx.x; k < n.C; k += 256 ) {
		float sum = CtcLogZero;
		for( int u = 0; u < n.U; ++u ) {
			if( ctcPaddedLabel( n, labels, b, u ) == k ) {
				const float f = both[u];
				sum = f >= sum ? f + log1pf( expf( sum - f ) ) : sum + log1pf( expf( f - sum ) );
			}
		}
		out[k] = p[k] - ctcExp( sum - all );
	}
}

static bool valid3d( const nh3dDesc* d )
{
	return d != nullptr && d->batch >= 0 && d->height > 0 && d->width > 0 && d->depth > 0 && d->channels > 0
		&& d->filterHeight > 0 && d->filterWidth > 0 && d->filterDepth > 0 && d->strideHeight > 0 && d->strideWidth > 0 && d->strideDepth > 0
		&& d->paddingHeight >= 0 && d->paddingWidth >= 0 && d->paddingDepth >= 0 && d->filterCount >= 0
		&& d->resultHeight > 0 && d->resultWidth > 0 && d->resultDepth > 0
		&& ( d->resultHeight - 1 ) * d->strideHeight - d->paddingHeight + d->filterHeight <= d->height + d->paddingHeight
		&& ( d->resultWidth - 1 ) * d->strideWidth - d->paddingWidth + d->filterWidth <= d->width + d->paddingWidth
		&& ( d->resultDepth - 1 ) * d->strideDepth - d->paddingDepth + d->filterDepth <= d->depth + d->paddingDepth
		&& static_cast<long long>( d->height ) * d->width * d->depth * d->channels < 0x7fffffffLL;
}

} // namespace nh

using namespace nh;

extern "C" {

int nhQrnnFPooling( nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* initialState, float* result )
{
	NH_REQUIRE( sequenceLength >= 1 && objectSize >= 1 && update != nullptr && forget != nullptr && result != nullptr );
	NH_LAUNCH( qrnnPoolingKernel, objectSize, reverse, sequenceLength, objectSize, update, forget, static_cast<const float*>( nullptr ),
		initialState, result );
	return NH_OK;
}

int nhQrnnIfPooling( nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* input, const float* initialState, float* result )
{
	NH_REQUIRE( sequenceLength >= 1 && objectSize >= 1 && update != nullptr && forget != nullptr && input != nullptr && result != nullptr );
	NH_LAUNCH( qrnnPoolingKernel, objectSize, reverse, sequenceLength, objectSize, update, forget, input, initialState, result );
	return NH_OK;
}

int nhQrnnFPoolingBackward( nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* initialState, const float* result, float* resultDiff, float* updateDiff, float* forgetDiff )
{
	NH_REQUIRE( sequenceLength >= 1 && objectSize >= 1 && update != nullptr && forget != nullptr && result != nullptr
		&& resultDiff != nullptr && updateDiff != nullptr && forgetDiff != nullptr );
	NH_LAUNCH( qrnnPoolingBackwardKernel, objectSize, reverse, sequenceLength, objectSize, update, forget, static_cast<const float*>( nullptr ),
		initialState, result, resultDiff, updateDiff, forgetDiff, static_cast<float*>( nullptr ) );
	return NH_OK;
}

int nhQrnnIfPoolingBackward( nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* input, const float* initialState, const float* result, float* resultDiff, float* updateDiff, float* forgetDiff,
	float* inputDiff )
{
	NH_REQUIRE( sequenceLength >= 1 && objectSize >= 1 && update != nullptr && forget != nullptr && input != nullptr && result != nullptr
		&& resultDiff != nullptr && updateDiff != nullptr && forgetDiff != nullptr && inputDiff != nullptr );
	NH_LAUNCH( qrnnPoolingBackwardKernel, objectSize, reverse, sequenceLength, objectSize, update, forget, input, initialState, result,
		resultDiff, updateDiff, forgetDiff, inputDiff );
	return NH_OK;
}

int nhIndRnnRecurrent( nhStream s, int reverse, int sequenceLength, int batchSize, int objectSize, int activation, const float* wx,
	const float* mask, const float* u, float* h )
{
	NH_REQUIRE( sequenceLength >= 1 && batchSize >= 1 && objectSize >= 1 && wx != nullptr && u != nullptr && h != nullptr );
	NH_REQUIRE( activation == NH_INDRNN_SIGMOID || activation == NH_INDRNN_RELU );
	const long long total = static_cast<long long>( batchSize ) * objectSize;
	NH_LAUNCH( indRnnKernel, total, reverse, sequenceLength, batchSize, objectSize, activation == NH_INDRNN_RELU ? 1 : 0, wx, mask, u, h );
	return NH_OK;
}

int nhIndRnnRecurrentBackward( nhStream s, int reverse, int sequenceLength, int batchSize, int objectSize, int activation,
	const float* mask, const float* u, const float* h, const float* hDiff, float* wxDiff )
{
	NH_REQUIRE( sequenceLength >= 1 && batchSize >= 1 && objectSize >= 1 && u != nullptr && h != nullptr && hDiff != nullptr && wxDiff != nullptr );
	NH_REQUIRE( activation == NH_INDRNN_SIGMOID || activation == NH_INDRNN_RELU );
	const long long total = static_cast<long long>( batchSize ) * objectSize;
	NH_LAUNCH( indRnnBackwardKernel, total, reverse, sequenceLength, batchSize, objectSize, activation == NH_INDRNN_RELU ? 1 : 0, mask, u, h,
		hDiff, wxDiff, static_cast<float*>( nullptr ) );
	return NH_OK;
}

int nhIndRnnRecurrentLearn( nhStream s, int reverse, int sequenceLength, int batchSize, int objectSize, int activation,
	const float* mask, const float* u, const float* h, const float* hDiff, float* uDiff )
{
	NH_REQUIRE( sequenceLength >= 1 && batchSize >= 1 && objectSize >= 1 && u != nullptr && h != nullptr && hDiff != nullptr && uDiff != nullptr );
	NH_REQUIRE( activation == NH_INDRNN_SIGMOID || activation == NH_INDRNN_RELU );
	const long long total = static_cast<long long>( batchSize ) * objectSize;
	NH_LAUNCH( indRnnBackwardKernel, total, reverse, sequenceLength, batchSize, objectSize, activation == NH_INDRNN_RELU ? 1 : 0, mask, u, h,
		hDiff, static_cast<float*>( nullptr ), uDiff );
	return NH_OK;
}

int nhBertConv( nhStream s, const float* data, const float* kernel, int seqLen, int batchSize, int numHeads, int headSize, int kernelSize,
	float* output )
{
	NH_REQUIRE( seqLen >= 1 && batchSize >= 1 && numHeads >= 1 && headSize >= 1 && kernelSize >= 1 );
	NH_REQUIRE( data != nullptr && kernel != nullptr && output != nullptr );
	const int lanes = batchSize * numHeads;
	const long long total = static_cast<long long>( seqLen ) * lanes * headSize;
	NH_LAUNCH( bertConvKernel, total, data, kernel, seqLen, lanes, headSize, kernelSize, output );
	return NH_OK;
}

int nhBertConvBackward( nhStream s, const float* data, const float* kernel, const float* outDiff, int seqLen, int batchSize, int numHeads,
	int headSize, int kernelSize, float* dataDiff, float* kernelDiff )
{
	NH_REQUIRE( seqLen >= 1 && batchSize >= 1 && numHeads >= 1 && headSize >= 1 && kernelSize >= 1 );
	NH_REQUIRE( data != nullptr && kernel != nullptr && outDiff != nullptr && dataDiff != nullptr && kernelDiff != nullptr );
	const int lanes = batchSize * numHeads;
	const long long total = static_cast<long long>( seqLen ) * lanes * headSize;
	NH_LAUNCH( bertConvDataDiffKernel, total, kernel, outDiff, seqLen, lanes, headSize, kernelSize, dataDiff );
	const long long taps = static_cast<long long>( seqLen ) * lanes * kernelSize;
	NH_LAUNCH( bertConvKernelDiffKernel, taps, data, outDiff, seqLen, lanes, headSize, kernelSize, kernelDiff );
	return NH_OK;
}

int nhLrn( nhStream s, const float* input, int vectorCount, int vectorSize, int windowSize, float bias, float alpha, float beta,
	float* invSum, float* invSumBeta, float* output )
{
	NH_REQUIRE( vectorCount >= 0 && vectorSize >= 1 && windowSize >= 1 );
	const long long total = static_cast<long long>( vectorCount ) * vectorSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && output != nullptr ) );
	NH_LAUNCH( lrnKernel, total, input, total, vectorSize, windowSize, bias, alpha / windowSize, beta, invSum, invSumBeta, output );
	return NH_OK;
}

int nhLrnBackward( nhStream s, const float* input, const float* output, const float* outputDiff, const float* invSum,
	const float* invSumBeta, int vectorCount, int vectorSize, int windowSize, float alpha, float beta, float* inputDiff )
{
	NH_REQUIRE( vectorCount >= 0 && vectorSize >= 1 && windowSize >= 1 );
	const long long total = static_cast<long long>( vectorCount ) * vectorSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && output != nullptr && outputDiff != nullptr && invSum != nullptr && invSumBeta != nullptr
		&& inputDiff != nullptr ) );
	NH_LAUNCH( lrnBackwardKernel, total, input, output, outputDiff, invSum, invSumBeta, total, vectorSize, windowSize,
		-2.f * alpha * beta / windowSize, inputDiff );
	return NH_OK;
}

int nhMultiplySparseMatrixByTransposedMatrix( nhStream s, int firstHeight, int firstWidth, int secondHeight, const int* rows,
	const int* columns, const float* values, const float* second, float* result )
{
	NH_REQUIRE( firstHeight >= 0 && firstWidth >= 0 && secondHeight >= 0 );
	const long long total = static_cast<long long>( firstHeight ) * secondHeight;
	NH_REQUIRE( total == 0 || ( rows != nullptr && second != nullptr && result != nullptr ) );
	NH_LAUNCH( sparseByTransposedKernel, total, rows, columns, values, second, firstHeight, firstWidth, secondHeight, result );
	return NH_OK;
}

int nhMultiplySparseMatrixByMatrix( nhStream s, int firstHeight, int firstWidth, int secondWidth, const int* rows, const int* columns,
	const float* values, const float* second, float* result )
{
	NH_REQUIRE( firstHeight >= 0 && firstWidth >= 0 && secondWidth >= 0 );
	const long long total = static_cast<long long>( firstHeight ) * secondWidth;
	NH_REQUIRE( total == 0 || ( rows != nullptr && second != nullptr && result != nullptr ) );
	NH_LAUNCH( sparseByMatrixKernel, total, rows, columns, values, second, firstHeight, secondWidth, result );
	return NH_OK;
}

int nhMultiplyTransposedSparseMatrixByMatrix( nhStream s, int firstHeight, int firstWidth, int secondWidth, const int* rows,
	const int* columns, const float* values, const float* second, float* result )
{
	NH_REQUIRE( firstHeight >= 0 && firstWidth >= 0 && secondWidth >= 0 );
	const long long resultSize = static_cast<long long>( firstWidth ) * secondWidth;
	NH_REQUIRE( resultSize == 0 || result != nullptr );
	NH_LAUNCH( zeroKernel, resultSize, result, resultSize );
	const long long total = static_cast<long long>( firstHeight ) * secondWidth;
	NH_REQUIRE( total == 0 || ( rows != nullptr && second != nullptr ) );
	NH_LAUNCH( transposedSparseByMatrixKernel, total, rows, columns, values, second, firstHeight, secondWidth, result );
	return NH_OK;
}

int nhMultiplyTransposedMatrixBySparseMatrix( nhStream s, int firstHeight, int firstWidth, int resultWidth, const float* first,
	const int* rows, const int* columns, const float* values, float* result, int isTransposedSparse, int add )
{
	NH_REQUIRE( firstHeight >= 0 && firstWidth >= 0 && resultWidth >= 0 && !( isTransposedSparse && add ) );
	const long long resultSize = static_cast<long long>( firstWidth ) * resultWidth;
	NH_REQUIRE( resultSize == 0 || ( result != nullptr && first != nullptr && rows != nullptr ) );
	if( isTransposedSparse ) {
		NH_LAUNCH( transposedByTransposedSparseKernel, resultSize, first, rows, columns, values, firstWidth, resultWidth, result );
		return NH_OK;
	}
	if( !add ) {
		NH_LAUNCH( zeroKernel, resultSize, result, resultSize );
	}
	const long long total = static_cast<long long>( firstHeight ) * firstWidth;
	NH_LAUNCH( transposedBySparseKernel, total, first, rows, columns, values, firstHeight, firstWidth, resultWidth, result );
	return NH_OK;
}

int nhVectorTopK( nhStream s, const float* first, int firstSize, int k, float* result, int* indices )
{
	NH_REQUIRE( firstSize >= 0 && k >= 0 );
	if( firstSize == 0 || k == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( first != nullptr && result != nullptr && indices != nullptr );
	hipLaunchKernelGGL( topKKernel, dim3( 1 ), dim3( 64 ), 0, toStream( s ), first, firstSize, k, result, indices );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhVectorTopKDiff( nhStream s, const float* sourceGrad, int sourceGradHeight, int sourceGradWidth, const int* indices, int k,
	float* resultGrad )
{
	NH_REQUIRE( sourceGradHeight >= 1 && sourceGradWidth >= 1 && k >= 0 );
	const long long total = static_cast<long long>( k ) * sourceGradWidth;
	NH_REQUIRE( total == 0 || ( sourceGrad != nullptr && indices != nullptr && resultGrad != nullptr ) );
	NH_LAUNCH( topKDiffKernel, total, sourceGrad, sourceGradHeight, sourceGradWidth, indices, k, resultGrad );
	return NH_OK;
}

int nhBlob3dConvolution( nhStream s, const nh3dDesc* d, const float* source, const float* filter, const float* freeTerm, float* result )
{
	NH_REQUIRE( valid3d( d ) && d->filterCount > 0 && source != nullptr && filter != nullptr && result != nullptr );
	const long long total = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->resultDepth * d->filterCount;
	NH_LAUNCH( conv3dKernel, total, *d, source, filter, freeTerm, result );
	return NH_OK;
}

int nhBlob3dConvolutionBackward( nhStream s, const nh3dDesc* d, const float* outputDiff, const float* filter, const float* freeTerm,
	float* inputDiff )
{
	NH_REQUIRE( valid3d( d ) && d->filterCount > 0 && outputDiff != nullptr && filter != nullptr && inputDiff != nullptr );
	const long long total = static_cast<long long>( d->batch ) * d->height * d->width * d->depth * d->channels;
	NH_LAUNCH( conv3dBackwardKernel, total, *d, outputDiff, filter, freeTerm, inputDiff );
	return NH_OK;
}

int nhBlob3dConvolutionLearnAdd( nhStream s, const nh3dDesc* d, const float* input, const float* outputDiff, float* filterDiff,
	float* freeTermDiff, int freeTermDiffFromInput )
{
	NH_REQUIRE( valid3d( d ) && d->filterCount > 0 && input != nullptr && outputDiff != nullptr && filterDiff != nullptr );
	const long long total = static_cast<long long>( d->filterCount ) * d->filterHeight * d->filterWidth * d->filterDepth * d->channels;
	NH_LAUNCH( conv3dLearnKernel, total, *d, input, outputDiff, filterDiff );
	if( freeTermDiff != nullptr ) {
		// ( the reference's 1 x 1 x 1 path without padding always sums the output gradient: CpuMathEngineDnn3dConv.cpp:212-214, 644-646 )
		const bool pointwise = d->paddingHeight == 0 && d->paddingWidth == 0 && d->paddingDepth == 0
			&& d->filterHeight == 1 && d->filterWidth == 1 && d->filterDepth == 1;
		if( freeTermDiffFromInput && !pointwise ) {
			NH_LAUNCH( addColumnSumsKernel, d->channels, input, static_cast<long long>( d->batch ) * d->height * d->width * d->depth, d->channels,
				freeTermDiff );
		} else {
			NH_LAUNCH( addColumnSumsKernel, d->filterCount, outputDiff,
				static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->resultDepth, d->filterCount, freeTermDiff );
		}
	}
	return NH_OK;
}

int nhBlob3dMaxPooling( nhStream s, const nh3dDesc* d, const float* source, int* maxIndices, float* result )
{
	NH_REQUIRE( valid3d( d ) && d->paddingHeight == 0 && d->paddingWidth == 0 && d->paddingDepth == 0 && source != nullptr && result != nullptr );
	const long long total = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->resultDepth * d->channels;
	NH_LAUNCH( maxPooling3dKernel, total, *d, source, maxIndices, result );
	return NH_OK;
}

int nhBlob3dMaxPoolingBackward( nhStream s, const nh3dDesc* d, const float* resultDiff, const int* maxIndices, float* sourceDiff )
{
	NH_REQUIRE( valid3d( d ) && resultDiff != nullptr && maxIndices != nullptr && sourceDiff != nullptr );
	const long long sourceSize = static_cast<long long>( d->batch ) * d->height * d->width * d->depth * d->channels;
	NH_LAUNCH( zeroKernel, sourceSize, sourceDiff, sourceSize );
	const long long total = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->resultDepth * d->channels;
	NH_LAUNCH( maxPooling3dBackwardKernel, total, *d, resultDiff, maxIndices, sourceDiff );
	return NH_OK;
}

int nhBlob3dMeanPooling( nhStream s, const nh3dDesc* d, const float* source, float* result )
{
	NH_REQUIRE( valid3d( d ) && d->paddingHeight == 0 && d->paddingWidth == 0 && d->paddingDepth == 0 && source != nullptr && result != nullptr );
	const long long total = static_cast<long long>( d->batch ) * d->resultHeight * d->resultWidth * d->resultDepth * d->channels;
	NH_LAUNCH( meanPooling3dKernel, total, *d, source, result );
	return NH_OK;
}

int nhBlob3dMeanPoolingBackward( nhStream s, const nh3dDesc* d, const float* resultDiff, float* sourceDiff )
{
	NH_REQUIRE( valid3d( d ) && resultDiff != nullptr && sourceDiff != nullptr );
	const long long total = static_cast<long long>( d->batch ) * d->height * d->width * d->depth * d->channels;
	NH_LAUNCH( meanPooling3dBackwardKernel, total, *d, resultDiff, sourceDiff );
	return NH_OK;
}

int nhRleImagesToDense( nhStream s, const void* rle, int batch, int height, int width, float strokeValue, float nonStrokeValue,
	float* dense )
{
	NH_REQUIRE( batch >= 0 && height >= 1 && width >= 1 && static_cast<long long>( height ) * width >= 5 );
	if( batch == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( rle != nullptr && dense != nullptr );
	hipLaunchKernelGGL( rleDecodeKernel, dim3( ( batch + 63 ) / 64 ), dim3( 64 ), 0, toStream( s ), static_cast<const int*>( rle ), batch,
		height, width, strokeValue, nonStrokeValue, dense );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

int nhCtcLossWorkspaceSize( int resultLen, int batchSize, int classCount, int labelLen, size_t* bytes )
{
	NH_REQUIRE( bytes != nullptr && resultLen >= 1 && batchSize >= 1 && classCount >= 1 && labelLen >= 1 );
	const size_t frames = static_cast<size_t>( resultLen ) * batchSize;
	const size_t padded = 2 * static_cast<size_t>( labelLen ) + 1;
	*bytes = ( 2 * frames * classCount + 2 * frames * padded + batchSize ) * sizeof( float );
	return NH_OK;
}

int nhCtcLossForward( nhStream s, int resultLen, int batchSize, int classCount, int labelLen, int blankLabel, int skipBlanks,
	const float* result, const int* labels, const int* labelLens, const int* resultLens, const float* labelWeights, float* loss,
	float* lossGradient, void* workspace, size_t workspaceBytes )
{
	size_t needed = 0;
	const int rc = nhCtcLossWorkspaceSize( resultLen, batchSize, classCount, labelLen, &needed );
	if( rc != NH_OK ) {
		return rc;
	}
	NH_REQUIRE( result != nullptr && loss != nullptr && labels != nullptr );
	NH_REQUIRE( blankLabel >= 0 && blankLabel < classCount );
	NH_REQUIRE( workspace != nullptr && workspaceBytes >= needed );
	const long long frames = static_cast<long long>( resultLen ) * batchSize;
	NH_REQUIRE( frames * classCount <= 0x7fffffffLL );
	CCtcShape n = { resultLen, batchSize, classCount, labelLen, 2 * labelLen + 1, blankLabel, skipBlanks ? 1 : 0 };
	NH_REQUIRE( 3 * static_cast<size_t>( n.U ) * sizeof( float ) <= 60 * 1024 );
	float* prob = static_cast<float*>( workspace );
	float* logProb = prob + frames * classCount;
	float* logAlpha = logProb + frames * classCount;
	float* logBeta = logAlpha + frames * n.U;
	float* total = logBeta + frames * n.U;
	int step = nhMatrixSoftmaxByRows( s, result, static_cast<int>( frames ), classCount, prob );
	if( step != NH_OK ) {
		return step;
	}
	step = nhVectorLog( s, prob, logProb, static_cast<int>( frames * classCount ) );
	if( step != NH_OK ) {
		return step;
	}
	hipLaunchKernelGGL( ctcLatticeKernel, dim3( batchSize ), dim3( 256 ), 3 * n.U * sizeof( float ), toStream( s ), n, logProb, labels,
		labelLens, resultLens, logAlpha, logBeta, total );
	NH_LAUNCH_CHECK();
	hipLaunchKernelGGL( ctcLossKernel, dim3( 1 ), dim3( 64 ), 0, toStream( s ), total, labelWeights, batchSize, loss );
	NH_LAUNCH_CHECK();
	if( lossGradient != nullptr ) {
		hipLaunchKernelGGL( ctcGradientKernel, dim3( static_cast<unsigned>( frames ) ), dim3( 256 ), ( n.U + 1 ) * sizeof( float ), toStream( s ), n,
			prob, labels, resultLens, logAlpha, logBeta, total, lossGradient );
		NH_LAUNCH_CHECK();
	}
	return NH_OK;
}

} // extern "C"
