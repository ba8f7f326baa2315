// Interface members beyond the benchmark networks' path: indexed additions, row scatters, lookups (embeddings),
// binarizations, column-wise softmax, index planes, sub-sequences, up-sampling, space <-> depth.
// None of these is performance-critical in the networks that call them (they move little data next to the
// contractions around them), so every kernel here is the plain form: one thread per result element, grid-stride,
// coalesced along the innermost dimension. Semantics are the reference CPU engine's, cited per kernel.
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

// ---- matrices --------------------------------------------------------------------------------------------------

// src/CPU/CpuMathEngineBlas.cpp:290-304
__global__ __launch_bounds__( 256 )
void addVectorToColumnsIntKernel( const int* matrix, int* result, long long total, int width, const int* vector )
{
	NH_FOR_EACH( i, total ) {
		result[i] = matrix[i] + vector[i / width];
	}
}

// :381-397
__global__ __launch_bounds__( 256 )
void sumMatrixRowsIntKernel( const int* matrix, int* result, int batch, int height, int width )
{
	NH_FOR_EACH( i, static_cast<long long>( batch ) * width ) {
		const long long b = i / width;
		const int* column = matrix + b * height * width + ( i - b * width );
		int sum = 0;
		for( int j = 0; j < height; ++j ) {
			sum += column[static_cast<long long>( j ) * width];
		}
		result[i] = sum;
	}
}

// :633-653
__global__ __launch_bounds__( 256 )
void addDiagToMatrixKernel( const float* diag, const float* matrix, float* result, long long total, int width )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / width;
		result[i] = ( i - row * width ) == row ? matrix[i] + diag[row] : matrix[i];
	}
}

// :339-357
__global__ __launch_bounds__( 256 )
void columnsDivideKernel( const float* matrix, const float* vector, float* result, long long total, int width )
{
	NH_FOR_EACH( i, total ) {
		result[i] = matrix[i] / vector[i / width];
	}
}

// :825-842: every matrix of the batch is multiplied by the same diagonal
__global__ __launch_bounds__( 256 )
void multiply1DiagKernel( const float* diag, const float* second, float* result, long long total, int firstSize, int width )
{
	NH_FOR_EACH( i, total ) {
		result[i] = second[i] * diag[( i / width ) % firstSize];
	}
}

// :1181-1205 (maximum, exp( x - maximum ), sum, reciprocal of the sum with the reference's VectorInv, product)
__global__ __launch_bounds__( 256 )
void softmaxByColumnsKernel( const float* matrix, float* result, int height, int width )
{
	NH_FOR_EACH( column, width ) {
		const float* in = matrix + column;
		float* out = result + column;
		float top = in[0];
		for( int j = 1; j < height; ++j ) {
			const float v = in[static_cast<long long>( j ) * width];
			top = v > top ? v : top;
		}
		float sum = 0.f;
		for( int j = 0; j < height; ++j ) {
			float x = in[static_cast<long long>( j ) * width] - top;
			x = x < -87.33654474f ? 0.f : ( x > 88.f ? FLT_MAX : expf( x ) );
			out[static_cast<long long>( j ) * width] = x;
			sum += x;
		}
		const float inv = 1.f / sum;
		for( int j = 0; j < height; ++j ) {
			out[static_cast<long long>( j ) * width] *= inv;
		}
	}
}

// :1207-1225: dE/dx = y * ( dE/dy - <dE/dy, y> ), the product taken per column
__global__ __launch_bounds__( 256 )
void softmaxDiffOpByColumnsKernel( const float* first, const float* second, float* result, int height, int width )
{
	NH_FOR_EACH( column, width ) {
		float dot = 0.f;
		for( int j = 0; j < height; ++j ) {
			const long long at = static_cast<long long>( j ) * width + column;
			dot += first[at] * second[at];
		}
		for( int j = 0; j < height; ++j ) {
			const long long at = static_cast<long long>( j ) * width + column;
			result[at] = first[at] * ( second[at] - dot );
		}
	}
}

// src/CPU/x86/CpuX86MathEngineBlas.cpp:261-420: the first of equal minima keeps its row
__global__ __launch_bounds__( 256 )
void findMinInColumnsKernel( const float* matrix, int height, int width, float* result, int* rowIndices )
{
	NH_FOR_EACH( column, width ) {
		float best = matrix[column];
		int bestRow = 0;
		for( int j = 1; j < height; ++j ) {
			const float v = matrix[static_cast<long long>( j ) * width + column];
			if( v < best ) {
				best = v;
				bestRow = j;
			}
		}
		result[column] = best;
		rowIndices[column] = bestRow;
	}
}

// src/CPU/x86/CpuX86MathEngineBlas.cpp:33-47: one wavefront per row
__global__ __launch_bounds__( 256 )
void rowsToVectorDistanceKernel( const float* matrix, int height, int width, const float* vector, float* result )
{
	const int lane = threadIdx.x & 63;
	for( long long row = blockIdx.x * 4LL + ( threadIdx.x >> 6 ); row < height; row += static_cast<long long>( gridDim.x ) * 4 ) {
		const float* in = matrix + row * width;
		float sum = 0.f;
		for( int j = lane; j < width; j += 64 ) {
			const float d = in[j] - vector[j];
			sum += d * d;
		}
		sum = waveReduceSum( sum );
		if( lane == 0 ) {
			result[row] = sum;
		}
	}
}

// src/CPU/CpuMathEngineBlas.cpp:983-1023: rows of 32-bit values to the rows their indices name ( negative: nowhere )
__global__ __launch_bounds__( 256 )
void spreadRowsKernel( const int* source, long long total, int width, int* result, const int* indices )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / width;
		const int to = indices[row];
		if( to >= 0 ) {
			result[static_cast<long long>( to ) * width + ( i - row * width )] = source[i];
		}
	}
}

// :1025-1041 ( several rows may name the same target: atomic additions )
__global__ __launch_bounds__( 256 )
void spreadRowsAddKernel( const float* source, long long total, int width, float* result, const int* indices )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / width;
		const int to = indices[row];
		if( to >= 0 ) {
			atomicAdd( result + static_cast<long long>( to ) * width + ( i - row * width ), source[i] );
		}
	}
}

// the four indexed additions, :613-727. MODE 0: result[j] += matrix[j][indices[j]]; 1: result[j][indices[j]] +=
// matrix[j][indices[j]]; 2: result[i] += matrix[rows[i]][columns[i]]; 3: matrix[j][indices[j]] += vector[j];
// 4: matrix[rows[i]][columns[i]] += vector[i] ( pairs may repeat: atomic )
template<int MODE>
__global__ __launch_bounds__( 256 )
void indexedAddKernel( const float* from, float* to, int count, int width, const int* first, const int* second )
{
	NH_FOR_EACH( i, count ) {
		if( MODE == 0 || MODE == 1 || MODE == 3 ) {
			const int index = first[i];
			if( index >= 0 && index < width ) {
				const long long at = i * width + index;
				if( MODE == 0 ) {
					to[i] += from[at];
				} else if( MODE == 1 ) {
					to[at] += from[at];
				} else {
					to[at] += from[i];
				}
			}
		} else {
			const long long at = static_cast<long long>( first[i] ) * width + second[i];
			if( MODE == 2 ) {
				to[i] += from[at];
			} else {
				atomicAdd( to + at, from[i] );
			}
		}
	}
}

// src/CPU/CpuMathEngineDnn.cpp:316-330
__global__ __launch_bounds__( 256 )
void integerHistKernel( const int* numbers, int count, int* result, int maxNumber )
{
	NH_FOR_EACH( i, count ) {
		const int n = numbers[i];
		if( n >= 0 && n < maxNumber ) {
			atomicAdd( result + n, 1 );
		}
	}
}

// src/CPU/CpuMathEngineBlas.cpp:573-611: one-hot rows; INPUT_FLOAT: the class arrives as a float
template<bool INPUT_FLOAT>
__global__ __launch_bounds__( 256 )
void enumBinarizationKernel( const void* input, long long total, int enumSize, float* result )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / enumSize;
		const int value = INPUT_FLOAT ? static_cast<int>( static_cast<const float*>( input )[row] ) : static_cast<const int*>( input )[row];
		result[i] = ( i - row * enumSize ) == value ? 1.f : 0.f;
	}
}

// :1227-1262: bit k of the set becomes element k
__global__ __launch_bounds__( 256 )
void bitSetBinarizationKernel( const int* input, long long total, int bitSetSize, int outputVectorSize, float* result )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / outputVectorSize;
		const int bit = static_cast<int>( i - row * outputVectorSize );
		const unsigned word = static_cast<unsigned>( input[row * bitSetSize + bit / 32] );
		result[i] = ( ( word >> ( bit & 31 ) ) & 1u ) != 0 ? 1.f : 0.f;
	}
}

// ---- lookups ( embeddings ) -------------------------------------------------------------------------------------

// One table of VectorMultichannelLookupAndCopy ( :432-512 ): channel `channel` of every input row is an index into
// `table`; the vector it names goes to columns [ outputOffset, outputOffset + vectorSize ) of the output row.
template<bool INPUT_FLOAT>
__global__ __launch_bounds__( 256 )
void lookupAndCopyKernel( const void* input, int channelCount, int channel, const int* table, int vectorCount, int vectorSize,
	int* output, int outputChannels, int outputOffset, long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / vectorSize;
		const int k = static_cast<int>( i - row * vectorSize );
		const long long at = row * channelCount + channel;
		const int index = INPUT_FLOAT ? static_cast<int>( static_cast<const float*>( input )[at] ) : static_cast<const int*>( input )[at];
		if( index >= 0 && index < vectorCount ) {
			output[row * outputChannels + outputOffset + k] = table[static_cast<long long>( index ) * vectorSize + k];
		}
	}
}

// the channels behind the last table are copied as they are
__global__ __launch_bounds__( 256 )
void copyColumnsKernel( const int* input, int inputWidth, int inputOffset, int* output, int outputWidth, int outputOffset, int count,
	long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long row = i / count;
		const int k = static_cast<int>( i - row * count );
		output[row * outputWidth + outputOffset + k] = input[row * inputWidth + inputOffset + k];
	}
}

// One table of VectorMultichannelLookupAndAddToTable ( :514-571 ): table[index] += mult * matrix row piece
template<bool INPUT_FLOAT>
__global__ __launch_bounds__( 256 )
void lookupAndAddToTableKernel( const void* input, int channelCount, int channel, float* table, int vectorCount, int vectorSize,
	const float* mult, const float* matrix, int matrixWidth, int matrixOffset, long long total )
{
	const float m = *mult;
	NH_FOR_EACH( i, total ) {
		const long long row = i / vectorSize;
		const int k = static_cast<int>( i - row * vectorSize );
		const long long at = row * channelCount + channel;
		const int index = INPUT_FLOAT ? static_cast<int>( static_cast<const float*>( input )[at] ) : static_cast<const int*>( input )[at];
		if( index >= 0 && index < vectorCount ) {
			atomicAdd( table + static_cast<long long>( index ) * vectorSize + k, m * matrix[row * matrixWidth + matrixOffset + k] );
		}
	}
}

// :729-756: the sum of the table rows that a row of indices names ( negative: none ), added in index order
__global__ __launch_bounds__( 256 )
void lookupAndSumKernel( const int* indices, int indexCount, const float* table, int vectorSize, float* result, long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long b = i / vectorSize;
		const int k = static_cast<int>( i - b * vectorSize );
		float sum = 0.f;
		for( int e = 0; e < indexCount; ++e ) {
			const int index = indices[b * indexCount + e];
			if( index >= 0 ) {
				const float v = table[static_cast<long long>( index ) * vectorSize + k];
				sum = e == 0 ? v : sum + v;
			}
		}
		result[i] = sum;
	}
}

// :758-779: table ( cleared by the caller ) [index] += additions[b] for every index of row b
__global__ __launch_bounds__( 256 )
void lookupAndAddKernel( const int* indices, int indexCount, const float* additions, int vectorSize, float* table, long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long pair = i / vectorSize; // ( b, e )
		const int k = static_cast<int>( i - pair * vectorSize );
		const int index = indices[pair];
		if( index >= 0 ) {
			atomicAdd( table + static_cast<long long>( index ) * vectorSize + k, additions[( pair / indexCount ) * vectorSize + k] );
		}
	}
}

// src/CPU/x86/CpuX86MathEngineBlas.cpp:459-560: result[b][j] = < table row rows[b][j], vector table row vectors[b] >;
// one wavefront per result element
__global__ __launch_bounds__( 256 )
void lookupMatrixByLookupVectorKernel( const float* matrixTable, const int* rows, int rowCount, int width,
	const float* vectorTable, const int* vectors, float* result, long long total )
{
	const int lane = threadIdx.x & 63;
	for( long long i = blockIdx.x * 4LL + ( threadIdx.x >> 6 ); i < total; i += static_cast<long long>( gridDim.x ) * 4 ) {
		const long long b = i / rowCount;
		const float* row = matrixTable + static_cast<long long>( rows[i] ) * width;
		const float* vec = vectorTable + static_cast<long long>( vectors[b] ) * width;
		float sum = 0.f;
		for( int k = lane; k < width; k += 64 ) {
			sum += row[k] * vec[k];
		}
		sum = waveReduceSum( sum );
		if( lane == 0 ) {
			result[i] = sum;
		}
	}
}

// src/CPU/CpuMathEngineBlas.cpp:1043-1081: result[b] (+)= sum over j of table row rows[b][j] * vector[b][j]
__global__ __launch_bounds__( 256 )
void transposedLookupMatrixByVectorKernel( const float* table, const int* rows, int rowCount, int width, const float* vector,
	float* result, int add, long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long b = i / width;
		const int k = static_cast<int>( i - b * width );
		float sum = add ? result[i] : 0.f;
		for( int j = 0; j < rowCount; ++j ) {
			const float term = table[static_cast<long long>( rows[b * rowCount + j] ) * width + k] * vector[b * rowCount + j];
			sum = ( j == 0 && !add ) ? term : sum + term;
		}
		result[i] = sum;
	}
}

// :1083-1101: table row index[b][j] += first[b][j] * second's vector of b
__global__ __launch_bounds__( 256 )
void vectorByTransposedLookupVectorKernel( float* table, int vectorSize, const int* index, const float* first, int firstSize,
	const float* secondTable, const int* secondVector, long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long pair = i / vectorSize; // ( b, j )
		const int k = static_cast<int>( i - pair * vectorSize );
		const long long b = pair / firstSize;
		atomicAdd( table + static_cast<long long>( index[pair] ) * vectorSize + k,
			first[pair] * secondTable[static_cast<long long>( secondVector[b] ) * vectorSize + k] );
	}
}

// ---- blobs ------------------------------------------------------------------------------------------------------

// src/CPU/CpuMathEngineDnnPooling.cpp:606-646: result = source + ( forward ? index : -index ) of the pixel's column
// ( or row ): the blob is [outer][indexed][inner]
template<typename T>
__global__ __launch_bounds__( 256 )
void addDimIndexKernel( const T* source, T* result, long long total, int indexedSize, int innerSize, int forward )
{
	NH_FOR_EACH( i, total ) {
		const int index = static_cast<int>( ( i / innerSize ) % indexedSize );
		result[i] = source[i] + static_cast<T>( forward ? index : -index );
	}
}

// src/CPU/CpuMathEngineDnn.cpp:174-204: `length` consecutive positions of every sequence, forwards or backwards from
// startPos; the indices of the source objects go to `indices` when asked for
__global__ __launch_bounds__( 256 )
void getSubSequenceKernel( const float* from, float* to, int* indices, int batchWidth, int objectSize, int startPos, int reverse, long long total )
{
	NH_FOR_EACH( i, total ) {
		const long long object = i / objectSize; // pos * batchWidth + seq
		const long long pos = object / batchWidth;
		const long long source = ( reverse ? startPos - pos : startPos + pos ) * batchWidth + ( object - pos * batchWidth );
		const int k = static_cast<int>( i - object * objectSize );
		to[i] = from[source * objectSize + k];
		if( indices != nullptr && k == 0 ) {
			indices[object] = static_cast<int>( source );
		}
	}
}

// :213-286: every pixel repeated heightCopyCount x widthCopyCount times ( 32-bit values )
__global__ __launch_bounds__( 256 )
void upsamplingForwardKernel( const int* input, int* result, int height, int width, int pixelSize, int heightCopy, int widthCopy, long long total )
{
	const int resultWidth = width * widthCopy;
	const int resultHeight = height * heightCopy;
	NH_FOR_EACH( i, total ) {
		const int k = static_cast<int>( i % pixelSize );
		long long rest = i / pixelSize;
		const int x = static_cast<int>( rest % resultWidth );
		rest /= resultWidth;
		const int y = static_cast<int>( rest % resultHeight );
		const long long object = rest / resultHeight;
		result[i] = input[( ( object * height + y / heightCopy ) * width + x / widthCopy ) * pixelSize + k];
	}
}

// :288-300: the gradient of a pixel is the sum over its copies; rows first, then columns, as the reference sums them
__global__ __launch_bounds__( 256 )
void upsamplingBackwardKernel( const float* input, float* result, int height, int width, int pixelSize, int heightCopy, int widthCopy, long long total )
{
	const int inputWidth = width * widthCopy;
	NH_FOR_EACH( i, total ) {
		const int k = static_cast<int>( i % pixelSize );
		long long rest = i / pixelSize;
		const int x = static_cast<int>( rest % width );
		rest /= width;
		const int y = static_cast<int>( rest % height );
		const long long object = rest / height;
		float sum = 0.f;
		for( int w = 0; w < widthCopy; ++w ) {
			float columnSum = 0.f;
			for( int h = 0; h < heightCopy; ++h ) {
				columnSum += input[( ( object * height * heightCopy + y * heightCopy + h ) * inputWidth + x * widthCopy + w ) * pixelSize + k];
			}
			sum += columnSum;
		}
		result[i] = sum;
	}
}

// :820-930: blocks of blockSize x blockSize pixels <-> channels ( 32-bit values ). In the "depth" layout a data row
// holds, per block, blockSize rows of blockSize * channels values one after another; in the "space" layout the same
// rows lie dataRowWidth blocks apart.
__global__ __launch_bounds__( 256 )
void spaceToDepthKernel( const int* source, int* result, int dataRowWidth, int blockChannels, int blockSize, int forward, long long total )
{
	const int blockRowSize = blockChannels * blockSize;
	const long long dataRowSize = static_cast<long long>( blockSize ) * dataRowWidth * blockRowSize;
	NH_FOR_EACH( i, total ) {
		// i in the depth layout: [dataRow][block][blockRow][k]
		const long long dataRow = i / dataRowSize;
		long long rest = i - dataRow * dataRowSize;
		const int block = static_cast<int>( rest / ( static_cast<long long>( blockSize ) * blockRowSize ) );
		rest -= static_cast<long long>( block ) * blockSize * blockRowSize;
		const int blockRow = static_cast<int>( rest / blockRowSize );
		const int k = static_cast<int>( rest - static_cast<long long>( blockRow ) * blockRowSize );
		const long long space = dataRow * dataRowSize + ( static_cast<long long>( blockRow ) * dataRowWidth + block ) * blockRowSize + k;
		if( forward ) {
			result[i] = source[space];
		} else {
			result[space] = source[i];
		}
	}
}

// :332-400: the YOLO "reorg" with the reference's legacy index arithmetic ( channels-first indices repacked to
// channels-last ); the loop nest of ReorgFunc, one thread per iteration
__device__ __forceinline__ long long legacyRepackIndex( long long fromIndex, int channels, int height, int width )
{
	const int x = static_cast<int>( fromIndex % width );
	fromIndex /= width;
	const int y = static_cast<int>( fromIndex % height );
	fromIndex /= height;
	const int c = static_cast<int>( fromIndex % channels );
	const long long b = fromIndex / channels;
	return c + static_cast<long long>( channels ) * ( x + static_cast<long long>( width ) * ( y + height * b ) );
}

__global__ __launch_bounds__( 256 )
void reorgKernel( const int* source, int* result, int stride, int forward, int channels, int height, int width, long long total )
{
	const int outputChannels = channels / ( stride * stride );
	NH_FOR_EACH( i, total ) {
		const int w = static_cast<int>( i % width );
		long long rest = i / width;
		const int h = static_cast<int>( rest % height );
		rest /= height;
		const int channel = static_cast<int>( rest % channels );
		const long long batch = rest / channels;
		long long inputIndex = w + static_cast<long long>( width ) * ( h + static_cast<long long>( height ) * ( channel + channels * batch ) );
		inputIndex = legacyRepackIndex( inputIndex, channels * stride * stride, height / stride, width / stride );
		const int outputChannelId = channel % outputChannels;
		const int offset = channel / outputChannels;
		const int outputW = w * stride + offset % stride;
		const int outputH = h * stride + offset / stride;
		long long outputIndex = outputW + static_cast<long long>( width ) * stride * ( outputH + static_cast<long long>( height ) * stride *
			( outputChannelId + outputChannels * batch ) );
		outputIndex = legacyRepackIndex( outputIndex, channels, height, width );
		if( forward ) {
			result[inputIndex] = source[outputIndex];
		} else {
			result[outputIndex] = source[inputIndex];
		}
	}
}

// ---- poolings over a whole object or over time ------------------------------------------------------------------

// src/CPU/x86/CpuX86MathEngineDnn.cpp:33-140: per ( object, channel ) the maxCount largest of the poolSize values in
// descending order with their pixel indices; a value that equals a kept one goes in front of it ( the comparison is
// >= ), slots that stay empty hold -FLT_MAX / -1. One thread per ( object, channel ) keeps its list in the result
// itself, as the reference does; a value below the smallest kept one is dropped without walking the list.
__global__ __launch_bounds__( 256 )
void globalMaxPoolingKernel( const float* source, int* maxIndices, float* result, long long columns, int poolSize, int channels, int maxCount )
{
	NH_FOR_EACH( column, columns ) {
		const long long b = column / channels;
		const int c = static_cast<int>( column - b * channels );
		const float* in = source + b * poolSize * channels + c;
		float* values = result + b * maxCount * channels + c;
		int* indices = maxIndices + b * maxCount * channels + c;
		for( int k = 0; k < maxCount; ++k ) {
			values[static_cast<long long>( k ) * channels] = -FLT_MAX;
			indices[static_cast<long long>( k ) * channels] = -1;
		}
		float smallest = -FLT_MAX;
		for( int i = 0; i < poolSize; ++i ) {
			float next = in[static_cast<long long>( i ) * channels];
			if( !( next >= smallest ) ) {
				continue;
			}
			int nextIndex = i;
			for( int k = 0; k < maxCount; ++k ) {
				const long long at = static_cast<long long>( k ) * channels;
				const float current = values[at];
				if( next >= current ) {
					const int currentIndex = indices[at];
					values[at] = next;
					indices[at] = nextIndex;
					next = current;
					nextIndex = currentIndex;
				}
			}
			smallest = values[static_cast<long long>( maxCount - 1 ) * channels];
		}
	}
}

// src/CPU/CpuMathEngineDnnPooling.cpp:318-350 ( the gradient blob is cleared by the caller )
__global__ __launch_bounds__( 256 )
void globalMaxPoolingBackwardKernel( const float* resultDiff, const int* maxIndices, float* sourceDiff, long long total, int poolSize,
	int channels, int maxCount )
{
	NH_FOR_EACH( i, total ) {
		const int index = maxIndices[i];
		if( index >= 0 && index < poolSize ) {
			const long long b = i / ( static_cast<long long>( maxCount ) * channels );
			const int c = static_cast<int>( i % channels );
			sourceDiff[( b * poolSize + index ) * channels + c] = resultDiff[i];
		}
	}
}

// src/CPU/x86/CpuX86MathEngineDnn.cpp:336-440: windows of filterLen steps, strideLen apart, over the sequence axis; the
// first of equal maxima keeps its step
__global__ __launch_bounds__( 256 )
void maxOverTimePoolingKernel( const float* source, int* maxIndices, float* result, long long total, int seqElemSize, int filterLen,
	int strideLen )
{
	NH_FOR_EACH( i, total ) {
		const long long l = i / seqElemSize;
		const int e = static_cast<int>( i - l * seqElemSize );
		const long long first = l * strideLen;
		float best = source[first * seqElemSize + e];
		int bestStep = static_cast<int>( first );
		for( int n = 1; n < filterLen; ++n ) {
			const float v = source[( first + n ) * seqElemSize + e];
			if( v > best ) {
				best = v;
				bestStep = static_cast<int>( first + n );
			}
		}
		result[i] = best;
		if( maxIndices != nullptr ) {
			maxIndices[i] = bestStep;
		}
	}
}

// src/CPU/CpuMathEngineDnnPooling.cpp:480-500 ( windows overlap: atomic additions into the cleared gradient ); with
// assign != 0 the plain store of the global form, :300-316
__global__ __launch_bounds__( 256 )
void overTimePoolingBackwardKernel( const float* resultDiff, const int* maxIndices, float* sourceDiff, long long total, int seqElemSize,
	int assign )
{
	NH_FOR_EACH( i, total ) {
		const int e = static_cast<int>( i % seqElemSize );
		float* to = sourceDiff + static_cast<long long>( maxIndices[i] ) * seqElemSize + e;
		if( assign ) {
			*to = resultDiff[i];
		} else {
			atomicAdd( to, resultDiff[i] );
		}
	}
}

// src/CPU/CpuMathEngineDnn.cpp:1016-1110: linear interpolation along the middle axis of [objectCount][scaledAxis][objectSize]
// coords 0 half pixel, 1 PyTorch half pixel, 2 align corners, 3 asymmetric; round 0 none, 1 half down, 2 half up, 3 floor, 4 ceil
__global__ __launch_bounds__( 256 )
void linearInterpolationKernel( const float* data, float* result, long long total, int scaledAxis, int newAxis, int objectSize, float scale,
	int coords, int round )
{
	NH_FOR_EACH( i, total ) {
		const int k = static_cast<int>( i % objectSize );
		const long long rest = i / objectSize;
		const int at = static_cast<int>( rest % newAxis );
		const long long b = rest / newAxis;
		float old;
		if( coords == 3 ) {
			old = at / scale;
		} else if( coords == 0 ) {
			old = ( at + 0.5f ) / scale - 0.5f;
		} else if( coords == 1 ) {
			old = newAxis > 1 ? ( at + 0.5f ) / scale - 0.5f : 0.f;
		} else {
			old = static_cast<float>( at * ( scaledAxis - 1 ) ) / ( newAxis - 1 );
		}
		if( round == 1 ) {
			old = old == static_cast<int>( old ) + 0.5f ? floorf( old ) : roundf( old );
		} else if( round == 2 ) {
			old = roundf( old );
		} else if( round == 3 ) {
			old = floorf( old );
		} else if( round == 4 ) {
			old = ceilf( old );
		}
		const float* in = data + b * scaledAxis * objectSize + k;
		float value;
		if( old <= 0.f ) {
			value = in[0];
		} else if( old >= static_cast<float>( scaledAxis - 1 ) ) {
			value = in[static_cast<long long>( scaledAxis - 1 ) * objectSize];
		} else {
			const float left = floorf( old );
			const float rightMul = old - left;
			const float leftMul = 1.f - rightMul;
			const long long cell = static_cast<long long>( static_cast<int>( old ) ) * objectSize;
			// two products, one sum, as the reference's multiply / multiply / add ( no fused multiply-add )
			{
#pragma clang fp contract( off )
				const float right = in[cell + objectSize] * rightMul;
				const float leftPart = in[cell] * leftMul;
				value = right + leftPart;
			}
		}
		result[i] = value;
	}
}

// :1112-1140: objects of 32-bit values to the places their index tuples name ( the strides of the indexed dimensions
// arrive precomputed; a repeated target keeps an unspecified one of its updates )
struct CScatterStrides {
	int Count;
	long long Stride[8];
};

__global__ __launch_bounds__( 256 )
void scatterNDKernel( const int* updates, const int* indices, int* data, long long total, int objectSize, CScatterStrides strides )
{
	NH_FOR_EACH( i, total ) {
		const long long update = i / objectSize;
		long long flat = 0;
		for( int d = 0; d < strides.Count; ++d ) {
			flat += strides.Stride[d] * indices[update * strides.Count + d];
		}
		data[flat + ( i - update * objectSize )] = updates[i];
	}
}

} // namespace nh

using namespace nh;

#define NH_LAUNCH( kernel, total, ... ) \
	do { \
		if( ( total ) > 0 ) { \
			hipLaunchKernelGGL( kernel, dim3( gridFor( total ) ), dim3( 256 ), 0, toStream( s ), __VA_ARGS__ ); \
			NH_LAUNCH_CHECK(); \
		} \
	} while( 0 )

extern "C" int nhAddVectorToMatrixColumnsInt( nhStream s, const int* matrix, int* result, int matrixHeight, int matrixWidth, const int* vector )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth >= 0 );
	const long long total = static_cast<long long>( matrixHeight ) * matrixWidth;
	NH_REQUIRE( total == 0 || ( matrix != nullptr && result != nullptr && vector != nullptr ) );
	NH_LAUNCH( addVectorToColumnsIntKernel, total, matrix, result, total, matrixWidth, vector );
	return NH_OK;
}

extern "C" int nhSumMatrixRowsInt( nhStream s, int batchSize, int* result, const int* matrix, int matrixHeight, int matrixWidth )
{
	NH_REQUIRE( batchSize >= 0 && matrixHeight >= 0 && matrixWidth >= 0 );
	const long long total = static_cast<long long>( batchSize ) * matrixWidth;
	NH_REQUIRE( total == 0 || ( result != nullptr && ( matrix != nullptr || matrixHeight == 0 ) ) );
	NH_LAUNCH( sumMatrixRowsIntKernel, total, matrix, result, batchSize, matrixHeight, matrixWidth );
	return NH_OK;
}

extern "C" int nhAddDiagMatrixToMatrix( nhStream s, const float* diagMatrix, const float* matrix, int height, int width, float* result )
{
	NH_REQUIRE( height >= 0 && width >= 0 );
	const long long total = static_cast<long long>( height ) * width;
	NH_REQUIRE( total == 0 || ( diagMatrix != nullptr && matrix != nullptr && result != nullptr ) );
	NH_LAUNCH( addDiagToMatrixKernel, total, diagMatrix, matrix, result, total, width );
	return NH_OK;
}

extern "C" int nhMatrixColumnsEltwiseDivide( nhStream s, const float* matrix, int matrixHeight, int matrixWidth, const float* vector, float* result )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth >= 0 );
	const long long total = static_cast<long long>( matrixHeight ) * matrixWidth;
	NH_REQUIRE( total == 0 || ( matrix != nullptr && vector != nullptr && result != nullptr ) );
	NH_LAUNCH( columnsDivideKernel, total, matrix, vector, result, total, matrixWidth );
	return NH_OK;
}

extern "C" int nhMultiply1DiagMatrixByMatrix( nhStream s, int batchSize, const float* first, int firstSize, const float* second, int secondWidth,
	float* result )
{
	NH_REQUIRE( batchSize >= 0 && firstSize >= 0 && secondWidth >= 0 );
	const long long total = static_cast<long long>( batchSize ) * firstSize * secondWidth;
	NH_REQUIRE( total == 0 || ( first != nullptr && second != nullptr && result != nullptr ) );
	NH_LAUNCH( multiply1DiagKernel, total, first, second, result, total, firstSize, secondWidth );
	return NH_OK;
}

extern "C" int nhMatrixSoftmaxByColumns( nhStream s, const float* matrix, int height, int width, float* result )
{
	NH_REQUIRE( height > 0 && width > 0 && matrix != nullptr && result != nullptr );
	NH_LAUNCH( softmaxByColumnsKernel, static_cast<long long>( width ), matrix, result, height, width );
	return NH_OK;
}

extern "C" int nhMatrixSoftmaxDiffOpByColumns( nhStream s, const float* first, const float* second, int height, int width, float* result )
{
	NH_REQUIRE( height > 0 && width > 0 && first != nullptr && second != nullptr && result != nullptr );
	NH_LAUNCH( softmaxDiffOpByColumnsKernel, static_cast<long long>( width ), first, second, result, height, width );
	return NH_OK;
}

extern "C" int nhFindMinValueInColumns( nhStream s, const float* matrix, int matrixHeight, int matrixWidth, float* result, int* rowIndices )
{
	NH_REQUIRE( matrixHeight > 0 && matrixWidth > 0 && matrix != nullptr && result != nullptr && rowIndices != nullptr );
	NH_LAUNCH( findMinInColumnsKernel, static_cast<long long>( matrixWidth ), matrix, matrixHeight, matrixWidth, result, rowIndices );
	return NH_OK;
}

extern "C" int nhMatrixRowsToVectorSquaredL2Distance( nhStream s, const float* matrix, int matrixHeight, int matrixWidth, const float* vector,
	float* result )
{
	NH_REQUIRE( matrixHeight >= 0 && matrixWidth > 0 );
	if( matrixHeight == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( matrix != nullptr && vector != nullptr && result != nullptr );
	const int blocks = ceilDiv( matrixHeight, 4 );
	hipLaunchKernelGGL( rowsToVectorDistanceKernel, dim3( blocks > 16384 ? 16384 : blocks ), dim3( 256 ), 0, toStream( s ), matrix, matrixHeight,
		matrixWidth, vector, result );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

extern "C" int nhVectorFillInt( nhStream s, int* result, int value, int vectorSize );
extern "C" int nhVectorFillFromHandleInt( nhStream s, int* result, int vectorSize, const int* value );

extern "C" int nhMatrixSpreadRows( nhStream s, const void* source, int height, int width, void* result, int resultHeight, const int* indices,
	const void* fillValue )
{
	NH_REQUIRE( height >= 0 && width >= 0 && resultHeight >= 0 );
	const long long resultTotal = static_cast<long long>( resultHeight ) * width;
	NH_REQUIRE( resultTotal <= 0x7fffffff );
	if( resultTotal > 0 ) {
		NH_REQUIRE( result != nullptr );
		const int rc = fillValue != nullptr ? nhVectorFillFromHandleInt( s, static_cast<int*>( result ), static_cast<int>( resultTotal ), static_cast<const int*>( fillValue ) )
			: nhVectorFillInt( s, static_cast<int*>( result ), 0, static_cast<int>( resultTotal ) );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	const long long total = static_cast<long long>( height ) * width;
	NH_REQUIRE( total == 0 || ( source != nullptr && indices != nullptr ) );
	NH_LAUNCH( spreadRowsKernel, total, static_cast<const int*>( source ), total, width, static_cast<int*>( result ), indices );
	return NH_OK;
}

extern "C" int nhMatrixSpreadRowsAdd( nhStream s, const float* source, int height, int width, float* result, const int* indices )
{
	NH_REQUIRE( height >= 0 && width >= 0 );
	const long long total = static_cast<long long>( height ) * width;
	NH_REQUIRE( total == 0 || ( source != nullptr && result != nullptr && indices != nullptr ) );
	NH_LAUNCH( spreadRowsAddKernel, total, source, total, width, result, indices );
	return NH_OK;
}

extern "C" int nhIndexedAdd( nhStream s, int mode, const float* from, float* to, int count, int width, const int* first, const int* second )
{
	NH_REQUIRE( count >= 0 && width >= 0 && mode >= 0 && mode <= 4 );
	if( count == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( from != nullptr && to != nullptr && first != nullptr && ( ( mode != 2 && mode != 4 ) || second != nullptr ) );
	const long long total = count;
	switch( mode ) {
		case 0: NH_LAUNCH( indexedAddKernel<0>, total, from, to, count, width, first, second ); break;
		case 1: NH_LAUNCH( indexedAddKernel<1>, total, from, to, count, width, first, second ); break;
		case 2: NH_LAUNCH( indexedAddKernel<2>, total, from, to, count, width, first, second ); break;
		case 3: NH_LAUNCH( indexedAddKernel<3>, total, from, to, count, width, first, second ); break;
		default: NH_LAUNCH( indexedAddKernel<4>, total, from, to, count, width, first, second ); break;
	}
	return NH_OK;
}

extern "C" int nhBuildIntegerHist( nhStream s, const int* numbers, int numbersCount, int* result, int maxNumber )
{
	NH_REQUIRE( numbersCount >= 0 && maxNumber >= 0 );
	if( maxNumber > 0 ) {
		NH_REQUIRE( result != nullptr );
		const int rc = nhVectorFillInt( s, result, 0, maxNumber );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	NH_REQUIRE( numbersCount == 0 || numbers != nullptr );
	NH_LAUNCH( integerHistKernel, static_cast<long long>( numbersCount ), numbers, numbersCount, result, maxNumber );
	return NH_OK;
}

extern "C" int nhEnumBinarization( nhStream s, int batchSize, const void* input, int inputIsFloat, int enumSize, float* result )
{
	NH_REQUIRE( batchSize >= 0 && enumSize >= 0 );
	const long long total = static_cast<long long>( batchSize ) * enumSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && result != nullptr ) );
	if( inputIsFloat ) {
		NH_LAUNCH( enumBinarizationKernel<true>, total, input, total, enumSize, result );
	} else {
		NH_LAUNCH( enumBinarizationKernel<false>, total, input, total, enumSize, result );
	}
	return NH_OK;
}

extern "C" int nhBitSetBinarization( nhStream s, int batchSize, int bitSetSize, const int* input, int outputVectorSize, float* result )
{
	NH_REQUIRE( batchSize >= 0 && bitSetSize >= 0 && outputVectorSize >= 0 && outputVectorSize <= bitSetSize * 32 );
	const long long total = static_cast<long long>( batchSize ) * outputVectorSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && result != nullptr ) );
	NH_LAUNCH( bitSetBinarizationKernel, total, input, total, bitSetSize, outputVectorSize, result );
	return NH_OK;
}

extern "C" int nhLookupAndCopy( nhStream s, int batchSize, int channelCount, const void* input, int inputIsFloat, int channel, const void* table,
	int vectorCount, int vectorSize, void* output, int outputChannels, int outputOffset )
{
	NH_REQUIRE( batchSize >= 0 && channel >= 0 && channel < channelCount && vectorCount >= 0 && vectorSize >= 0
		&& outputOffset >= 0 && outputOffset + vectorSize <= outputChannels );
	const long long total = static_cast<long long>( batchSize ) * vectorSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && table != nullptr && output != nullptr ) );
	if( inputIsFloat ) {
		NH_LAUNCH( lookupAndCopyKernel<true>, total, input, channelCount, channel, static_cast<const int*>( table ), vectorCount, vectorSize,
			static_cast<int*>( output ), outputChannels, outputOffset, total );
	} else {
		NH_LAUNCH( lookupAndCopyKernel<false>, total, input, channelCount, channel, static_cast<const int*>( table ), vectorCount, vectorSize,
			static_cast<int*>( output ), outputChannels, outputOffset, total );
	}
	return NH_OK;
}

extern "C" int nhCopyColumns( nhStream s, int rows, const void* input, int inputWidth, int inputOffset, void* output, int outputWidth, int outputOffset,
	int count )
{
	NH_REQUIRE( rows >= 0 && count >= 0 && inputOffset >= 0 && outputOffset >= 0 && inputOffset + count <= inputWidth
		&& outputOffset + count <= outputWidth );
	const long long total = static_cast<long long>( rows ) * count;
	NH_REQUIRE( total == 0 || ( input != nullptr && output != nullptr ) );
	NH_LAUNCH( copyColumnsKernel, total, static_cast<const int*>( input ), inputWidth, inputOffset, static_cast<int*>( output ), outputWidth,
		outputOffset, count, total );
	return NH_OK;
}

extern "C" int nhLookupAndAddToTable( nhStream s, int batchSize, int channelCount, const void* input, int inputIsFloat, int channel, float* table,
	int vectorCount, int vectorSize, const float* mult, const float* matrix, int matrixWidth, int matrixOffset )
{
	NH_REQUIRE( batchSize >= 0 && channel >= 0 && channel < channelCount && vectorCount >= 0 && vectorSize >= 0
		&& matrixOffset >= 0 && matrixOffset + vectorSize <= matrixWidth );
	const long long total = static_cast<long long>( batchSize ) * vectorSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && table != nullptr && mult != nullptr && matrix != nullptr ) );
	if( inputIsFloat ) {
		NH_LAUNCH( lookupAndAddToTableKernel<true>, total, input, channelCount, channel, table, vectorCount, vectorSize, mult, matrix, matrixWidth,
			matrixOffset, total );
	} else {
		NH_LAUNCH( lookupAndAddToTableKernel<false>, total, input, channelCount, channel, table, vectorCount, vectorSize, mult, matrix, matrixWidth,
			matrixOffset, total );
	}
	return NH_OK;
}

extern "C" int nhLookupAndSum( nhStream s, const int* indices, int batchSize, int indexCount, const float* table, int vectorSize, float* result )
{
	NH_REQUIRE( batchSize >= 0 && indexCount > 0 && vectorSize >= 0 );
	const long long total = static_cast<long long>( batchSize ) * vectorSize;
	NH_REQUIRE( total == 0 || ( indices != nullptr && table != nullptr && result != nullptr ) );
	NH_LAUNCH( lookupAndSumKernel, total, indices, indexCount, table, vectorSize, result, total );
	return NH_OK;
}

extern "C" int nhVectorFill( nhStream s, float* result, float value, int vectorSize );

extern "C" int nhLookupAndAddToWholeTable( nhStream s, const int* indices, int batchSize, int indexCount, const float* additions, int vectorSize,
	float* table, int vectorCount )
{
	NH_REQUIRE( batchSize >= 0 && indexCount >= 0 && vectorSize >= 0 && vectorCount >= 0
		&& static_cast<long long>( vectorCount ) * vectorSize <= 0x7fffffff );
	if( vectorCount * vectorSize > 0 ) {
		NH_REQUIRE( table != nullptr );
		const int rc = nhVectorFill( s, table, 0.f, vectorCount * vectorSize );
		if( rc != NH_OK ) {
			return rc;
		}
	}
	const long long total = static_cast<long long>( batchSize ) * indexCount * vectorSize;
	NH_REQUIRE( total == 0 || ( indices != nullptr && additions != nullptr ) );
	NH_LAUNCH( lookupAndAddKernel, total, indices, indexCount, additions, vectorSize, table, total );
	return NH_OK;
}

extern "C" int nhMultiplyLookupMatrixByLookupVector( nhStream s, int batchSize, const float* matrixTable, const int* rows, int rowCount, int width,
	const float* vectorTable, const int* vectors, float* result )
{
	NH_REQUIRE( batchSize >= 0 && rowCount >= 0 && width > 0 );
	const long long total = static_cast<long long>( batchSize ) * rowCount;
	if( total == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( matrixTable != nullptr && rows != nullptr && vectorTable != nullptr && vectors != nullptr && result != nullptr );
	const long long blocks = ( total + 3 ) / 4;
	hipLaunchKernelGGL( lookupMatrixByLookupVectorKernel, dim3( static_cast<unsigned>( blocks > 16384 ? 16384 : blocks ) ), dim3( 256 ), 0, toStream( s ),
		matrixTable, rows, rowCount, width, vectorTable, vectors, result, total );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

extern "C" int nhMultiplyTransposedLookupMatrixByVector( nhStream s, int batchSize, const float* table, const int* rows, int rowCount, int width,
	const float* vector, float* result, int add )
{
	NH_REQUIRE( batchSize >= 0 && rowCount > 0 && width >= 0 );
	const long long total = static_cast<long long>( batchSize ) * width;
	NH_REQUIRE( total == 0 || ( table != nullptr && rows != nullptr && vector != nullptr && result != nullptr ) );
	NH_LAUNCH( transposedLookupMatrixByVectorKernel, total, table, rows, rowCount, width, vector, result, add, total );
	return NH_OK;
}

extern "C" int nhMultiplyVectorByTransposedLookupVectorAndAddToTable( nhStream s, int batchSize, float* table, int vectorSize, const int* index,
	const float* first, int firstSize, const float* secondTable, const int* secondVector )
{
	NH_REQUIRE( batchSize >= 0 && vectorSize >= 0 && firstSize >= 0 );
	const long long total = static_cast<long long>( batchSize ) * firstSize * vectorSize;
	NH_REQUIRE( total == 0 || ( table != nullptr && index != nullptr && first != nullptr && secondTable != nullptr && secondVector != nullptr ) );
	NH_LAUNCH( vectorByTransposedLookupVectorKernel, total, table, vectorSize, index, first, firstSize, secondTable, secondVector, total );
	return NH_OK;
}

extern "C" int nhAddDimIndex( nhStream s, const void* source, void* result, int isFloat, int outerSize, int indexedSize, int innerSize, int forward )
{
	NH_REQUIRE( outerSize >= 0 && indexedSize >= 0 && innerSize >= 0 );
	const long long total = static_cast<long long>( outerSize ) * indexedSize * innerSize;
	NH_REQUIRE( total == 0 || ( source != nullptr && result != nullptr ) );
	if( isFloat ) {
		NH_LAUNCH( addDimIndexKernel<float>, total, static_cast<const float*>( source ), static_cast<float*>( result ), total, indexedSize, innerSize, forward );
	} else {
		NH_LAUNCH( addDimIndexKernel<int>, total, static_cast<const int*>( source ), static_cast<int*>( result ), total, indexedSize, innerSize, forward );
	}
	return NH_OK;
}

extern "C" int nhBlobGetSubSequence( nhStream s, const float* from, int fromLength, int batchWidth, int objectSize, int* indices, float* to,
	int toLength, int startPos, int isRev )
{
	NH_REQUIRE( fromLength >= 0 && batchWidth >= 0 && objectSize >= 0 && toLength >= 0 );
	if( toLength > 0 ) {
		const int last = isRev ? startPos - ( toLength - 1 ) : startPos + ( toLength - 1 );
		NH_REQUIRE( startPos >= 0 && startPos < fromLength && last >= 0 && last < fromLength );
	}
	const long long total = static_cast<long long>( toLength ) * batchWidth * objectSize;
	NH_REQUIRE( total == 0 || ( from != nullptr && to != nullptr ) );
	NH_LAUNCH( getSubSequenceKernel, total, from, to, indices, batchWidth, objectSize, startPos, isRev, total );
	return NH_OK;
}

extern "C" int nhUpsampling2DForward( nhStream s, int objectCount, int height, int width, int pixelSize, const void* input, int heightCopyCount,
	int widthCopyCount, void* result )
{
	NH_REQUIRE( objectCount >= 0 && height >= 0 && width >= 0 && pixelSize >= 0 && heightCopyCount > 0 && widthCopyCount > 0 );
	const long long total = static_cast<long long>( objectCount ) * height * heightCopyCount * width * widthCopyCount * pixelSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && result != nullptr ) );
	NH_LAUNCH( upsamplingForwardKernel, total, static_cast<const int*>( input ), static_cast<int*>( result ), height, width, pixelSize, heightCopyCount,
		widthCopyCount, total );
	return NH_OK;
}

extern "C" int nhUpsampling2DBackward( nhStream s, int objectCount, int height, int width, int pixelSize, const float* input, int heightCopyCount,
	int widthCopyCount, float* result )
{
	NH_REQUIRE( objectCount >= 0 && height >= 0 && width >= 0 && pixelSize >= 0 && heightCopyCount > 0 && widthCopyCount > 0 );
	const long long total = static_cast<long long>( objectCount ) * height * width * pixelSize;
	NH_REQUIRE( total == 0 || ( input != nullptr && result != nullptr ) );
	NH_LAUNCH( upsamplingBackwardKernel, total, input, result, height, width, pixelSize, heightCopyCount, widthCopyCount, total );
	return NH_OK;
}

extern "C" int nhSpaceToDepth( nhStream s, const void* source, int dataRowCount, int dataRowWidth, int blockChannels, int blockSize, int isForward,
	void* result )
{
	NH_REQUIRE( dataRowCount >= 0 && dataRowWidth >= 0 && blockChannels >= 0 && blockSize > 0 );
	const long long total = static_cast<long long>( dataRowCount ) * blockSize * dataRowWidth * blockSize * blockChannels;
	NH_REQUIRE( total == 0 || ( source != nullptr && result != nullptr ) );
	NH_LAUNCH( spaceToDepthKernel, total, static_cast<const int*>( source ), static_cast<int*>( result ), dataRowWidth, blockChannels, blockSize, isForward, total );
	return NH_OK;
}

extern "C" int nhReorg( nhStream s, const void* source, int stride, int isForward, int batchSize, int channels, int height, int width, void* result )
{
	NH_REQUIRE( batchSize >= 0 && channels >= 0 && height >= 0 && width >= 0 && stride > 0 && channels % ( stride * stride ) == 0
		&& channels >= stride * stride );
	const long long total = static_cast<long long>( batchSize ) * channels * height * width;
	NH_REQUIRE( total == 0 || ( source != nullptr && result != nullptr ) );
	NH_LAUNCH( reorgKernel, total, static_cast<const int*>( source ), static_cast<int*>( result ), stride, isForward, channels, height, width, total );
	return NH_OK;
}

extern "C" int nhBlobGlobalMaxPooling( nhStream s, int objectCount, int poolSize, int channels, int maxCount, const float* source, int* maxIndices,
	float* result )
{
	NH_REQUIRE( objectCount >= 0 && poolSize > 0 && channels > 0 && maxCount > 0 );
	const long long columns = static_cast<long long>( objectCount ) * channels;
	NH_REQUIRE( columns == 0 || ( source != nullptr && maxIndices != nullptr && result != nullptr ) );
	NH_LAUNCH( globalMaxPoolingKernel, columns, source, maxIndices, result, columns, poolSize, channels, maxCount );
	return NH_OK;
}

extern "C" int nhBlobGlobalMaxPoolingBackward( nhStream s, int objectCount, int poolSize, int channels, int maxCount, const float* resultDiff,
	const int* maxIndices, float* sourceDiff )
{
	NH_REQUIRE( objectCount >= 0 && poolSize > 0 && channels > 0 && maxCount > 0 );
	const long long sourceTotal = static_cast<long long>( objectCount ) * poolSize * channels;
	NH_REQUIRE( sourceTotal <= 0x7fffffff );
	if( sourceTotal == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( resultDiff != nullptr && maxIndices != nullptr && sourceDiff != nullptr );
	const int rc = nhVectorFill( s, sourceDiff, 0.f, static_cast<int>( sourceTotal ) );
	if( rc != NH_OK ) {
		return rc;
	}
	const long long total = static_cast<long long>( objectCount ) * maxCount * channels;
	NH_LAUNCH( globalMaxPoolingBackwardKernel, total, resultDiff, maxIndices, sourceDiff, total, poolSize, channels, maxCount );
	return NH_OK;
}

extern "C" int nhBlobMaxOverTimePooling( nhStream s, int sourceLength, int seqElemSize, int filterLen, int strideLen, const float* source,
	int* maxIndices, float* result )
{
	NH_REQUIRE( sourceLength > 0 && seqElemSize >= 0 && filterLen > 0 && strideLen > 0 && filterLen <= sourceLength );
	const int resultLength = ( sourceLength - filterLen ) / strideLen + 1;
	const long long total = static_cast<long long>( resultLength ) * seqElemSize;
	NH_REQUIRE( total == 0 || ( source != nullptr && result != nullptr ) );
	NH_LAUNCH( maxOverTimePoolingKernel, total, source, maxIndices, result, total, seqElemSize, filterLen, strideLen );
	return NH_OK;
}

extern "C" int nhBlobOverTimePoolingBackward( nhStream s, int sourceLength, int resultLength, int seqElemSize, const float* resultDiff,
	const int* maxIndices, float* sourceDiff, int global )
{
	NH_REQUIRE( sourceLength > 0 && resultLength > 0 && seqElemSize >= 0 );
	const long long sourceTotal = static_cast<long long>( sourceLength ) * seqElemSize;
	NH_REQUIRE( sourceTotal <= 0x7fffffff );
	if( sourceTotal == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( resultDiff != nullptr && maxIndices != nullptr && sourceDiff != nullptr );
	const int rc = nhVectorFill( s, sourceDiff, 0.f, static_cast<int>( sourceTotal ) );
	if( rc != NH_OK ) {
		return rc;
	}
	const long long total = static_cast<long long>( resultLength ) * seqElemSize;
	NH_LAUNCH( overTimePoolingBackwardKernel, total, resultDiff, maxIndices, sourceDiff, total, seqElemSize, global );
	return NH_OK;
}

extern "C" int nhLinearInterpolation( nhStream s, const float* data, float* result, int coords, int round, int objectCount, int scaledAxis,
	int objectSize, float scale )
{
	NH_REQUIRE( coords >= 0 && coords <= 3 && round >= 0 && round <= 4 && objectCount >= 0 && scaledAxis > 0 && objectSize >= 0 && scale > 0.f );
	const int newAxis = static_cast<int>( scaledAxis * scale );
	const long long total = static_cast<long long>( objectCount ) * newAxis * objectSize;
	NH_REQUIRE( total == 0 || ( data != nullptr && result != nullptr ) );
	NH_LAUNCH( linearInterpolationKernel, total, data, result, total, scaledAxis, newAxis, objectSize, scale, coords, round );
	return NH_OK;
}

extern "C" int nhScatterND( nhStream s, const int* indices, const void* updates, void* data, const nhBlobDesc* dataDesc, int updateCount,
	int indexDims )
{
	NH_REQUIRE( dataDesc != nullptr && updateCount >= 0 && indexDims >= 1 && indexDims <= 7 );
	long long objectSize = 1;
	for( int i = indexDims; i < 7; ++i ) {
		objectSize *= dataDesc->dims[i];
	}
	CScatterStrides strides = {};
	strides.Count = indexDims;
	strides.Stride[indexDims - 1] = objectSize;
	for( int i = indexDims - 2; i >= 0; --i ) {
		strides.Stride[i] = strides.Stride[i + 1] * dataDesc->dims[i + 1];
	}
	NH_REQUIRE( objectSize <= 0x7fffffff );
	const long long total = static_cast<long long>( updateCount ) * objectSize;
	NH_REQUIRE( total == 0 || ( indices != nullptr && updates != nullptr && data != nullptr ) );
	NH_LAUNCH( scatterNDKernel, total, static_cast<const int*>( updates ), indices, static_cast<int*>( data ), total, static_cast<int>( objectSize ),
		strides );
	return NH_OK;
}
