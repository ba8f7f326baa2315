/* neoml_hip.h — C ABI of the MI355X (gfx950) math-engine kernels.
 *
 * Every entry point below replaces one method of NeoML's IMathEngine interface
 * (NeoMathEngine/include/NeoMathEngine/NeoMathEngine.h, cited per function as NME.h:<line>).
 * A handle of the reference (CFloatHandle / CIntHandle = object pointer + byte offset) arrives here
 * already resolved to a plain device pointer; blob descriptors arrive as plain ints.
 *
 * Conventions
 *   - all pointers are device pointers unless the parameter name ends in _host
 *   - tensors are dense row-major; images are N,H,W,C (channels last) as in BlobDesc.h:25-35
 *   - scalars that the reference keeps in engine memory (thresholds, multipliers) are device pointers
 *   - every function enqueues work on `stream` (a hipStream_t cast to void*, 0 = the null stream)
 *     and returns without waiting for it
 *   - return value: NH_OK or an NH_ERR_* code; nhGetLastError() gives the message for the calling thread
 *   - in-place use (result aliasing an input exactly) is allowed wherever the reference allows it
 *   - convolutions and matrix products with few output tiles cut their reduction into slices that meet in a scratch
 *     block which the library allocates per (device, stream) on first need and keeps until nhStreamDestroy; their
 *     results do not depend on timing. Calls on one stream may come from several threads; do not share the block
 *     across streams by replaying a captured graph elsewhere: while a stream is being captured these calls neither
 *     allocate nor use the block (the slices then meet through fp32 atomic adds, reproducible to rounding) and
 *     record kernels only
 */
#ifndef NEOML_HIP_H
#define NEOML_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NH_API __attribute__((visibility("default")))

typedef void* nhStream;

enum {
	NH_OK = 0,
	NH_ERR_ARGUMENT = 1,   /* contract violation: the reference would hit ASSERT_EXPR */
	NH_ERR_HIP = 2,        /* a HIP runtime call failed */
	NH_ERR_MEMORY = 3,     /* allocation failed or the memory limit was exceeded (OnMemoryError) */
	NH_ERR_UNSUPPORTED = 4
};

/* ------------------------------------------------------------------------------------------------
 * Runtime: device, stream, raw memory, transfers, timing
 * ---------------------------------------------------------------------------------------------- */

NH_API const char* nhGetLastError(void);
NH_API int nhGetDeviceCount(int* count);
/* name_host: at least 256 bytes (CMathEngineInfo::Name, NME.h:1142-1150) */
NH_API int nhGetDeviceInfo(int device, char* name_host, size_t* total_memory, size_t* free_memory,
	int* compute_units, int* wave_size);
NH_API int nhSetDevice(int device);
NH_API int nhStreamCreate(nhStream* stream);
NH_API int nhStreamDestroy(nhStream stream);
NH_API int nhStreamSynchronize(nhStream stream);
/* The scratch block of a stream (see the conventions above) normally comes from the raw allocator. After
 * nhStreamBindPool it is taken from `pool` instead, so that the pool's memory limit, statistics and clean-up cover
 * everything an engine allocates (HeapAlloc's contract, src/MemoryEngineMixin.cpp:99-115); when the pool cannot give the
 * block the launch still runs, its slices meeting through atomic adds. Binding to another pool or to null hands the blocks
 * back first: the stream must be idle, and a bound pool must outlive the binding (rebind to null, release or destroy the
 * stream before nhPoolDestroy). nhStreamReleaseScratch drains the stream and frees its block, for CleanUp (NME.h:1211)
 * and for streams the library did not create; the next launch that needs a block allocates a new one. */
NH_API int nhStreamBindPool(nhStream stream, void* pool);
NH_API int nhStreamReleaseScratch(nhStream stream);

/* raw allocator under the caching pool (IRawMemoryManager, src/RawMemoryManager.h:24-29) */
NH_API int nhRawAlloc(void** ptr, size_t size);
NH_API int nhRawFree(void* ptr);

/* DataExchangeRaw (NME.h:1219-1220): both wait for completion, like the reference's memcpy */
NH_API int nhCopyHostToDevice(nhStream stream, void* dst, const void* src_host, size_t size);
NH_API int nhCopyDeviceToHost(nhStream stream, void* dst_host, const void* src, size_t size);
NH_API int nhCopyDeviceToDevice(nhStream stream, void* dst, const void* src, size_t size);

/* pinned host staging for GetBuffer/ReleaseBuffer (NME.h:1215-1216) */
NH_API int nhHostAlloc(void** ptr_host, size_t size);
NH_API int nhHostFree(void* ptr_host);

/* time between two points of a stream (IPerformanceCounters, PerformanceCounters.h:27-60) */
typedef void* nhEvent;
NH_API int nhEventCreate(nhEvent* event);
NH_API int nhEventDestroy(nhEvent event);
NH_API int nhEventRecord(nhEvent event, nhStream stream);
NH_API int nhEventSynchronize(nhEvent event);
NH_API int nhEventElapsedMs(nhEvent start, nhEvent stop, float* ms_host);

/* ------------------------------------------------------------------------------------------------
 * Caching device allocator (CMemoryPool + stack allocator behaviour,
 * src/MemoryPool.cpp:81-88,141-170,275-323; src/MathEngineStackAllocator.cpp:196-320;
 * src/MemoryEngineMixin.cpp:38-216). kind 0 = device memory, kind 1 = host memory (for tests of the
 * pool logic on machines without a GPU).
 * ---------------------------------------------------------------------------------------------- */
typedef void* nhPool;
NH_API int nhPoolCreate(nhPool* pool, int kind, size_t memory_limit);
NH_API int nhPoolDestroy(nhPool pool);
NH_API int nhPoolSetReuseMemoryMode(nhPool pool, int enable);            /* NME.h:1170 */
NH_API int nhPoolGetReuseMemoryMode(nhPool pool, int* enabled);          /* NME.h:1171 */
NH_API int nhPoolSetThreadBufferMemoryThreshold(nhPool pool, size_t t);  /* NME.h:1176 */
NH_API int nhPoolGetThreadBufferMemoryThreshold(nhPool pool, size_t* t); /* NME.h:1178 */
NH_API int nhPoolHeapAlloc(nhPool pool, size_t size, void** ptr);        /* NME.h:1180 */
NH_API int nhPoolHeapFree(nhPool pool, void* ptr);                       /* NME.h:1181 */
NH_API int nhPoolTransferToThisThread(nhPool pool, void* ptr, size_t size); /* NME.h:1185 */
NH_API int nhPoolStackAlloc(nhPool pool, size_t size, void** ptr);       /* NME.h:1195 */
NH_API int nhPoolStackFree(nhPool pool, void* ptr);                      /* NME.h:1196 */
NH_API int nhPoolCleanUp(nhPool pool);                                   /* NME.h:1211 */
NH_API int nhPoolGetPeakMemoryUsage(nhPool pool, size_t* bytes);         /* NME.h:1201 */
NH_API int nhPoolResetPeakMemoryUsage(nhPool pool);                      /* NME.h:1203 */
NH_API int nhPoolGetCurrentMemoryUsage(nhPool pool, size_t* bytes);      /* NME.h:1205 */
NH_API int nhPoolGetMemoryInPools(nhPool pool, size_t* bytes);           /* NME.h:1207 */

/* ------------------------------------------------------------------------------------------------
 * IVectorMathEngine (NME.h:69-387): element-wise kernels, HBM bound
 * ---------------------------------------------------------------------------------------------- */
NH_API int nhVectorCopy(nhStream s, float* first, const float* second, int vectorSize);              /* NME.h:73 */
NH_API int nhVectorCopyInt(nhStream s, int* first, const int* second, int vectorSize);               /* NME.h:74 */
NH_API int nhVectorFill(nhStream s, float* result, float value, int vectorSize);                     /* NME.h:86 */
NH_API int nhVectorFillInt(nhStream s, int* result, int value, int vectorSize);                      /* NME.h:87 */
NH_API int nhVectorFillFromHandle(nhStream s, float* result, int vectorSize, const float* value);    /* NME.h:90 */
NH_API int nhVectorFillFromHandleInt(nhStream s, int* result, int vectorSize, const int* value);     /* NME.h:91 */
NH_API int nhVectorConvertFloatToInt(nhStream s, const float* from, int* to, int vectorSize);        /* NME.h:94 */
NH_API int nhVectorConvertIntToFloat(nhStream s, const int* from, float* to, int vectorSize);        /* NME.h:95 */
NH_API int nhVectorELU(nhStream s, const float* first, float* result, int vectorSize, const float* alpha);      /* NME.h:136 */
NH_API int nhVectorReLU(nhStream s, const float* first, float* result, int vectorSize,
	const float* upperThreshold);                                                                    /* NME.h:144 */
NH_API int nhVectorLeakyReLU(nhStream s, const float* first, float* result, int vectorSize, const float* alpha); /* NME.h:152 */
NH_API int nhVectorHSwish(nhStream s, const float* first, float* result, int vectorSize);            /* NME.h:162 */
NH_API int nhVectorEltwiseMax(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:169 */
NH_API int nhVectorEltwiseMin(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:172 */
NH_API int nhVectorAbs(nhStream s, const float* first, float* result, int vectorSize);               /* NME.h:177 */
NH_API int nhVectorHardTanh(nhStream s, const float* first, float* result, int vectorSize);          /* NME.h:197 */
NH_API int nhVectorHardSigmoid(nhStream s, const float* first, float* result, int vectorSize,
	const float* slope, const float* bias);                                                          /* NME.h:204 */
NH_API int nhVectorNeg(nhStream s, const float* first, float* result, int vectorSize);               /* NME.h:212 */
NH_API int nhVectorExp(nhStream s, const float* first, float* result, int vectorSize);               /* NME.h:215 */
NH_API int nhVectorLog(nhStream s, const float* first, float* result, int vectorSize);               /* NME.h:218 */
NH_API int nhVectorErf(nhStream s, const float* first, float* result, int vectorSize);               /* NME.h:228 */
NH_API int nhVectorAdd(nhStream s, const float* first, const float* second, float* result, int vectorSize);     /* NME.h:236 */
NH_API int nhVectorAddInt(nhStream s, const int* first, const int* second, int* result, int vectorSize);        /* NME.h:238 */
NH_API int nhVectorAddValue(nhStream s, const float* first, float* result, int vectorSize, const float* addition); /* NME.h:240 */
NH_API int nhVectorAddValueInt(nhStream s, const int* first, int* result, int vectorSize, const int* addition); /* NME.h:242 */
NH_API int nhVectorSub(nhStream s, const float* first, const float* second, float* result, int vectorSize);     /* NME.h:249 */
NH_API int nhVectorSubInt(nhStream s, const int* first, const int* second, int* result, int vectorSize);        /* NME.h:247 */
NH_API int nhVectorMultiplyAndAdd(nhStream s, const float* first, const float* second, float* result,
	int vectorSize, const float* mult);                                                              /* NME.h:259 */
NH_API int nhVectorMultiplyAndSub(nhStream s, const float* first, const float* second, float* result,
	int vectorSize, const float* mult);                                                              /* NME.h:263 */
NH_API int nhVectorMultiply(nhStream s, const float* first, float* result, int vectorSize, const float* multiplier); /* NME.h:268 */
NH_API int nhVectorMultiplyInt(nhStream s, const int* first, int* result, int vectorSize, const int* multiplier);    /* NME.h:270 */
NH_API int nhVectorNegMultiply(nhStream s, const float* first, float* result, int vectorSize, const float* multiplier); /* NME.h:273 */
NH_API int nhVectorEltwiseMultiply(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:279 */
NH_API int nhVectorEltwiseMultiplyInt(nhStream s, const int* first, const int* second, int* result, int vectorSize);    /* NME.h:277 */
NH_API int nhVectorEltwiseMultiplyAdd(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:282 */
NH_API int nhVectorEltwiseNegMultiply(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:285 */
NH_API int nhVectorEltwiseDivide(nhStream s, const float* first, const float* second, float* result, int vectorSize);   /* NME.h:291 */
NH_API int nhVectorSqrt(nhStream s, const float* first, float* result, int vectorSize);              /* NME.h:299 */
NH_API int nhVectorInv(nhStream s, const float* first, float* result, int vectorSize);               /* NME.h:302 */
NH_API int nhVectorMinMax(nhStream s, const float* first, float* result, int vectorSize,
	const float* minValue, const float* maxValue);                                                   /* NME.h:305 */
NH_API int nhVectorSigmoid(nhStream s, const float* first, float* result, int vectorSize);           /* NME.h:311 */
NH_API int nhVectorTanh(nhStream s, const float* first, float* result, int vectorSize);              /* NME.h:319 */

/* ---- derivatives of the activations, backward pass: result = f'(first) * second; the ...DiffOp forms take the
 * activation's OUTPUT as first (NME.h:146-149, 164, 225, 313-325). upperThreshold: device scalar, as for nhVectorReLU */
NH_API int nhVectorNegLog(nhStream s, const float* first, float* result, int vectorSize);            /* NME.h:225 */
NH_API int nhVectorReLUDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* upperThreshold);                                                                    /* NME.h:146,148 */
/* The other activations' derivatives, same convention (Op = through the activation's output). alpha, slope, bias are
 * read from device memory like the forward parameters. Leaky ReLU and hard tanh have one entry for both forms: the
 * test is the same on either side of the activation. */
NH_API int nhVectorELUDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* alpha_dev);                                                                         /* NME.h:138 */
NH_API int nhVectorELUDiffOp(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* alpha_dev);                                                                         /* NME.h:140 */
NH_API int nhVectorLeakyReLUDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* alpha_dev);                                                                         /* NME.h:154,157 */
NH_API int nhVectorHardTanhDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:198,200 */
NH_API int nhVectorHardSigmoidDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* slope_dev, const float* bias_dev);                                                  /* NME.h:206 */
NH_API int nhVectorHardSigmoidDiffOp(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* slope_dev);                                                                         /* NME.h:208 */
NH_API int nhVectorAbsDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:178 */
/* element-wise parts of the hinge / squared hinge / Huber losses and their derivatives (times second), and of the L1
 * regulariser: result = first + mult * clamp( second, -threshold, threshold ), both scalars in device memory */
NH_API int nhVectorHinge(nhStream s, const float* first, float* result, int vectorSize);             /* NME.h:184 */
NH_API int nhVectorHingeDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:185 */
NH_API int nhVectorSquaredHinge(nhStream s, const float* first, float* result, int vectorSize);      /* NME.h:188 */
NH_API int nhVectorSquaredHingeDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:189 */
NH_API int nhVectorHuber(nhStream s, const float* first, float* result, int vectorSize);             /* NME.h:193 */
NH_API int nhVectorHuberDerivative(nhStream s, const float* first, float* result, int vectorSize);   /* NME.h:194 */
NH_API int nhVectorL1DiffAdd(nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* threshold_dev, const float* mult_dev);                                              /* NME.h:335 */
/* first - value, or value - first when reverse != 0: the two scalar overloads of VectorSub */
NH_API int nhVectorSubValue(nhStream s, const float* first, float value, int reverse, float* result, int vectorSize); /* NME.h:251,253 */
NH_API int nhVectorHSwishDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize);   /* NME.h:164 */
NH_API int nhVectorSigmoidDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize);  /* NME.h:313 */
NH_API int nhVectorSigmoidDiffOp(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:316 */
NH_API int nhVectorTanhDiff(nhStream s, const float* first, const float* second, float* result, int vectorSize);     /* NME.h:321 */
NH_API int nhVectorTanhDiffOp(nhStream s, const float* first, const float* second, float* result, int vectorSize);   /* NME.h:324 */
NH_API int nhVectorSum(nhStream s, const float* first, int vectorSize, float* result);               /* NME.h:105 */
NH_API int nhVectorDotProduct(nhStream s, const float* first, const float* second, int vectorSize, float* result); /* NME.h:339 */

/* ------------------------------------------------------------------------------------------------
 * IBlasEngine (NME.h:389-645)
 * ---------------------------------------------------------------------------------------------- */
NH_API int nhSetVectorToMatrixRows(nhStream s, float* result, int matrixHeight, int matrixWidth, const float* vector); /* NME.h:393 */
/* result[b][r][c] = matrix[b][r][c] + vector[b][c] */
NH_API int nhAddVectorToMatrixRows(nhStream s, int batchSize, const float* matrix, float* result,
	int matrixHeight, int matrixWidth, const float* vector);                                         /* NME.h:419 */
/* result[r][c] = matrix[r][c] + vector[r] */
NH_API int nhAddVectorToMatrixColumns(nhStream s, const float* matrix, float* result,
	int matrixHeight, int matrixWidth, const float* vector);                                         /* NME.h:423 */
NH_API int nhSubVectorFromMatrixColumns(nhStream s, const float* matrix, float* result,
	int matrixHeight, int matrixWidth, const float* vector);                                         /* NME.h:427 */
/* result[b][c] = sum_r matrix[b][r][c] */
NH_API int nhSumMatrixRows(nhStream s, int batchSize, float* result, const float* matrix,
	int matrixHeight, int matrixWidth);                                                              /* NME.h:433 */
NH_API int nhSumMatrixRowsAdd(nhStream s, int batchSize, float* result, const float* matrix,
	int matrixHeight, int matrixWidth);                                                              /* NME.h:431 */
/* result[r] = sum_c matrix[r][c] */
NH_API int nhSumMatrixColumns(nhStream s, float* result, const float* matrix, int matrixHeight, int matrixWidth); /* NME.h:439 */
NH_API int nhMatrixSoftmaxByRows(nhStream s, const float* matrix, int height, int width, float* result);          /* NME.h:450 */
NH_API int nhMatrixLogSumExpByRows(nhStream s, const float* matrix, int height, int width, float* result, int resultSize); /* NME.h:448 */
/* columnIndices may be null (the overload at NME.h:468) */
NH_API int nhFindMaxValueInRows(nhStream s, const float* matrix, int matrixHeight, int matrixWidth,
	float* result, int* columnIndices, int vectorSize);                                              /* NME.h:466-469 */
NH_API int nhFindMaxValueInColumns(nhStream s, int batchSize, const float* matrix, int matrixHeight,
	int matrixWidth, float* result, int* rowIndices, int vectorSize);                                /* NME.h:473 */
/* result[M x N] = first[M x K] * second[N x K]^T with row strides; resultBufferSize is ignored, as the reference
 * CPU engine ignores it (its fully-connected layer passes 0) */
NH_API int nhMultiplyMatrixByTransposedMatrix(nhStream s, const float* first, int firstHeight, int firstWidth,
	int firstRowSize, const float* second, int secondHeight, int secondRowSize,
	float* result, int resultRowSize, int resultBufferSize);                                         /* NME.h:529 */
NH_API int nhBatchMultiplyMatrixByTransposedMatrix(nhStream s, int batchSize, const float* first, int firstHeight,
	int firstWidth, const float* second, int secondHeight, float* result, int resultBufferSize);     /* NME.h:533 */
/* result[K1 x N] += first[M x K1]^T * second[M x N] */
NH_API int nhMultiplyTransposedMatrixByMatrixAndAdd(nhStream s, const float* first, int firstHeight, int firstWidth,
	int firstRowSize, const float* second, int secondWidth, int secondRowSize,
	float* result, int resultRowSize, int resultBufferSize);                                         /* NME.h:562 */
NH_API int nhBatchMultiplyTransposedMatrixByMatrix(nhStream s, int batchSize, const float* first, int firstHeight,
	int firstWidth, const float* second, int secondWidth, float* result, int resultBufferSize);      /* NME.h:567 */
/* result[firstSize x secondWidth] += sum over the batch of diag( first[b] ) * second[b] */
NH_API int nhMultiplyDiagMatrixByMatrixAndAdd(nhStream s, int batchSize, const float* first, int firstSize,
	const float* second, int secondWidth, float* result);                                            /* NME.h:607 */
/* result[r] = dot product of row r of first and of second */
NH_API int nhRowMultiplyMatrixByMatrix(nhStream s, const float* first, const float* second, int height, int width,
	float* result);                                                                                  /* NME.h:611 */
/* softmax derivative through its output: result = first * ( second - rowwise <first, second> ), first = softmax(x) */
NH_API int nhMatrixSoftmaxDiffOpByRows(nhStream s, const float* first, const float* second, int height, int width,
	float* result);                                                                                  /* NME.h:453 */
NH_API int nhMultiplyDiagMatrixByMatrix(nhStream s, const float* first, int firstSize, const float* second,
	int secondWidth, float* result, int resultBufferSize);                                           /* NME.h:570 */
NH_API int nhBatchMultiplyMatrixByMatrix(nhStream s, int batchSize, const float* first, int firstHeight,
	int firstWidth, const float* second, int secondWidth, float* result, int resultBufferSize);      /* NME.h:580 */
NH_API int nhBatchMultiplyMatrixByDiagMatrix(nhStream s, int batchSize, const float* first, int height, int width,
	int firstMatrixOffset, const float* second, int secondMatrixOffset, float* result, int resultBufferSize); /* NME.h:588 */
/* [b,h,m,w,c] -> [b,w,m,h,c]; resultBufferSize is ignored, as in the reference CPU engine */
NH_API int nhTransposeMatrix(nhStream s, int batchSize, const float* first, int height, int medium, int width,
	int channels, float* result, int resultBufferSize);                                              /* NME.h:599 */
NH_API int nhTransposeMatrixInt(nhStream s, int batchSize, const int* first, int height, int medium, int width,
	int channels, int* result, int resultBufferSize);                                                /* NME.h:602 */

/* ------------------------------------------------------------------------------------------------
 * IDnnEngine (NME.h:691-1113)
 * ---------------------------------------------------------------------------------------------- */

/* The seven blob dimensions of BlobDesc.h:25-35 in storage order. */
typedef struct nhBlobDesc {
	int dims[7]; /* BatchLength, BatchWidth, ListSize, Height, Width, Depth, Channels */
} nhBlobDesc;

#define NH_MAX_BLOB_DESCS 32 /* MaxBlobDescs, NME.h:1129 */

NH_API int nhBlobMergeByDim(nhStream s, int dim, const nhBlobDesc* from_host, const float* const* fromData_host,
	int fromCount, const nhBlobDesc* to_host, float* toData);                                        /* NME.h:696 (float) and :698 (int, same bytes) */
NH_API int nhBlobSplitByDim(nhStream s, int dim, const nhBlobDesc* from_host, const float* fromData,
	const nhBlobDesc* to_host, float* const* toData_host, int toCount);                              /* NME.h:700,702 */

/* BroadcastCopy: every dimension of `from` is 1 or equal to the one of `to`; values repeat along the dimensions of
 * size 1. additionalWidth (>= 1) is one more, innermost, unbroadcast dimension. 4-byte elements: serves the float
 * and the int member alike. */
NH_API int nhBroadcastCopy(nhStream s, void* to, const void* from, const nhBlobDesc* to_host,
	const nhBlobDesc* from_host, int additionalWidth);                                               /* NME.h:80,82 */

/* Dropout (InitDropout + Dropout, NME.h:932-935) with the very mask the reference's CPU engine draws for the same seed
 * (src/CPU/CpuRandom.h): out = in * mask / (1 - rate). Spatial: whole channels of an object; batchwise: the same mask
 * for every object. in == out is allowed. */
NH_API int nhDropout(nhStream s, const nhBlobDesc* input_host, float rate, int isSpatial, int isBatchwise, int seed,
	const float* in, float* out);

enum { NH_PAD_CONSTANT = 0, NH_PAD_EDGE = 1, NH_PAD_REFLECT = 2 }; /* TBlobResizePadding, NME.h:62-66 */
NH_API int nhBlobResizeImage(nhStream s, const nhBlobDesc* from_host, const float* fromData, int deltaLeft,
	int deltaRight, int deltaTop, int deltaBottom, int padding, float defaultValue,
	const nhBlobDesc* to_host, float* toData);                                                       /* NME.h:708 */

/* Plain-int form of CCommonConvolutionDesc (src/MathEngineDnnConv.h:24-46).
 * source N,H,W,Cin (Depth folded into channels); filter [Cout][fh][fw][Cin]; result N,Ho,Wo,Cout. */
typedef struct nhConvDesc {
	int batch, height, width, channels;      /* source */
	int filterCount, filterHeight, filterWidth;
	int paddingHeight, paddingWidth;
	int strideHeight, strideWidth;
	int dilationHeight, dilationWidth;
	int resultHeight, resultWidth;
} nhConvDesc;

/* InitBlobConvolution (NME.h:751): fills resultHeight/resultWidth and validates; returns NH_ERR_ARGUMENT
 * where the reference asserts. The convolution entry points also accept other result sizes: fewer or more rows (columns)
 * than equal padding on both sides gives stand for a different padding at the end (below the filter's span), which is how
 * the convolution over time runs through them (InitTimeConvolution / BlobTimeConvolution*, NME.h:724-731: the sequence
 * axis as the height, the batch width as the width, paddingFront as paddingHeight, paddingBack implied by the length). */
NH_API int nhInitBlobConvolution(nhConvDesc* desc_host);
/* freeTerm may be null */
NH_API int nhBlobConvolution(nhStream s, const nhConvDesc* desc_host, const float* source, const float* filter,
	const float* freeTerm, float* result);                                                           /* NME.h:755 */

/* nhBlobConvolution for callers that cannot allocate device memory: code recording a HIP graph, serving loops and
 * harnesses that forbid hipMalloc. No counterpart in the reference. Same arguments and results as nhBlobConvolution
 * (bit for bit: the same kernels and the same summation order). Where nhBlobConvolution lets the K slices of a launch
 * meet in a block it allocates per stream, this one uses a fixed array inside the library's device image: it never
 * calls hipMalloc / hipFree, also not while the stream is being captured (its counters are cleared by a fill kernel).
 * Limits: the partial tiles of one launch (sliced tiles x slices x 16 KiB) must fit NH_NOALLOC_SCRATCH_BYTES and the
 * sliced tiles NH_NOALLOC_MAX_SLICED_TILES, otherwise NH_ERR_ARGUMENT and nothing is launched (the ResNet-18 stages at
 * batch 64 need up to 38.5 MB). Every GPU the library runs on holds its own copy of the array until the process ends.
 * All calls on one GPU share that copy: calls that may overlap there (different streams, replays of graphs recorded
 * from it) race; serialise them. */
#define NH_NOALLOC_SCRATCH_BYTES (64u << 20)
#define NH_NOALLOC_MAX_SLICED_TILES 16384
NH_API int nhBlobConvolutionNoAlloc(nhStream s, const nhConvDesc* desc_host, const float* source, const float* filter,
	const float* freeTerm, float* result);

/* Gradients of the convolution (NME.h:757-761), same descriptor as the forward pass.
 * Backward: inputDiff = the gradient by the source; freeTerm (per source channel, may be null) is added, as the
 * reference does for the layers that run a convolution backwards as their forward pass. workspace: the filter with its
 * channel axes swapped (for the 7x7/2 stem over 3 channels: the filter in the kernel's order and the windows of the
 * input gradient that its tiles leave to be summed), nhBlobConvolutionBackwardWorkspaceSize bytes.
 * LearnAdd: filterDiff += the gradient by the filter. The gradient by the free term is a column sum of outputDiff
 * (nhSumMatrixRowsAdd over [pixels x filterCount]). */
NH_API int nhBlobConvolutionBackwardWorkspaceSize(const nhConvDesc* desc_host, size_t* bytes);
NH_API int nhBlobConvolutionBackward(nhStream s, const nhConvDesc* desc_host, const float* outputDiff,
	const float* filter, const float* freeTerm, float* inputDiff, void* workspace, size_t workspaceSize); /* NME.h:757 */
NH_API int nhBlobConvolutionLearnAdd(nhStream s, const nhConvDesc* desc_host, const float* input,
	const float* outputDiff, float* filterDiff);                                                     /* NME.h:759 */

/* depthwise: filter [fh][fw][C], no dilation (src/MathEngineDnnConv.h:69-90) */
NH_API int nhInitBlobChannelwiseConvolution(nhConvDesc* desc_host);                                  /* NME.h:766 */
NH_API int nhBlobChannelwiseConvolution(nhStream s, const nhConvDesc* desc_host, const float* source,
	const float* filter, const float* freeTerm, float* result);                                      /* NME.h:770 */

/* Gradients of the depthwise convolution. Backward: inputDiff = the gradient by the source. LearnAdd: filterDiff +=
 * the gradient by the filter, freeTermDiff (may be null) += the sum of outputDiff over the pixels. */
NH_API int nhBlobChannelwiseConvolutionBackward(nhStream s, const nhConvDesc* desc_host, const float* outputDiff,
	const float* filter, float* inputDiff);                                                          /* NME.h:774 */
NH_API int nhBlobChannelwiseConvolutionLearnAdd(nhStream s, const nhConvDesc* desc_host, const float* input,
	const float* outputDiff, float* filterDiff, float* freeTermDiff);                                /* NME.h:778 */

/* The fused blocks the graph optimizer emits for depthwise-separable networks (NME.h:1066-1072, layer classes
 * CMobileNetV2BlockLayer / CChannelwiseWith1x1Layer). Activations are TActivationFunction values reduced to what
 * the blocks support (src/CPU/Rowwise/CpuRowwiseCommon.h:79-86): ReLU with an optional upper threshold (param > 0),
 * h-swish, anything else = none. The depthwise stage is 3x3, padding 1, stride 1 or 2 (Ho = (H + stride - 1) / stride).
 * Filters: expand [E][Cin], channelwise [3][3][E], down / conv [Cout][E]; free terms may be null.
 * residual != 0 adds the block's input to its output (needs Cin == Cout, stride 1); input == output is allowed then.
 * workspace: the expanded activations between the stages, nh...WorkspaceSize bytes of device memory. */
#define NH_ACT_NONE 0
#define NH_ACT_RELU 1
#define NH_ACT_HSWISH 2
typedef struct nhSeparableBlockDesc {
	int batch, height, width;
	int inputChannels;     /* MobileNetV2Block only */
	int expandedChannels;  /* channels of the depthwise stage (= input channels of ChannelwiseWith1x1) */
	int outputChannels;
	int stride, residual;
	int expandActivation; float expandParam;           /* MobileNetV2Block only */
	int channelwiseActivation; float channelwiseParam;
} nhSeparableBlockDesc;
NH_API int nhMobileNetV2BlockWorkspaceSize(const nhSeparableBlockDesc* desc_host, size_t* bytes);
NH_API int nhMobileNetV2Block(nhStream s, const nhSeparableBlockDesc* desc_host, const float* input,
	const float* expandFilter, const float* expandFreeTerm, const float* channelwiseFilter,
	const float* channelwiseFreeTerm, const float* downFilter, const float* downFreeTerm, float* output,
	void* workspace, size_t workspaceSize);                                                          /* NME.h:1069 */
NH_API int nhChannelwiseWith1x1WorkspaceSize(const nhSeparableBlockDesc* desc_host, size_t* bytes);
NH_API int nhChannelwiseWith1x1(nhStream s, const nhSeparableBlockDesc* desc_host, const float* input,
	const float* channelwiseFilter, const float* channelwiseFreeTerm, const float* convFilter,
	const float* convFreeTerm, float* output, void* workspace, size_t workspaceSize);                /* NME.h:1066 */

/* The two halves of a MobileNetV3 block, before and after its squeeze-and-excite branch (NME.h:1073-1083, layer classes
 * CMobileNetV3PreSEBlockLayer / CMobileNetV3PostSEBlockLayer). Pre: expand 1x1 (+act) -> depthwise of any
 * nhInitBlobChannelwiseConvolution descriptor (+act); channelwise_desc describes the depthwise stage, its `channels` is
 * the expanded width; workspace holds the expanded tensor (nhMobileNetV3PreSEBlockWorkspaceSize bytes).
 * Post: output = down 1x1( act( channelwiseOutput * squeezeAndExcite[image][channel] ) ) + residual (may be null);
 * workspace: batch * pixelsPerImage * channels floats. Activations as for the blocks above. */
NH_API int nhMobileNetV3PreSEBlockWorkspaceSize(const nhConvDesc* channelwise_desc_host, size_t* bytes);
NH_API int nhMobileNetV3PreSEBlock(nhStream s, const nhConvDesc* channelwise_desc_host, int inputChannels,
	const float* input, const float* expandFilter, const float* expandFreeTerm, int expandActivation,
	float expandParam, const float* channelwiseFilter, const float* channelwiseFreeTerm, int channelwiseActivation,
	float channelwiseParam, float* output, void* workspace, size_t workspaceSize);                  /* NME.h:1073 */
NH_API int nhMobileNetV3PostSEBlock(nhStream s, int batch, int pixelsPerImage, int channels, int outputChannels,
	const float* channelwiseOutput, const float* squeezeAndExcite, const float* residual, int activation,
	float param, const float* downFilter, const float* downFreeTerm, float* output, void* workspace,
	size_t workspaceSize);                                                                          /* NME.h:1079 */
/* A convolution with the activation behind it in the same launch, as the rowwise operation chains pair them
 * (NME.h:1080-1087): nhBlobConvolution followed by NH_ACT_* (a launch that is cut into K slices applies the activation
 * as a pass of its own); the pointwise form takes a 1x1 filter [Cout][Cin] over rows = pixels */
NH_API int nhBlobConvolutionWithActivation(nhStream s, const nhConvDesc* desc_host, const float* source,
	const float* filter, const float* freeTerm, int activation, float param, float* result);
NH_API int nhPointwiseConvolutionWithActivation(nhStream s, const float* source, int rows, int channels,
	const float* filter, const float* freeTerm, int filterCount, int activation, float param, float* result);

/* CCommon2DPoolingDesc (src/MathEngineDnnPoolings.h:24-60): no padding; Ho = (H - fh) / sh + 1 */
typedef struct nhPoolingDesc {
	int batch, height, width, channels;
	int filterHeight, filterWidth, strideHeight, strideWidth;
	int resultHeight, resultWidth;
} nhPoolingDesc;
NH_API int nhInitPooling(nhPoolingDesc* desc_host);                                                  /* NME.h:817,837 */
/* maxIndices may be null; when given it receives the reference CPU engine's index (see the kernel) */
NH_API int nhBlobMaxPooling(nhStream s, const nhPoolingDesc* desc_host, const float* source, int* maxIndices,
	float* result);                                                                                  /* NME.h:821 */
NH_API int nhBlobMeanPooling(nhStream s, const nhPoolingDesc* desc_host, const float* source, float* result); /* NME.h:841 */
/* backward passes (NME.h:823-824, 842): sourceDiff receives the gradient by the pooling input; maxIndices are the
 * ones the forward pass wrote */
NH_API int nhBlobMaxPoolingBackward(nhStream s, const nhPoolingDesc* desc_host, const float* resultDiff,
	const int* maxIndices, float* sourceDiff);                                                       /* NME.h:823 */
NH_API int nhBlobMeanPoolingBackward(nhStream s, const nhPoolingDesc* desc_host, const float* resultDiff,
	float* sourceDiff);                                                                              /* NME.h:842 */

/* Two one-launch LSTMs side by side. No counterpart in the reference: its bidirectional layers are two CLstmLayer calls in
 * stream order. On a stream that has asked for it (enable != 0) a whole-sequence nhLstm launch takes at most half of the
 * compute units, and an nhLstm that follows it directly (nothing else enqueued on the stream through this library in
 * between) and touches none of its inputs, results or workspace runs beside it on a stream of the library's own; the
 * caller's stream waits for it right there, so work enqueued later is ordered behind both. Only for streams whose work
 * all goes through this library (an engine's own stream). Results are those of the calls in order. */
NH_API int nhStreamOverlapLstm(nhStream s, int enable);

/* Several small element-wise calls in one launch. No counterpart in the reference: there every call runs at once on the
 * calling thread. On a stream that has asked for it (enable != 0) a float element-wise call
 * (fill, copy, add, sub, multiply, divide, negate, abs, max, min, sqrt, inv, ReLU, sigmoid, tanh, h-swish, and the forms
 * with a device scalar: add value, multiply, neg-multiply, multiply-and-add, multiply-and-sub, eltwise multiply-add,
 * eltwise neg-multiply) is put aside: calls over at most 262144 elements together whatever their counts, a call over more
 * elements only with calls of its own count (the passes of an activation layer or of a solver over one blob: the three
 * calls of CGELULayer's sigmoid form become one pass; a large call that no other joins goes out as the launch it
 * always was; nhAddVectorToMatrixColumns, nhMultiplyDiagMatrixByMatrix, nhAddVectorToMatrixRows and
 * nhBatchMultiplyMatrixByDiagMatrix with batch 1 over more than 262144 elements are such calls too, their vector spread
 * over the rows or columns: the last four calls of CObjectNormalizationLayer are one pass). Up to eight of them are
 * launched together, in call order and with bit-identical results (a result that a later call of the same launch
 * overwrites before anything reads it is not stored), as soon as ANY other call
 * on the stream through this library arrives: a larger or different operation, a copy, an event, nhStreamSynchronize,
 * nhStreamDestroy, enable = 0, or a release of device memory (nhRawFree, a pool's clean-up). Until then their results are
 * not in memory and their operands must stay valid, so this is only for streams whose work, synchronisation included,
 * all goes through this library (an engine's own stream): synchronise with nhStreamSynchronize, not with HIP calls of
 * your own. Nothing is put aside while the stream is being captured into a graph (synchronise through the library
 * before a capture begins: what was put aside before it would otherwise become the graph's first launch). What it
 * saves: a row-normalising
 * layer (CObjectNormalizationLayer) asks for five such calls per run, each a launch of about 4 us.
 * On such a stream nhMultiplyMatrixByTransposedMatrix with a dense result (resultRowSize == secondHeight) waits for the
 * call behind it as well: nhAddVectorToMatrixRows over that result in place (batchSize 1, the same height and width) is
 * then part of the product's launch, the vector added to the accumulators on their way out, as the fully connected
 * layer's two calls ask (NeoML/src/Dnn/Layers/FullyConnectedLayer.cpp:91-99); any other call launches the product first,
 * as it was asked for. The sum is the same; where the product is cut into slices of its reduction the vector is added
 * in front of the slices instead of behind them, i.e. the last bits may differ from the two launches'.
 * In the same way nhBlobConvolution and nhBlobChannelwiseConvolution wait for an nhVectorReLU or nhVectorHSwish over
 * their result in place
 * (CConvLayer / CChannelwiseConvLayer followed by CReLULayer: the activation runs on the accumulators' way out, its
 * threshold read from the device scalar), and an nhVectorAdd over more than 262144 elements waits for an nhVectorReLU
 * over the sum in place (CEltwiseSumLayer + CReLULayer at the end of a residual block: one pass), and
 * nhBatchMultiplyMatrixByMatrix with a reduction of at most 256 waits for an nhVectorMultiply over its whole result in
 * place (CMatrixMultiplicationLayer + CLinearLayer: an attention layer's scores and their factor), and nhBlobResizeImage
 * with constant padding waits for an nhBlobMaxPooling (3x3, no indices) over the padded blob (CImageResizeLayer +
 * CMaxPoolingLayer: one launch writes both blobs), and nhSumMatrixColumns waits for the element-wise calls with one
 * operand in place over its sums (the mean and the inverse deviation of CObjectNormalizationLayer: the reduction's launch
 * applies them to each row's value). Same bits as the separate launches. */
NH_API int nhStreamDeferSmallOps(nhStream s, int enable);
/* LSTM (NME.h:1005-1011). Weights: inputWeights [4H x objectSize], recurrentWeights [4H x H]; gate order in
 * the 4H vector: main(tanh) | forget | input | output (src/CPU/CpuMathEngineDnnLstm.h:49-90).
 * Free terms, inputStateBackLink, inputMainBackLink and outputStateBackLink may be null.
 * workspace: nhLstmWorkspaceSize bytes of device memory, owned by the caller.
 * Sequences of 2+ steps with H a multiple of 16, H <= 512 and a grid that fits the device run as ONE launch whose
 * workgroups stay resident and hand the step outputs to one another through memory; it needs the device to itself
 * for that launch. The library therefore orders every such launch of the process behind the previous one on the device
 * (an event wait; the host does not block), whichever streams they use, and takes the launch-per-step kernels while the
 * stream is being captured into a graph. Its wait for a step's values is bounded: should it still trip (another process
 * occupying the device for seconds), the launch ends normally with invalid output, and the next nhStreamSynchronize /
 * nhCopyDeviceToHost ON THAT STREAM returns NH_ERR_HIP once; no other stream is told or touched. */
NH_API int nhLstmWorkspaceSize(int hiddenSize, int objectSize, int sequenceLength, int sequenceCount, size_t* bytes);
NH_API int nhLstm(nhStream s, int hiddenSize, int objectSize, const float* inputWeights, const float* inputFreeTerm,
	const float* recurrentWeights, const float* recurrentFreeTerm, int reverse, int sequenceLength,
	int sequenceCount, const float* inputStateBackLink, const float* inputMainBackLink, const float* input,
	float* outputStateBackLink, float* outputMainBackLink, void* workspace, size_t workspaceSize);

/* ---- Element-wise members beyond the inference path: comparisons, selections, powers, masked gradients, sums along a
 * dimension (what losses, ONNX-style operators and NeoML's automatic differentiation call). Semantics are the
 * reference CPU engine's (src/CPU/CpuMathEngineVectorMath.cpp, src/CPU/x86/CpuX86MathEngineVectorMath.cpp). */
NH_API int nhVectorFillBernoulli(nhStream s, float* result, float p, int vectorSize, float value, int seed);           /* NME.h:99, the CPU engine's generator */
NH_API int nhFilterSmallValues(nhStream s, float* data, int dataSize, float threshold);                              /* NME.h:102 */
NH_API int nhVectorSumAdd(nhStream s, const float* first, int vectorSize, float* result);                            /* NME.h:107 */
NH_API int nhVectorSumAlongDimension(nhStream s, const float* first, int precedingDimension, int dimension,
	int followingDimension, float* result);                                                                          /* NME.h:109 */
NH_API int nhVectorCumSumAlongDimension(nhStream s, const float* first, int precedingDimension, int dimension,
	int followingDimension, float* result, int reverse);                                                             /* NME.h:112 */
NH_API int nhVectorCumSumAlongDimensionInt(nhStream s, const int* first, int precedingDimension, int dimension,
	int followingDimension, int* result, int reverse);                                                               /* NME.h:114 */
/* cumulative = 0: VectorSumAlongDimensionDiag (NME.h:117), 1: VectorCumSumAlongDimensionDiag (NME.h:119) */
NH_API int nhVectorSumAlongDimensionDiag(nhStream s, const float* first, int precedingDimension, int dimension,
	int followingDimension, float* result, int cumulative);
NH_API int nhVectorEqualInt(nhStream s, const int* first, const int* second, float* result, int vectorSize);         /* NME.h:123 */
NH_API int nhVectorEqualValueInt(nhStream s, const int* first, float* result, int vectorSize, const int* value);     /* NME.h:126 */
NH_API int nhVectorMax(nhStream s, const float* first, float secondValue, float* result, int vectorSize);            /* NME.h:130 */
NH_API int nhVectorMaxDiff(nhStream s, const float* first, float secondValue, float* grad, int gradHeight, int gradWidth); /* NME.h:132 */
NH_API int nhVectorAbsDiffRows(nhStream s, const float* sourceGrad, int gradHeight, int gradWidth, const float* first,
	float* result);                                                                                                  /* NME.h:180 */
NH_API int nhVectorLogDiff(nhStream s, const float* sourceGrad, int gradHeight, int gradWidth, const float* value,
	float* result);                                                                                                  /* NME.h:221 */
NH_API int nhVectorBernulliKLDerivative(nhStream s, const float* estimation, float* result, int vectorSize,
	const float* target);                                                                                            /* NME.h:231 */
NH_API int nhVectorEltwiseDivideInt(nhStream s, const int* first, const int* second, int* result, int vectorSize);   /* NME.h:289 */
NH_API int nhVectorEltwisePower(nhStream s, const float* first, const float* second, float* result, int vectorSize); /* NME.h:295 */
NH_API int nhVectorMinMaxDiff(nhStream s, const float* sourceGrad, int gradHeight, int gradWidth, const float* first,
	float* result, const float* minValue, const float* maxValue);                                                    /* NME.h:307 */
NH_API int nhVectorPower(nhStream s, float exponent, const float* first, float* result, int vectorSize);             /* NME.h:327 */
NH_API int nhVectorPowerDiff(nhStream s, float exponent, const float* first, const float* second, float* result,
	int vectorSize);                                                                                                 /* NME.h:328 */
NH_API int nhVectorPowerDiffOp(nhStream s, float exponent, const float* first, const float* second, float* result,
	int vectorSize);                                                                                                 /* NME.h:330 */
NH_API int nhVectorEltwiseNotInt(nhStream s, const int* first, int* result, int vectorSize);                         /* NME.h:343 */
NH_API int nhVectorEltwiseNotNegative(nhStream s, const int* first, float* result, int vectorSize);                  /* NME.h:346 */
NH_API int nhVectorEltwiseLess(nhStream s, const float* first, const float* second, float* result, int vectorSize);  /* NME.h:349 */
/* valueFirst = 0: first[i] < second (NME.h:351); 1: second < first[i] (NME.h:353) */
NH_API int nhVectorEltwiseLessValue(nhStream s, const float* first, float second, float* result, int vectorSize, int valueFirst);
NH_API int nhVectorEltwiseLessToInt(nhStream s, const float* first, const float* second, int* result, int vectorSize); /* NME.h:357 */
NH_API int nhVectorEltwiseLessInt(nhStream s, const int* first, const int* second, int* result, int vectorSize);     /* NME.h:359 */
NH_API int nhVectorEltwiseEqualToInt(nhStream s, const float* first, const float* second, int* result, int vectorSize); /* NME.h:363 */
NH_API int nhVectorEltwiseEqualInt(nhStream s, const int* first, const int* second, int* result, int vectorSize);    /* NME.h:365 */
/* result = first != 0 ? second : third on 32-bit elements: the float (NME.h:369) and the int (NME.h:371) overload */
NH_API int nhVectorEltwiseWhere(nhStream s, const int* first, const void* second, const void* third, void* result, int vectorSize);
/* One step of VectorFindMaxValueInSet with indices (NME.h:375): where candidate[i] > result[i], both result[i] and
 * indices[i] = index follow; the caller starts from the first vector with indices 0. */
NH_API int nhVectorMaxWithIndex(nhStream s, const float* candidate, float* result, int* indices, int index, int vectorSize);
/* One target of VectorSpreadValues (NME.h:377): target[i] = source[i] where indices[i] == index. */
NH_API int nhVectorSpreadValuesTo(nhStream s, const float* source, float* target, const int* indices, int index, int vectorSize);

/* ---- Indexed additions, row scatters, lookups (embeddings), binarizations, column-wise softmax, index planes,
 * sub-sequences, up-sampling, space <-> depth: members beyond the benchmark networks' path. Semantics are the
 * reference CPU engine's (src/CPU/CpuMathEngineBlas.cpp, CpuMathEngineDnn.cpp, CpuMathEngineDnnPooling.cpp). */
NH_API int nhAddVectorToMatrixColumnsInt(nhStream s, const int* matrix, int* result, int matrixHeight, int matrixWidth,
	const int* vector);                                                                                              /* NME.h:425 */
NH_API int nhSumMatrixRowsInt(nhStream s, int batchSize, int* result, const int* matrix, int matrixHeight, int matrixWidth); /* NME.h:435 */
NH_API int nhAddDiagMatrixToMatrix(nhStream s, const float* diagMatrix, const float* matrix, int height, int width, float* result); /* NME.h:411 */
NH_API int nhMatrixColumnsEltwiseDivide(nhStream s, const float* matrix, int matrixHeight, int matrixWidth, const float* vector,
	float* result);                                                                                                  /* NME.h:443 */
NH_API int nhMultiply1DiagMatrixByMatrix(nhStream s, int batchSize, const float* first, int firstSize, const float* second,
	int secondWidth, float* result);                                                                                 /* NME.h:575 */
NH_API int nhMatrixSoftmaxByColumns(nhStream s, const float* matrix, int height, int width, float* result);          /* NME.h:458 */
NH_API int nhMatrixSoftmaxDiffOpByColumns(nhStream s, const float* first, const float* second, int height, int width,
	float* result);                                                                                                  /* NME.h:462 */
NH_API int nhFindMinValueInColumns(nhStream s, const float* matrix, int matrixHeight, int matrixWidth, float* result,
	int* rowIndices);                                                                                                /* NME.h:477 */
NH_API int nhMatrixRowsToVectorSquaredL2Distance(nhStream s, const float* matrix, int matrixHeight, int matrixWidth,
	const float* vector, float* result);                                                                             /* NME.h:865 */
/* 32-bit elements, float (NME.h:616) or int (NME.h:621); fillValue: device pointer or null for zero. Rows with a negative
 * index go nowhere; when two rows name the same target, which one stays is unspecified. */
NH_API int nhMatrixSpreadRows(nhStream s, const void* source, int height, int width, void* result, int resultHeight,
	const int* indices, const void* fillValue);
NH_API int nhMatrixSpreadRowsAdd(nhStream s, const float* source, int height, int width, float* result, const int* indices); /* NME.h:619 */
/* The indexed additions. mode 0: to[j] += from[j][first[j]] (AddMatrixElementsToVector, NME.h:404); 1: to[j][first[j]] +=
 * from[j][first[j]] (AddMatrixElementsToMatrix, NME.h:415); 2: to[i] += from[first[i]][second[i]] (NME.h:406);
 * 3: to[j][first[j]] += from[j] (AddVectorToMatrixElements, NME.h:397); 4: to[first[i]][second[i]] += from[i] (NME.h:400).
 * count = rows (modes 0, 1, 3) or elements (2, 4); width = the matrix width; indices outside the row are skipped in 0, 1, 3. */
NH_API int nhIndexedAdd(nhStream s, int mode, const float* from, float* to, int count, int width, const int* first, const int* second);
NH_API int nhBuildIntegerHist(nhStream s, const int* numbers, int numbersCount, int* result, int maxNumber);         /* NME.h:861 */
NH_API int nhEnumBinarization(nhStream s, int batchSize, const void* input, int inputIsFloat, int enumSize, float* result); /* NME.h:506, 508 */
NH_API int nhBitSetBinarization(nhStream s, int batchSize, int bitSetSize, const int* input, int outputVectorSize, float* result); /* NME.h:513 */
/* One lookup table of VectorMultichannelLookupAndCopy (NME.h:483-489): channel `channel` of each of the batchSize input
 * rows (float or int) indexes `table` (32-bit elements); the vector goes to output columns [outputOffset, +vectorSize). */
NH_API int nhLookupAndCopy(nhStream s, int batchSize, int channelCount, const void* input, int inputIsFloat, int channel,
	const void* table, int vectorCount, int vectorSize, void* output, int outputChannels, int outputOffset);
/* columns [inputOffset, +count) of every row to columns [outputOffset, +count): the channels behind the last table */
NH_API int nhCopyColumns(nhStream s, int rows, const void* input, int inputWidth, int inputOffset, void* output, int outputWidth,
	int outputOffset, int count);
/* One table of VectorMultichannelLookupAndAddToTable (NME.h:493-496): table[index] += *mult * matrix[row][matrixOffset..] */
NH_API int nhLookupAndAddToTable(nhStream s, int batchSize, int channelCount, const void* input, int inputIsFloat, int channel,
	float* table, int vectorCount, int vectorSize, const float* mult, const float* matrix, int matrixWidth, int matrixOffset);
NH_API int nhLookupAndSum(nhStream s, const int* indices, int batchSize, int indexCount, const float* table, int vectorSize,
	float* result);                                                                                                  /* NME.h:500 */
NH_API int nhLookupAndAddToWholeTable(nhStream s, const int* indices, int batchSize, int indexCount, const float* additions,
	int vectorSize, float* table, int vectorCount);                                                                  /* LookupAndAddToTable, NME.h:502 */
NH_API int nhMultiplyLookupMatrixByLookupVector(nhStream s, int batchSize, const float* matrixTable, const int* rows, int rowCount,
	int width, const float* vectorTable, const int* vectors, float* result);                                         /* NME.h:518 */
/* add = 0: NME.h:520, 1: ...AndAdd, NME.h:522 */
NH_API int nhMultiplyTransposedLookupMatrixByVector(nhStream s, int batchSize, const float* table, const int* rows, int rowCount,
	int width, const float* vector, float* result, int add);
NH_API int nhMultiplyVectorByTransposedLookupVectorAndAddToTable(nhStream s, int batchSize, float* table, int vectorSize,
	const int* index, const float* first, int firstSize, const float* secondTable, const int* secondVector);         /* NME.h:524 */
/* result = source +- the index along the middle one of [outer][indexed][inner]: AddWidthIndex (NME.h:919-920) with
 * indexed = width, AddHeightIndex (NME.h:927-928) with indexed = height */
NH_API int nhAddDimIndex(nhStream s, const void* source, void* result, int isFloat, int outerSize, int indexedSize, int innerSize,
	int forward);
NH_API int nhBlobGetSubSequence(nhStream s, const float* from, int fromLength, int batchWidth, int objectSize, int* indices,
	float* to, int toLength, int startPos, int isRev);                                                               /* NME.h:719 */
NH_API int nhUpsampling2DForward(nhStream s, int objectCount, int height, int width, int pixelSize, const void* input,
	int heightCopyCount, int widthCopyCount, void* result);                                                          /* NME.h:853, 855; 32-bit elements */
NH_API int nhUpsampling2DBackward(nhStream s, int objectCount, int height, int width, int pixelSize, const float* input,
	int heightCopyCount, int widthCopyCount, float* result);                                                         /* NME.h:857; height, width: of the result */
/* SpaceToDepth (isForward, NME.h:902-904) and DepthToSpace (NME.h:909-911) on 32-bit elements; dataRowCount = objects x rows
 * of blocks, dataRowWidth = blocks per row, blockChannels = channels of the "space" side */
NH_API int nhSpaceToDepth(nhStream s, const void* source, int dataRowCount, int dataRowWidth, int blockChannels, int blockSize,
	int isForward, void* result);
NH_API int nhReorg(nhStream s, const void* source, int stride, int isForward, int batchSize, int channels, int height, int width,
	void* result);                                                                                                   /* NME.h:895-897; 32-bit elements */

/* BlobGlobalMaxPooling (NME.h:787): per (object, channel) the maxCount largest of poolSize values, descending, with their
 * pixel indices; equal values: the later pixel first; empty slots hold -FLT_MAX / -1. source [objects][poolSize][channels],
 * result and maxIndices [objects][maxCount][channels]. */
NH_API int nhBlobGlobalMaxPooling(nhStream s, int objectCount, int poolSize, int channels, int maxCount, const float* source,
	int* maxIndices, float* result);
NH_API int nhBlobGlobalMaxPoolingBackward(nhStream s, int objectCount, int poolSize, int channels, int maxCount,
	const float* resultDiff, const int* maxIndices, float* sourceDiff);                                              /* NME.h:789 */
/* BlobMaxOverTimePooling (NME.h:830): source [sourceLength][seqElemSize]; maxIndices may be null */
NH_API int nhBlobMaxOverTimePooling(nhStream s, int sourceLength, int seqElemSize, int filterLen, int strideLen, const float* source,
	int* maxIndices, float* result);
/* global = 0: BlobMaxOverTimePoolingBackward (NME.h:832, additions); 1: BlobGlobalMaxOverTimePoolingBackward (NME.h:850, stores).
 * The forward pass of the global form is nhFindMaxValueInColumns over [sourceLength][seqElemSize]. */
NH_API int nhBlobOverTimePoolingBackward(nhStream s, int sourceLength, int resultLength, int seqElemSize, const float* resultDiff,
	const int* maxIndices, float* sourceDiff, int global);
/* LinearInterpolation (NME.h:1049). coords: 0 half pixel, 1 PyTorch half pixel, 2 align corners, 3 asymmetric
 * (TInterpolationCoords, NME.h:40-46); round: 0 none, 1 half down, 2 half up, 3 floor, 4 ceil (TInterpolationRound, NME.h:51-57) */
NH_API int nhLinearInterpolation(nhStream s, const float* data, float* result, int coords, int round, int objectCount, int scaledAxis,
	int objectSize, float scale);
NH_API int nhScatterND(nhStream s, const int* indices, const void* updates, void* data, const nhBlobDesc* dataDesc_host, int updateCount,
	int indexDims);                                                                                                  /* NME.h:1061-1063; 32-bit elements */

/* ---- members that no network of the benchmark configurations calls (rare_ops.hip): plain kernels -------------------- */
/* QRNN poolings (NME.h:943-962). reverse != 0: the sequence is walked from its last element. initialState may be null.
 * The backward passes walk in the same direction, read the state "before" an element at the next position of the walk and
 * add every element's recurrent share onto resultDiff there: resultDiff is modified, as in the reference. */
NH_API int nhQrnnFPooling(nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* initialState, float* result);                                                                        /* NME.h:943 */
NH_API int nhQrnnFPoolingBackward(nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* initialState, const float* result, float* resultDiff, float* updateDiff, float* forgetDiff);         /* NME.h:948 */
NH_API int nhQrnnIfPooling(nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* input, const float* initialState, float* result);                                                    /* NME.h:954 */
NH_API int nhQrnnIfPoolingBackward(nhStream s, int reverse, int sequenceLength, int objectSize, const float* update, const float* forget,
	const float* input, const float* initialState, const float* result, float* resultDiff, float* updateDiff, float* forgetDiff,
	float* inputDiff);                                                                                                /* NME.h:959 */
/* IndRNN (NME.h:979-990): h_t = activation( wx_t + u * mask * h_(t-1) ); mask [batch x object] may be null; uDiff is added to */
#define NH_INDRNN_SIGMOID 0
#define NH_INDRNN_RELU 1
NH_API int nhIndRnnRecurrent(nhStream s, int reverse, int sequenceLength, int batchSize, int objectSize, int activation, const float* wx,
	const float* mask, const float* u, float* h);                                                                     /* NME.h:979 */
NH_API int nhIndRnnRecurrentBackward(nhStream s, int reverse, int sequenceLength, int batchSize, int objectSize, int activation,
	const float* mask, const float* u, const float* h, const float* hDiff, float* wxDiff);                            /* NME.h:983 */
NH_API int nhIndRnnRecurrentLearn(nhStream s, int reverse, int sequenceLength, int batchSize, int objectSize, int activation,
	const float* mask, const float* u, const float* h, const float* hDiff, float* uDiff);                             /* NME.h:988 */
/* BERT's light-weight convolution (NME.h:1039-1043): data [seqLen][batch][heads x headSize], kernel [seqLen][batch x heads][kernelSize] */
NH_API int nhBertConv(nhStream s, const float* data, const float* kernel, int seqLen, int batchSize, int numHeads, int headSize,
	int kernelSize, float* output);
NH_API int nhBertConvBackward(nhStream s, const float* data, const float* kernel, const float* outDiff, int seqLen, int batchSize,
	int numHeads, int headSize, int kernelSize, float* dataDiff, float* kernelDiff);
/* Local response normalization over the channels (NME.h:994-1002; CMathEngineLrnDesc: vectorCount = objects x positions,
 * vectorSize = channels). invSum and invSumBeta may be null in the forward pass (they are what the backward pass needs). */
NH_API int nhLrn(nhStream s, const float* input, int vectorCount, int vectorSize, int windowSize, float bias, float alpha, float beta,
	float* invSum, float* invSumBeta, float* output);
NH_API int nhLrnBackward(nhStream s, const float* input, const float* output, const float* outputDiff, const float* invSum,
	const float* invSumBeta, int vectorCount, int vectorSize, int windowSize, float alpha, float beta, float* inputDiff);
/* Products with a sparse matrix in CSR form (CSparseMatrixDesc: rows [height + 1], columns and values [elements]; NME.h:541-559) */
NH_API int nhMultiplySparseMatrixByTransposedMatrix(nhStream s, int firstHeight, int firstWidth, int secondHeight, const int* rows,
	const int* columns, const float* values, const float* second, float* result);                                     /* NME.h:541 */
/* isTransposedSparse: the sparse matrix is [resultWidth x firstHeight]; add: onto result (NME.h:550) instead of into it (NME.h:545) */
NH_API int nhMultiplyTransposedMatrixBySparseMatrix(nhStream s, int firstHeight, int firstWidth, int resultWidth, const float* first,
	const int* rows, const int* columns, const float* values, float* result, int isTransposedSparse, int add);
NH_API int nhMultiplySparseMatrixByMatrix(nhStream s, int firstHeight, int firstWidth, int secondWidth, const int* rows,
	const int* columns, const float* values, const float* second, float* result);                                     /* NME.h:554 */
NH_API int nhMultiplyTransposedSparseMatrixByMatrix(nhStream s, int firstHeight, int firstWidth, int secondWidth, const int* rows,
	const int* columns, const float* values, const float* second, float* result);                                     /* NME.h:558 */
/* the k largest values in descending order and their positions, equal values in the order of their positions (NME.h:380-383) */
NH_API int nhVectorTopK(nhStream s, const float* first, int firstSize, int k, float* result, int* indices);
NH_API int nhVectorTopKDiff(nhStream s, const float* sourceGrad, int sourceGradHeight, int sourceGradWidth, const int* indices, int k,
	float* resultGrad);
/* 3-D convolution and pooling over blobs [batch][height][width][depth][channels] (CCommon3dConvolutionDesc,
 * CCommon3dMaxPoolingDesc, CCommon3dMeanPoolingDesc); filter [filterCount][fh][fw][fd][channels]; poolings have no padding and
 * filterCount is unused there */
typedef struct nh3dDesc {
	int batch, height, width, depth, channels;
	int filterCount, filterHeight, filterWidth, filterDepth;
	int paddingHeight, paddingWidth, paddingDepth;
	int strideHeight, strideWidth, strideDepth;
	int resultHeight, resultWidth, resultDepth;
} nh3dDesc;
NH_API int nhBlob3dConvolution(nhStream s, const nh3dDesc* desc_host, const float* source, const float* filter, const float* freeTerm,
	float* result);                                                                                                   /* NME.h:741 */
/* freeTerm [channels] or null is added to every position of inputDiff */
NH_API int nhBlob3dConvolutionBackward(nhStream s, const nh3dDesc* desc_host, const float* outputDiff, const float* filter,
	const float* freeTerm, float* inputDiff);                                                                         /* NME.h:743 */
NH_API int nhBlob3dConvolutionLearnAdd(nhStream s, const nh3dDesc* desc_host, const float* input, const float* outputDiff,
	float* filterDiff, float* freeTermDiff, int freeTermDiffFromInput);                                               /* NME.h:745 */
/* maxIndices (may be null in the forward pass): offset of channel 0 of the winning position inside the source object */
NH_API int nhBlob3dMaxPooling(nhStream s, const nh3dDesc* desc_host, const float* source, int* maxIndices, float* result);   /* NME.h:798 */
NH_API int nhBlob3dMaxPoolingBackward(nhStream s, const nh3dDesc* desc_host, const float* resultDiff, const int* maxIndices,
	float* sourceDiff);                                                                                               /* NME.h:800 */
NH_API int nhBlob3dMeanPooling(nhStream s, const nh3dDesc* desc_host, const float* source, float* result);                  /* NME.h:810 */
NH_API int nhBlob3dMeanPoolingBackward(nhStream s, const nh3dDesc* desc_host, const float* resultDiff, float* sourceDiff);  /* NME.h:812 */
/* CTC loss (NME.h:1033-1036): result [resultLen][batch][classCount] before its softmax, labels [labelLen][batch]; labelLens,
 * resultLens, labelWeights and lossGradient may be null; loss receives - sum( weight * log p( labels ) ) / batch, lossGradient the
 * gradient by result (not weighted, not divided by the batch: the loss layer does both). workspace: device memory of at
 * least nhCtcLossWorkspaceSize bytes. */
NH_API int nhCtcLossWorkspaceSize(int resultLen, int batchSize, int classCount, int labelLen, size_t* bytes);
NH_API int nhCtcLossForward(nhStream s, int resultLen, int batchSize, int classCount, int labelLen, int blankLabel, int skipBlanks,
	const float* result, const int* labels, const int* labelLens, const int* resultLens, const float* labelWeights, float* loss,
	float* lossGradient, void* workspace, size_t workspaceBytes);
/* Run-length encoded black-and-white images (CRleImage, NME.h:664-686) to dense ones of stroke / non-stroke values: what
 * BlobRleConvolution and BlobRleConvolutionLearnAdd (NME.h:871-878) run in front of the ordinary convolution entry points */
NH_API int nhRleImagesToDense(nhStream s, const void* rle, int batch, int height, int width, float strokeValue, float nonStrokeValue,
	float* dense);

#ifdef __cplusplus
}
#endif

#endif /* NEOML_HIP_H */
