/*
 * THC.h -- C ABI of the MI355X-native pointwise-apply / reduction engine.
 *
 * The entry points keep the names, argument order and argument meaning of the
 * cutorch THC C API so that a binding written against lib/THC (the
 * cwrap-generated TensorMath.c, TensorOperator.c, a LuaJIT FFI cdef) links
 * against this library unchanged for the functions declared here.
 * Each block cites the reference declaration it replaces (paths relative to
 * the cutorch source tree).
 *
 * Conventions shared with the reference:
 *   - `long` is 64 bit (LP64); sizes, strides and storage offsets count
 *     elements, not bytes.
 *   - `dim` arguments of the reductions are 0-based (the Lua binding converts).
 *   - indices written by max/min are 1-based int64 (Lua convention).
 *   - outputs may be resized in place; arguments are never consumed.
 *   - errors are reported through the TH error handler (THSetErrorHandler /
 *     THSetArgErrorHandler); the default handler prints and aborts.
 */
#ifndef THC_AMD_THC_H
#define THC_AMD_THC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
#define THC_API extern "C" __attribute__((visibility("default")))
#else
#define THC_API extern
#endif

/* ------------------------------------------------------------------------ */
/* TH error hooks (replaces THGeneral.h of torch7's TH, which cutorch takes   */
/* from outside its own tree: lib/THC/THCGeneral.h.in:4-5).                   */
/* ------------------------------------------------------------------------ */
typedef void (*THErrorHandlerFunction)(const char *msg, void *data);
typedef void (*THArgErrorHandlerFunction)(int argNumber, const char *msg, void *data);

/* Install a handler (NULL restores print-and-abort). A handler may longjmp
 * (Lua) or return; when it returns, the failing entry point returns to its
 * caller without having launched anything and THCAmd_lastError() holds the
 * message until THCAmd_clearLastError(). */
THC_API void THSetErrorHandler(THErrorHandlerFunction handler, void *data);
THC_API void THSetArgErrorHandler(THArgErrorHandlerFunction handler, void *data);
THC_API const char *THCAmd_lastError(void);
THC_API void THCAmd_clearLastError(void);

/* ------------------------------------------------------------------------ */
/* State, stream, raw device memory. lib/THC/THCGeneral.h.in:76-214           */
/* ------------------------------------------------------------------------ */
typedef struct THCState THCState;
typedef struct ihipStream_t *hipStream_t_;   /* same pointee as hipStream_t */

THC_API THCState *THCState_alloc(void);                       /* THCGeneral.h.in:125 */
THC_API void THCState_free(THCState *state);                  /* :126 */
THC_API void THCudaInit(THCState *state);                     /* :128 */
THC_API void THCudaShutdown(THCState *state);                 /* :129 */
THC_API int THCState_getNumDevices(THCState *state);          /* :161 */
THC_API hipStream_t_ THCState_getCurrentStream(THCState *state);       /* :167 */
/* The engine launches on `stream` (NULL = the device's default stream).
 * Replaces THCState_setStream (:169) for a caller that owns a HIP stream. */
THC_API void THCState_setCurrentStream(THCState *state, hipStream_t_ stream);
THC_API void *THCState_getCurrentDeviceScratchSpace(THCState *state);  /* :197 */
THC_API size_t THCState_getCurrentDeviceScratchSpaceSize(THCState *state); /* :199 */
THC_API int THCudaMalloc(THCState *state, void **ptr, size_t size);    /* :213 */
THC_API int THCudaFree(THCState *state, void *ptr);                    /* :214 */
THC_API void __THCudaCheck(int err, const char *file, const int line); /* :208 */

/* Allocator selection. THCGeneral.h.in:155-157,215-216; the caching allocator
 * replaces lib/THC/THCCachingAllocator.h:11. Storages remember the allocator
 * they came from. cutorch's init.c:1037-1042 installs the caching allocator
 * unless THC_CACHING_ALLOCATOR=0; a host does the same with
 * THCState_setDeviceAllocator(state, THCCachingAllocator_get()). */
struct _THCDeviceAllocator;
THC_API struct _THCDeviceAllocator *THCState_getDeviceAllocator(THCState *state);
THC_API void THCState_setDeviceAllocator(THCState *state, struct _THCDeviceAllocator *allocator);
THC_API int THCState_isCachingAllocatorEnabled(THCState *state);
THC_API struct _THCDeviceAllocator *THCCachingAllocator_get(void);
THC_API int THCudaMemGetInfoCached(THCState *state, size_t *freeBytes, size_t *totalBytes,
                                   size_t *largestBlock);
/* `ptr` (the start of a block handed out by the caching allocator) is used by
 * work queued on `stream`, which is not the stream it was allocated for: when
 * the block is freed it is held back until that work has completed
 * (lib/THC/THCCachingAllocator.h:13, THCCachingAllocator.cpp:221-240; the
 * stream is a raw HIP stream here, as for THCState_setCurrentStream). The
 * engine's own entry points report their operands themselves; a host calls
 * this for work it launches on its own streams. Other pointers are ignored. */
THC_API void THCCachingAllocator_recordStream(void *ptr, hipStream_t_ stream);
/* Blocks freed but still held back behind such events (diagnostic). */
THC_API size_t THCAmd_cachingAllocatorPendingBlocks(void);

/* Diagnostics with no counterpart in the reference. */
THC_API int THCAmd_getNumComputeUnits(THCState *state);
/* Force the 64-bit index kernels even when 32 bits would do (tests). */
THC_API void THCAmd_setForce64BitIndex(int enable);
/* Kernel family chosen by the last apply / reduce call on this thread
 * ("contig", "strided", "tiled", "generic", "rows", "cols", ...). */
THC_API const char *THCAmd_lastKernel(void);
/* Launch-shape tuning knobs, by name; returns 0 if the knob table is full. */
THC_API int THCAmd_setTuning(const char *key, long value);
THC_API long THCAmd_getTuning(const char *key);

/* Layout core exposed for host-side tests (no GPU needed).
 * collapse: lib/THC/THCTensorInfo.cuh:76-224; overlap and 32-bit rule:
 * lib/THC/THCTensorTypeUtils.cu:164-245; offset: THCTensorInfo.cuh:229-278. */
THC_API int THCAmd_collapseDims(int nDim, const long *size, const long *stride,
                                int excludeDim, long *outSize, long *outStride,
                                int *outDims);
THC_API int THCAmd_overlappingIndices(int nDim, const long *size, const long *stride);
THC_API int THCAmd_canUse32BitIndexMath(int nDim, const long *size, const long *stride);
THC_API long THCAmd_indexToOffset(int nDim, const long *size, const long *stride, long linearId);
/* The multiply-shift division the 64-bit index kernels use in place of
 * IndexToOffset's `/` and `%` (THCTensorInfo.cuh:229-278), evaluated on the
 * host: q = n / d, r = n % d for d >= 1. */
THC_API void THCAmd_divmod64(unsigned long long n, unsigned long long d,
                             unsigned long long *q, unsigned long long *r);
/* Joint collapse of n same-shaped operands (strides laid out operand-major,
 * n*nDim entries). Returns the collapsed rank, or -1 if the shapes cannot be
 * walked jointly. */
THC_API int THCAmd_jointCollapse(int nOperands, int nDim, const long *size,
                                 const long *strides, long *outSize, long *outStrides);
/* fp16 <-> fp32 conversion used for host staging (round-to-nearest-even);
 * THC_float2half / THC_half2float, lib/THC/THCHalf.h and THCGeneral.c:960-972 */
typedef struct { unsigned short x; } THHalf;
THC_API THHalf THC_float2half(float a);
THC_API float THC_half2float(THHalf a);

/* ------------------------------------------------------------------------ */
/* Storage / tensor structs. Field order and types follow                     */
/* lib/THC/generic/THCStorage.h:9-19 and lib/THC/generic/THCTensor.h:7-19     */
/* (mirrored a second time in FFI.lua:57-81).                                 */
/* ------------------------------------------------------------------------ */
#define TH_STORAGE_REFCOUNTED 1
#define TH_STORAGE_RESIZABLE  2
#define TH_STORAGE_FREEMEM    4
#define TH_TENSOR_REFCOUNTED  1

typedef struct _THCDeviceAllocator {          /* THCGeneral.h.in:48-55 */
  int (*malloc)(void *, void **, size_t, hipStream_t_);
  int (*realloc)(void *, void **, size_t, size_t, hipStream_t_);
  int (*free)(void *, void *);
  int (*emptyCache)(void *);
  int (*cacheInfo)(void *, int, size_t *, size_t *);
  void *state;
} THCDeviceAllocator;

#define THC_AMD_DECLARE_STRUCTS(Storage, Tensor, real)                        \
  typedef struct Storage {                                                    \
    real *data;                                                               \
    ptrdiff_t size;                                                           \
    int refcount;                                                             \
    char flag;                                                                \
    THCDeviceAllocator *allocator;                                            \
    void *allocatorContext;                                                   \
    struct Storage *view;                                                     \
    int device;                                                               \
  } Storage;                                                                  \
  typedef struct Tensor {                                                     \
    long *size;                                                               \
    long *stride;                                                             \
    int nDimension;                                                           \
    Storage *storage;                                                         \
    ptrdiff_t storageOffset;                                                  \
    int refcount;                                                             \
    char flag;                                                                \
  } Tensor;

THC_AMD_DECLARE_STRUCTS(THCudaStorage, THCudaTensor, float)
THC_AMD_DECLARE_STRUCTS(THCudaHalfStorage, THCudaHalfTensor, THHalf)
THC_AMD_DECLARE_STRUCTS(THCudaLongStorage, THCudaLongTensor, long)
THC_AMD_DECLARE_STRUCTS(THCudaByteStorage, THCudaByteTensor, unsigned char)
THC_AMD_DECLARE_STRUCTS(THCudaCharStorage, THCudaCharTensor, char)
THC_AMD_DECLARE_STRUCTS(THCudaShortStorage, THCudaShortTensor, short)
THC_AMD_DECLARE_STRUCTS(THCudaIntStorage, THCudaIntTensor, int)
THC_AMD_DECLARE_STRUCTS(THCudaDoubleStorage, THCudaDoubleTensor, double)

/* ------------------------------------------------------------------------ */
/* Storage and tensor management. generic/THCStorage.h:22-61,                 */
/* generic/THCTensor.h:22-139, generic/THCTensorCopy.h:5-6.                   */
/* The *FromHost / *ToHost calls take raw host pointers and stand in for      */
/* copyFloat / THFloatTensor_copyCuda (generic/THCTensorCopy.c:7-164), whose  */
/* THFloatTensor argument type lives in torch7's TH.                          */
/* ------------------------------------------------------------------------ */
#define THC_AMD_DECLARE_TENSOR_API(Storage, Tensor, real)                      \
  THC_API real *Storage##_data(THCState *, const Storage *);                   \
  THC_API ptrdiff_t Storage##_size(THCState *, const Storage *);               \
  THC_API int Storage##_elementSize(THCState *);                               \
  THC_API void Storage##_set(THCState *, Storage *, ptrdiff_t, real);          \
  THC_API real Storage##_get(THCState *, const Storage *, ptrdiff_t);          \
  THC_API Storage *Storage##_new(THCState *);                                  \
  THC_API Storage *Storage##_newWithSize(THCState *, ptrdiff_t size);          \
  THC_API void Storage##_retain(THCState *, Storage *);                        \
  THC_API void Storage##_free(THCState *, Storage *);                          \
  THC_API void Storage##_resize(THCState *, Storage *, ptrdiff_t size);        \
  THC_API int Storage##_getDevice(THCState *, const Storage *);                \
  THC_API void Storage##_copyFromHost(THCState *, Storage *, const real *src,  \
                                      ptrdiff_t n);                            \
  THC_API void Storage##_copyToHost(THCState *, real *dst, const Storage *,    \
                                    ptrdiff_t n);                              \
  THC_API Storage *Tensor##_storage(THCState *, const Tensor *);               \
  THC_API ptrdiff_t Tensor##_storageOffset(THCState *, const Tensor *);        \
  THC_API int Tensor##_nDimension(THCState *, const Tensor *);                 \
  THC_API long Tensor##_size(THCState *, const Tensor *, int dim);             \
  THC_API long Tensor##_stride(THCState *, const Tensor *, int dim);           \
  THC_API real *Tensor##_data(THCState *, const Tensor *);                     \
  THC_API Tensor *Tensor##_new(THCState *);                                    \
  THC_API Tensor *Tensor##_newWithTensor(THCState *, Tensor *);                \
  THC_API Tensor *Tensor##_newWithStorage1d(THCState *, Storage *, ptrdiff_t,  \
                                            long, long);                       \
  THC_API Tensor *Tensor##_newWithStorage2d(THCState *, Storage *, ptrdiff_t,  \
                                            long, long, long, long);           \
  THC_API Tensor *Tensor##_newWithStorage3d(THCState *, Storage *, ptrdiff_t,  \
                                            long, long, long, long, long,      \
                                            long);                             \
  THC_API Tensor *Tensor##_newWithStorage4d(THCState *, Storage *, ptrdiff_t,  \
                                            long, long, long, long, long,      \
                                            long, long, long);                 \
  THC_API Tensor *Tensor##_newWithSize1d(THCState *, long);                    \
  THC_API Tensor *Tensor##_newWithSize2d(THCState *, long, long);              \
  THC_API Tensor *Tensor##_newWithSize3d(THCState *, long, long, long);        \
  THC_API Tensor *Tensor##_newWithSize4d(THCState *, long, long, long, long);  \
  THC_API Tensor *Tensor##_newClone(THCState *, Tensor *);                     \
  THC_API Tensor *Tensor##_newContiguous(THCState *, Tensor *);                \
  THC_API Tensor *Tensor##_newSelect(THCState *, Tensor *, int, long);         \
  THC_API Tensor *Tensor##_newNarrow(THCState *, Tensor *, int, long, long);   \
  THC_API Tensor *Tensor##_newTranspose(THCState *, Tensor *, int, int);       \
  THC_API void Tensor##_resizeAs(THCState *, Tensor *, Tensor *src);           \
  THC_API void Tensor##_resize1d(THCState *, Tensor *, long);                  \
  THC_API void Tensor##_resize2d(THCState *, Tensor *, long, long);            \
  THC_API void Tensor##_resize3d(THCState *, Tensor *, long, long, long);      \
  THC_API void Tensor##_resize4d(THCState *, Tensor *, long, long, long,       \
                                 long);                                        \
  THC_API void Tensor##_resizeNd(THCState *, Tensor *, int nDimension,         \
                                 long *size, long *stride);                    \
  THC_API void Tensor##_set(THCState *, Tensor *, Tensor *src);                \
  THC_API void Tensor##_setStorageNd(THCState *, Tensor *, Storage *,          \
                                     ptrdiff_t, int, long *, long *);          \
  THC_API void Tensor##_narrow(THCState *, Tensor *, Tensor *src, int, long,   \
                               long);                                          \
  THC_API void Tensor##_select(THCState *, Tensor *, Tensor *src, int, long);  \
  THC_API void Tensor##_transpose(THCState *, Tensor *, Tensor *src, int,      \
                                  int);                                        \
  THC_API void Tensor##_squeeze(THCState *, Tensor *, Tensor *src);            \
  THC_API void Tensor##_squeeze1d(THCState *, Tensor *, Tensor *src, int);     \
  THC_API void Tensor##_unsqueeze1d(THCState *, Tensor *, Tensor *src, int);   \
  THC_API int Tensor##_isContiguous(THCState *, const Tensor *);               \
  THC_API int Tensor##_isSameSizeAs(THCState *, const Tensor *,                \
                                    const Tensor *);                           \
  THC_API int Tensor##_isSetTo(THCState *, const Tensor *, const Tensor *);    \
  THC_API ptrdiff_t Tensor##_nElement(THCState *, const Tensor *);             \
  THC_API void Tensor##_retain(THCState *, Tensor *);                          \
  THC_API void Tensor##_free(THCState *, Tensor *);                            \
  THC_API void Tensor##_freeCopyTo(THCState *, Tensor *, Tensor *dst);         \
  THC_API int Tensor##_getDevice(THCState *, const Tensor *);                  \
  THC_API void Tensor##_copy(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_copyIgnoringOverlaps(THCState *, Tensor *self,         \
                                             Tensor *src);                     \
  THC_API void Tensor##_copyFromHost(THCState *, Tensor *self,                 \
                                     const real *src);                         \
  THC_API void Tensor##_copyToHost(THCState *, real *dst, Tensor *src);        \
  /* generic/THCTensorCopy.h:40-41 (copyAsyncCPU / copyAsyncCuda, whose host  \
   * operand is a contiguous TH tensor): `n` elements of host memory, queued  \
   * on the current stream without waiting; the device tensor must be         \
   * contiguous and hold n elements. Pin the host memory (hipHostMalloc) for  \
   * the copy to overlap with other work, and keep it until the stream has    \
   * passed the copy. */                                                       \
  THC_API void Tensor##_copyAsyncFromHost(THCState *, Tensor *self,            \
                                          const real *src, ptrdiff_t n);      \
  THC_API void Tensor##_copyAsyncToHost(THCState *, real *dst, ptrdiff_t n,    \
                                        Tensor *src);

THC_AMD_DECLARE_TENSOR_API(THCudaStorage, THCudaTensor, float)
THC_AMD_DECLARE_TENSOR_API(THCudaHalfStorage, THCudaHalfTensor, THHalf)
THC_AMD_DECLARE_TENSOR_API(THCudaLongStorage, THCudaLongTensor, long)
THC_AMD_DECLARE_TENSOR_API(THCudaByteStorage, THCudaByteTensor, unsigned char)
THC_AMD_DECLARE_TENSOR_API(THCudaCharStorage, THCudaCharTensor, char)
THC_AMD_DECLARE_TENSOR_API(THCudaShortStorage, THCudaShortTensor, short)
THC_AMD_DECLARE_TENSOR_API(THCudaIntStorage, THCudaIntTensor, int)
THC_AMD_DECLARE_TENSOR_API(THCudaDoubleStorage, THCudaDoubleTensor, double)

/* Type-converting device copies, every destination type from every source  */
/* type: THCTensor_(copyCudaByte) ... (copyCudaHalf),                        */
/* generic/THCTensorCopy.h:16-24. Values convert as C casts do; half goes    */
/* through float. (THCudaTensor_copyCudaFloat etc. are plain copies.)        */
#define THC_AMD_DECLARE_COPY_API(Tensor)                                       \
  THC_API void Tensor##_copyCudaByte(THCState *, Tensor *self, THCudaByteTensor *src);     \
  THC_API void Tensor##_copyCudaChar(THCState *, Tensor *self, THCudaCharTensor *src);     \
  THC_API void Tensor##_copyCudaShort(THCState *, Tensor *self, THCudaShortTensor *src);   \
  THC_API void Tensor##_copyCudaInt(THCState *, Tensor *self, THCudaIntTensor *src);       \
  THC_API void Tensor##_copyCudaLong(THCState *, Tensor *self, THCudaLongTensor *src);     \
  THC_API void Tensor##_copyCudaFloat(THCState *, Tensor *self, THCudaTensor *src);        \
  THC_API void Tensor##_copyCudaDouble(THCState *, Tensor *self, THCudaDoubleTensor *src); \
  THC_API void Tensor##_copyCudaHalf(THCState *, Tensor *self, THCudaHalfTensor *src);
THC_AMD_DECLARE_COPY_API(THCudaByteTensor)
THC_AMD_DECLARE_COPY_API(THCudaCharTensor)
THC_AMD_DECLARE_COPY_API(THCudaShortTensor)
THC_AMD_DECLARE_COPY_API(THCudaIntTensor)
THC_AMD_DECLARE_COPY_API(THCudaLongTensor)
THC_AMD_DECLARE_COPY_API(THCudaTensor)
THC_AMD_DECLARE_COPY_API(THCudaDoubleTensor)
THC_AMD_DECLARE_COPY_API(THCudaHalfTensor)
/* generic/THCTensorCopy.h:35 for the half tensor */
THC_API void THCudaHalfTensor_copyCuda(THCState *, THCudaHalfTensor *self, THCudaTensor *src);

/* ------------------------------------------------------------------------ */
/* Pointwise math on the apply engine.                                        */
/*   tensor (op) scalar : generic/THCTensorMathPairwise.h:5-8                 */
/*   tensor (op) tensor : generic/THCTensorMathPointwise.h:49-53,66-67        */
/*   unary math, clamp, pow, tpow, lerp, atan2 :                              */
/*                        generic/THCTensorMathPointwise.h:7-38,43-47          */
/*   cpow cmax cmin cfmod cremainder cmaxValue cminValue : same file :52-63    */
/*   fmod remainder equal : generic/THCTensorMathPairwise.h:11-12,18           */
/*   fill / zero        : generic/THCTensorMath.h:5-6                         */
/* Reductions on the reduce engine: generic/THCTensorMathReduce.h:9-36        */
/* Scans: generic/THCTensorMathScan.h (cumsum, cumprod)                       */
/* renorm: generic/THCTensorMathReduce.h:7                                    */
/* lshift rshift clshift crshift (x * 2^v, x / 2^v for the floating types):   */
/*   generic/THCTensorMathPairwise.h:9-10, generic/THCTensorMathPointwise.h:54-55 */
/* ------------------------------------------------------------------------ */
#define THC_AMD_DECLARE_MATH_API(Tensor, real, accreal)                        \
  THC_API void Tensor##_add(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_sub(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_mul(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_div(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_cadd(THCState *, Tensor *self, Tensor *src1, real v,   \
                             Tensor *src2);                                    \
  THC_API void Tensor##_csub(THCState *, Tensor *self, Tensor *src1, real v,   \
                             Tensor *src2);                                    \
  THC_API void Tensor##_cmul(THCState *, Tensor *self, Tensor *src1,           \
                             Tensor *src2);                                    \
  THC_API void Tensor##_cdiv(THCState *, Tensor *self, Tensor *src1,           \
                             Tensor *src2);                                    \
  THC_API void Tensor##_addcmul(THCState *, Tensor *self, Tensor *t, real v,   \
                                Tensor *src1, Tensor *src2);                   \
  THC_API void Tensor##_addcdiv(THCState *, Tensor *self, Tensor *t, real v,   \
                                Tensor *src1, Tensor *src2);                   \
  THC_API void Tensor##_sigmoid(THCState *, Tensor *self, Tensor *src);       \
  THC_API void Tensor##_log(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_lgamma(THCState *, Tensor *self, Tensor *src);        \
  THC_API void Tensor##_log1p(THCState *, Tensor *self, Tensor *src);         \
  THC_API void Tensor##_exp(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_cos(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_acos(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_cosh(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_sin(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_asin(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_sinh(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_tan(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_atan(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_tanh(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_sqrt(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_rsqrt(THCState *, Tensor *self, Tensor *src);         \
  THC_API void Tensor##_ceil(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_floor(THCState *, Tensor *self, Tensor *src);         \
  THC_API void Tensor##_round(THCState *, Tensor *self, Tensor *src);         \
  THC_API void Tensor##_trunc(THCState *, Tensor *self, Tensor *src);         \
  THC_API void Tensor##_frac(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_cinv(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_neg(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_abs(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_sign(THCState *, Tensor *self, Tensor *src);          \
  THC_API void Tensor##_clamp(THCState *, Tensor *self, Tensor *src, real lo,  \
                              real hi);                                        \
  THC_API void Tensor##_pow(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_tpow(THCState *, Tensor *self, real v, Tensor *src);   \
  THC_API void Tensor##_cmaxValue(THCState *, Tensor *self, Tensor *src,       \
                                  real v);                                     \
  THC_API void Tensor##_cminValue(THCState *, Tensor *self, Tensor *src,       \
                                  real v);                                     \
  THC_API void Tensor##_fmod(THCState *, Tensor *self, Tensor *src, real v);   \
  THC_API void Tensor##_remainder(THCState *, Tensor *self, Tensor *src,       \
                                  real v);                                     \
  THC_API void Tensor##_cpow(THCState *, Tensor *self, Tensor *src1,           \
                             Tensor *src2);                                    \
  THC_API void Tensor##_cmax(THCState *, Tensor *self, Tensor *src1,           \
                             Tensor *src2);                                    \
  THC_API void Tensor##_cmin(THCState *, Tensor *self, Tensor *src1,           \
                             Tensor *src2);                                    \
  THC_API void Tensor##_cfmod(THCState *, Tensor *self, Tensor *src1,          \
                              Tensor *src2);                                   \
  THC_API void Tensor##_cremainder(THCState *, Tensor *self, Tensor *src1,     \
                                   Tensor *src2);                              \
  THC_API void Tensor##_atan2(THCState *, Tensor *self, Tensor *tx,            \
                              Tensor *ty);                                     \
  THC_API void Tensor##_lerp(THCState *, Tensor *self, Tensor *a, Tensor *b,   \
                             real w);                                          \
  THC_API int Tensor##_equal(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_fill(THCState *, Tensor *self, real v);                \
  THC_API void Tensor##_zero(THCState *, Tensor *self);                        \
  THC_API void Tensor##_sum(THCState *, Tensor *self, Tensor *src, long dim,   \
                            int keepdim);                                      \
  THC_API void Tensor##_prod(THCState *, Tensor *self, Tensor *src, long dim,  \
                             int keepdim);                                     \
  THC_API void Tensor##_mean(THCState *, Tensor *self, Tensor *src, long dim,  \
                             int keepdim);                                     \
  THC_API void Tensor##_norm(THCState *, Tensor *self, Tensor *src, real p,    \
                             long dim, int keepdim);                           \
  THC_API void Tensor##_max(THCState *, Tensor *values,                        \
                            THCudaLongTensor *indices, Tensor *src, long dim,  \
                            int keepdim);                                      \
  THC_API void Tensor##_min(THCState *, Tensor *values,                        \
                            THCudaLongTensor *indices, Tensor *src, long dim,  \
                            int keepdim);                                      \
  THC_API void Tensor##_var(THCState *, Tensor *self, Tensor *src, long dim,   \
                            int biased, int keepdim);                          \
  THC_API void Tensor##_std(THCState *, Tensor *self, Tensor *src, long dim,   \
                            int biased, int keepdim);                          \
  THC_API accreal Tensor##_varall(THCState *, Tensor *self, int biased);       \
  THC_API accreal Tensor##_stdall(THCState *, Tensor *self, int biased);       \
  THC_API void Tensor##_lshift(THCState *, Tensor *self, Tensor *src, real v); \
  THC_API void Tensor##_rshift(THCState *, Tensor *self, Tensor *src, real v); \
  THC_API void Tensor##_clshift(THCState *, Tensor *self, Tensor *src1,        \
                                Tensor *src2);                                 \
  THC_API void Tensor##_crshift(THCState *, Tensor *self, Tensor *src1,        \
                                Tensor *src2);                                 \
  THC_API void Tensor##_renorm(THCState *, Tensor *self, Tensor *src,          \
                               real p, long dim, real maxnorm);                \
  THC_API accreal Tensor##_dist(THCState *, Tensor *self, Tensor *src,         \
                                real p);                                       \
  THC_API void Tensor##_cumsum(THCState *, Tensor *self, Tensor *src,          \
                               long dim);                                      \
  THC_API void Tensor##_cumprod(THCState *, Tensor *self, Tensor *src,         \
                                long dim);                                     \
  THC_API accreal Tensor##_sumall(THCState *, Tensor *self);                   \
  THC_API accreal Tensor##_prodall(THCState *, Tensor *self);                  \
  THC_API accreal Tensor##_meanall(THCState *, Tensor *self);                  \
  THC_API accreal Tensor##_normall(THCState *, Tensor *self, real p);          \
  THC_API real Tensor##_minall(THCState *, Tensor *self);                      \
  THC_API real Tensor##_maxall(THCState *, Tensor *self);

/* ------------------------------------------------------------------------ */
/* Comparisons, every element type. Output 0/1 in a Byte tensor             */
/* (generic/THCTensorMathCompare.h:5-10, generic/THCTensorMathCompareT.h:5-10) */
/* or in a tensor of the input type (the ...T forms, same files :12-17).     */
/* The output is resized to the input's sizes.                               */
/* ------------------------------------------------------------------------ */
#define THC_AMD_DECLARE_ONE_COMPARE(TT, real, name)                        \
  THC_API void TT##_##name##Value(THCState *, THCudaByteTensor *self,      \
                                      TT *src, real value);                \
  THC_API void TT##_##name##ValueT(THCState *, TT *self, TT *src,  \
                                       real value);                            \
  THC_API void TT##_##name##Tensor(THCState *, THCudaByteTensor *self,     \
                                       TT *src1, TT *src2);            \
  THC_API void TT##_##name##TensorT(THCState *, TT *self, TT *src1,\
                                        TT *src2);
#define THC_AMD_DECLARE_COMPARE_API(Tensor, real)                              \
  THC_AMD_DECLARE_ONE_COMPARE(Tensor, real, lt)                                \
  THC_AMD_DECLARE_ONE_COMPARE(Tensor, real, gt)                                \
  THC_AMD_DECLARE_ONE_COMPARE(Tensor, real, le)                                \
  THC_AMD_DECLARE_ONE_COMPARE(Tensor, real, ge)                                \
  THC_AMD_DECLARE_ONE_COMPARE(Tensor, real, eq)                                \
  THC_AMD_DECLARE_ONE_COMPARE(Tensor, real, ne)
THC_AMD_DECLARE_COMPARE_API(THCudaByteTensor, unsigned char)
THC_AMD_DECLARE_COMPARE_API(THCudaCharTensor, char)
THC_AMD_DECLARE_COMPARE_API(THCudaShortTensor, short)
THC_AMD_DECLARE_COMPARE_API(THCudaIntTensor, int)
THC_AMD_DECLARE_COMPARE_API(THCudaLongTensor, long)
THC_AMD_DECLARE_COMPARE_API(THCudaTensor, float)
THC_AMD_DECLARE_COMPARE_API(THCudaDoubleTensor, double)
THC_AMD_DECLARE_COMPARE_API(THCudaHalfTensor, THHalf)

/* ------------------------------------------------------------------------ */
/* Pointwise math of the integer types and double: the per-type expansion    */
/* of generic/THCTensorMathPairwise.h:5-15 (scalar forms),                   */
/* generic/THCTensorMathPointwise.h:40-67 (tensor forms, addcmul/addcdiv)    */
/* and generic/THCTensorMath.h:5-6 (fill, zero). Integer arithmetic wraps    */
/* in the element type as C does; fmod takes the sign of the dividend,       */
/* remainder the sign of the divisor.                                        */
/* ------------------------------------------------------------------------ */
#define THC_AMD_DECLARE_WIDE_API(Tensor, real)                                 \
  THC_API void Tensor##_add(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_sub(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_mul(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_div(THCState *, Tensor *self, Tensor *src, real v);    \
  THC_API void Tensor##_fmod(THCState *, Tensor *self, Tensor *src, real v);   \
  THC_API void Tensor##_remainder(THCState *, Tensor *self, Tensor *src,       \
                                  real v);                                     \
  THC_API void Tensor##_lshift(THCState *, Tensor *self, Tensor *src, real v); \
  THC_API void Tensor##_rshift(THCState *, Tensor *self, Tensor *src, real v); \
  THC_API void Tensor##_cmaxValue(THCState *, Tensor *self, Tensor *src,       \
                                  real v);                                     \
  THC_API void Tensor##_cminValue(THCState *, Tensor *self, Tensor *src,       \
                                  real v);                                     \
  THC_API void Tensor##_abs(THCState *, Tensor *self, Tensor *src);            \
  THC_API void Tensor##_sign(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_clamp(THCState *, Tensor *self, Tensor *src, real lo,  \
                              real hi);                                        \
  THC_API void Tensor##_cadd(THCState *, Tensor *self, Tensor *src1, real v,   \
                             Tensor *src2);                                    \
  THC_API void Tensor##_csub(THCState *, Tensor *self, Tensor *src1, real v,   \
                             Tensor *src2);                                    \
  THC_API void Tensor##_cmul(THCState *, Tensor *self, Tensor *a, Tensor *b);  \
  THC_API void Tensor##_cdiv(THCState *, Tensor *self, Tensor *a, Tensor *b);  \
  THC_API void Tensor##_cpow(THCState *, Tensor *self, Tensor *a, Tensor *b);  \
  THC_API void Tensor##_cmax(THCState *, Tensor *self, Tensor *a, Tensor *b);  \
  THC_API void Tensor##_cmin(THCState *, Tensor *self, Tensor *a, Tensor *b);  \
  THC_API void Tensor##_cfmod(THCState *, Tensor *self, Tensor *a, Tensor *b); \
  THC_API void Tensor##_cremainder(THCState *, Tensor *self, Tensor *a,        \
                                   Tensor *b);                                 \
  THC_API void Tensor##_clshift(THCState *, Tensor *self, Tensor *a,           \
                                Tensor *b);                                    \
  THC_API void Tensor##_crshift(THCState *, Tensor *self, Tensor *a,           \
                                Tensor *b);                                    \
  THC_API void Tensor##_addcmul(THCState *, Tensor *self, Tensor *t, real v,   \
                                Tensor *src1, Tensor *src2);                   \
  THC_API void Tensor##_addcdiv(THCState *, Tensor *self, Tensor *t, real v,   \
                                Tensor *src1, Tensor *src2);                   \
  THC_API void Tensor##_fill(THCState *, Tensor *self, real v);                \
  THC_API void Tensor##_zero(THCState *, Tensor *self);
#define THC_AMD_DECLARE_BITS_API(Tensor, real)                                 \
  THC_API void Tensor##_bitand(THCState *, Tensor *self, Tensor *src, real v); \
  THC_API void Tensor##_bitor(THCState *, Tensor *self, Tensor *src, real v);  \
  THC_API void Tensor##_bitxor(THCState *, Tensor *self, Tensor *src, real v); \
  THC_API void Tensor##_cbitand(THCState *, Tensor *self, Tensor *a,           \
                                Tensor *b);                                    \
  THC_API void Tensor##_cbitor(THCState *, Tensor *self, Tensor *a, Tensor *b);\
  THC_API void Tensor##_cbitxor(THCState *, Tensor *self, Tensor *a,           \
                                Tensor *b);
THC_AMD_DECLARE_WIDE_API(THCudaByteTensor, unsigned char)
THC_AMD_DECLARE_WIDE_API(THCudaCharTensor, char)
THC_AMD_DECLARE_WIDE_API(THCudaShortTensor, short)
THC_AMD_DECLARE_WIDE_API(THCudaIntTensor, int)
THC_AMD_DECLARE_WIDE_API(THCudaLongTensor, long)
THC_AMD_DECLARE_WIDE_API(THCudaDoubleTensor, double)
THC_AMD_DECLARE_BITS_API(THCudaByteTensor, unsigned char)
THC_AMD_DECLARE_BITS_API(THCudaCharTensor, char)
THC_AMD_DECLARE_BITS_API(THCudaShortTensor, short)
THC_AMD_DECLARE_BITS_API(THCudaIntTensor, int)
THC_AMD_DECLARE_BITS_API(THCudaLongTensor, long)
/* neg: signed types only (generic/THCTensorMathPointwise.h:37-42) */
THC_API void THCudaCharTensor_neg(THCState *, THCudaCharTensor *self, THCudaCharTensor *src);
THC_API void THCudaShortTensor_neg(THCState *, THCudaShortTensor *self, THCudaShortTensor *src);
THC_API void THCudaIntTensor_neg(THCState *, THCudaIntTensor *self, THCudaIntTensor *src);
THC_API void THCudaLongTensor_neg(THCState *, THCudaLongTensor *self, THCudaLongTensor *src);
THC_API void THCudaDoubleTensor_neg(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src);
/* double: the floating-point family (generic/THCTensorMathPointwise.h:5-35) */
#define THC_AMD_DECLARE_DOUBLE_UNARY(name)                                     \
  THC_API void THCudaDoubleTensor_##name(THCState *, THCudaDoubleTensor *self, \
                                         THCudaDoubleTensor *src);
THC_AMD_DECLARE_DOUBLE_UNARY(sigmoid) THC_AMD_DECLARE_DOUBLE_UNARY(log)
THC_AMD_DECLARE_DOUBLE_UNARY(lgamma) THC_AMD_DECLARE_DOUBLE_UNARY(log1p)
THC_AMD_DECLARE_DOUBLE_UNARY(exp) THC_AMD_DECLARE_DOUBLE_UNARY(cos)
THC_AMD_DECLARE_DOUBLE_UNARY(acos) THC_AMD_DECLARE_DOUBLE_UNARY(cosh)
THC_AMD_DECLARE_DOUBLE_UNARY(sin) THC_AMD_DECLARE_DOUBLE_UNARY(asin)
THC_AMD_DECLARE_DOUBLE_UNARY(sinh) THC_AMD_DECLARE_DOUBLE_UNARY(tan)
THC_AMD_DECLARE_DOUBLE_UNARY(atan) THC_AMD_DECLARE_DOUBLE_UNARY(tanh)
THC_AMD_DECLARE_DOUBLE_UNARY(sqrt) THC_AMD_DECLARE_DOUBLE_UNARY(rsqrt)
THC_AMD_DECLARE_DOUBLE_UNARY(ceil) THC_AMD_DECLARE_DOUBLE_UNARY(floor)
THC_AMD_DECLARE_DOUBLE_UNARY(round) THC_AMD_DECLARE_DOUBLE_UNARY(trunc)
THC_AMD_DECLARE_DOUBLE_UNARY(frac) THC_AMD_DECLARE_DOUBLE_UNARY(cinv)
THC_API void THCudaDoubleTensor_pow(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src, double v);
THC_API void THCudaDoubleTensor_tpow(THCState *, THCudaDoubleTensor *self, double v, THCudaDoubleTensor *src);
THC_API void THCudaDoubleTensor_atan2(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *tx, THCudaDoubleTensor *ty);
THC_API void THCudaDoubleTensor_lerp(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *a, THCudaDoubleTensor *b, double w);

/* Reductions of the integer types and double: the per-type expansion of     */
/* generic/THCTensorMathReduce.h:18-36 and generic/THCTensorMathPairwise.h:17. */
/* accreal is long for the integer types, double for double.                  */
#define THC_AMD_DECLARE_WIDE_REDUCE_API(Tensor, real, accreal)                 \
  THC_API void Tensor##_sum(THCState *, Tensor *self, Tensor *src, long dim,   \
                            int keepdim);                                      \
  THC_API void Tensor##_prod(THCState *, Tensor *self, Tensor *src, long dim,  \
                             int keepdim);                                     \
  THC_API void Tensor##_mean(THCState *, Tensor *self, Tensor *src, long dim,  \
                             int keepdim);                                     \
  THC_API void Tensor##_max(THCState *, Tensor *values,                        \
                            THCudaLongTensor *indices, Tensor *src, long dim,  \
                            int keepdim);                                      \
  THC_API void Tensor##_min(THCState *, Tensor *values,                        \
                            THCudaLongTensor *indices, Tensor *src, long dim,  \
                            int keepdim);                                      \
  THC_API accreal Tensor##_sumall(THCState *, Tensor *self);                   \
  THC_API accreal Tensor##_prodall(THCState *, Tensor *self);                  \
  THC_API accreal Tensor##_meanall(THCState *, Tensor *self);                  \
  THC_API real Tensor##_minall(THCState *, Tensor *self);                      \
  THC_API real Tensor##_maxall(THCState *, Tensor *self);                      \
  THC_API int Tensor##_equal(THCState *, Tensor *self, Tensor *src);           \
  THC_API void Tensor##_cumsum(THCState *, Tensor *self, Tensor *src,          \
                               long dim);                                      \
  THC_API void Tensor##_cumprod(THCState *, Tensor *self, Tensor *src,         \
                                long dim);
THC_AMD_DECLARE_WIDE_REDUCE_API(THCudaByteTensor, unsigned char, long)
THC_AMD_DECLARE_WIDE_REDUCE_API(THCudaCharTensor, char, long)
THC_AMD_DECLARE_WIDE_REDUCE_API(THCudaShortTensor, short, long)
THC_AMD_DECLARE_WIDE_REDUCE_API(THCudaIntTensor, int, long)
THC_AMD_DECLARE_WIDE_REDUCE_API(THCudaLongTensor, long, long)
THC_AMD_DECLARE_WIDE_REDUCE_API(THCudaDoubleTensor, double, double)
/* lib/THC/THCTensorMath.h:52-53 */
THC_API int THCudaByteTensor_logicalall(THCState *, THCudaByteTensor *self);
THC_API int THCudaByteTensor_logicalany(THCState *, THCudaByteTensor *self);
/* double: generic/THCTensorMathReduce.h:7-14,44-45 */
THC_API void THCudaDoubleTensor_norm(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src, double p, long dim, int keepdim);
THC_API void THCudaDoubleTensor_var(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src, long dim, int biased, int keepdim);
THC_API void THCudaDoubleTensor_std(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src, long dim, int biased, int keepdim);
THC_API void THCudaDoubleTensor_renorm(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src, double p, long dim, double maxnorm);
THC_API double THCudaDoubleTensor_normall(THCState *, THCudaDoubleTensor *self, double p);
THC_API double THCudaDoubleTensor_varall(THCState *, THCudaDoubleTensor *self, int biased);
THC_API double THCudaDoubleTensor_stdall(THCState *, THCudaDoubleTensor *self, int biased);
THC_API double THCudaDoubleTensor_dist(THCState *, THCudaDoubleTensor *self, THCudaDoubleTensor *src, double p);

THC_AMD_DECLARE_MATH_API(THCudaTensor, float, float)
THC_AMD_DECLARE_MATH_API(THCudaHalfTensor, THHalf, float)

/* No counterpart in the reference. For callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc. The sum of all elements of `self`, as
 * THCudaTensor_sumall computes it (up to 2^31 elements: same launches, same
 * bits; beyond that more workgroups share the work than sumall uses, so the
 * order of the partial sums, and with it the last bits of a non-integer sum,
 * may differ), except that
 *   - `self` must be contiguous (or empty) and hold at most 2^32 elements;
 *     anything else is an argument error and nothing is launched;
 *   - the scalar is written to `*result`, a device-accessible pointer the
 *     caller owns (4 bytes), by the second launch on the current stream; the
 *     call does not wait for the stream and returns nothing. `result` is a raw
 *     pointer: if it lies in a block of the caching allocator that belongs to
 *     another stream, the caller reports that use itself
 *     (THCCachingAllocator_recordStream); `self` is reported by the call;
 *   - no device memory is allocated or freed: the per-workgroup partials go
 *     to a fixed 4 KiB array that every GPU the library runs on holds until
 *     the process ends. All calls on one GPU share that array, so calls that
 *     overlap on one GPU (several streams or host threads) race: serialise
 *     them. */
THC_API void THCudaTensor_sumallNoAlloc(THCState *state, THCudaTensor *self, float *result);

#endif /* THC_AMD_THC_H */
