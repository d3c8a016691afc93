// Refcounted device storages and strided tensor views behind the
// THCuda{,Half,Long}{Storage,Tensor}_* entry points. One type-erased
// implementation serves all element types (they share a struct layout).
// Semantics follow lib/THC/generic/THCStorage.{c,cu} and
// lib/THC/generic/THCTensor.c (resize rule :773-838, views :440-520,
// squeeze :540-598, contiguity test :627-642, refcounting :702-724).
#include <cstdlib>
#include <cstring>
#include <vector>

#include "common.hpp"
#include "stream_guard.hpp"

struct THCState;

namespace thc {

static_assert(sizeof(AnyStorage) == sizeof(THCudaStorage), "storage layout");
static_assert(offsetof(AnyStorage, device) == offsetof(THCudaStorage, device), "storage layout");
static_assert(sizeof(AnyTensor) == sizeof(THCudaTensor), "tensor layout");
static_assert(offsetof(AnyTensor, flag) == offsetof(THCudaTensor, flag), "tensor layout");

// ------------------------------------------------------------- storages --

AnyStorage* storage_new(THCState* s, DType dt, ptrdiff_t size) {
  THC_ARG_CHECK(size >= 0, 2, "invalid size");
  AnyStorage* st = (AnyStorage*)calloc(1, sizeof(AnyStorage));
  st->allocator = state_allocator(s);
  st->allocatorContext = st->allocator->state;
  st->refcount = 1;
  st->flag = TH_STORAGE_REFCOUNTED | TH_STORAGE_RESIZABLE | TH_STORAGE_FREEMEM;
  st->device = state_device(s);
  st->size = size;
  if (size > 0) {
    hipError_t e = (hipError_t)st->allocator->malloc(st->allocatorContext, &st->data,
                                                     (size_t)size * dtype_size(dt),
                                                     (hipStream_t_)current_stream(s));
    if (e != hipSuccess) {
      free(st);
      THC_CHECK(e);
    }
  }
  return st;
}

void storage_retain(AnyStorage* st) {
  if (st && (st->flag & TH_STORAGE_REFCOUNTED)) __atomic_add_fetch(&st->refcount, 1, __ATOMIC_SEQ_CST);
}

void storage_free(THCState* s, AnyStorage* st) {
  if (!st || !(st->flag & TH_STORAGE_REFCOUNTED)) return;
  if (__atomic_sub_fetch(&st->refcount, 1, __ATOMIC_SEQ_CST) > 0) return;
  if ((st->flag & TH_STORAGE_FREEMEM) && st->data)
    THC_CHECK((hipError_t)st->allocator->free(st->allocatorContext, st->data));
  if (st->view) storage_free(s, st->view);
  free(st);
}

void storage_resize(THCState* s, AnyStorage* st, ptrdiff_t size, DType dt) {
  THC_ARG_CHECK(size >= 0, 2, "invalid size");
  if (!(st->flag & TH_STORAGE_RESIZABLE)) raise_error("Trying to resize storage that is not resizable");
  if (size == st->size) return;
  const size_t esz = dtype_size(dt);
  void* fresh = nullptr;
  if (size > 0) {
    THC_CHECK((hipError_t)st->allocator->malloc(st->allocatorContext, &fresh, (size_t)size * esz,
                                                (hipStream_t_)current_stream(s)));
    if (st->data) {
      const size_t keep = (size_t)(size < st->size ? size : st->size) * esz;
      if (keep)
        THC_CHECK(hipMemcpyAsync(fresh, st->data, keep, hipMemcpyDeviceToDevice, current_stream(s)));
    }
  }
  if (st->data) {
    // The copy above is still in flight on the current stream. Plain hipFree waits
    // for the device; the caching allocator parks the block for the stream it was
    // allocated on, so a copy on any other stream is reported to it first (the
    // block is then held back behind an event on that stream).
    caching_record_stream(st->data, current_stream(s));
    THC_CHECK((hipError_t)st->allocator->free(st->allocatorContext, st->data));
  }
  st->data = fresh;
  st->size = size;
  st->device = state_device(s);
}

// --------------------------------------------------------------- tensors --
AnyTensor* tensor_new(THCState*) {
  AnyTensor* t = (AnyTensor*)calloc(1, sizeof(AnyTensor));
  t->refcount = 1;
  t->flag = TH_TENSOR_REFCOUNTED;
  return t;
}

void tensor_retain(AnyTensor* t) {
  if (t->flag & TH_TENSOR_REFCOUNTED) __atomic_add_fetch(&t->refcount, 1, __ATOMIC_SEQ_CST);
}

void tensor_free(THCState* s, AnyTensor* t) {
  if (!t || !(t->flag & TH_TENSOR_REFCOUNTED)) return;
  if (__atomic_sub_fetch(&t->refcount, 1, __ATOMIC_SEQ_CST) > 0) return;
  free(t->size);
  free(t->stride);
  if (t->storage) storage_free(s, t->storage);
  free(t);
}

void tensor_resize_nd(THCState* s, AnyTensor* self, int nd, const long* size, const long* stride,
                      DType dt) {
  // Leading run of positive sizes defines the rank (a size <= 0 ends it).
  int rank = 0;
  bool same = true;
  for (int d = 0; d < nd; ++d) {
    if (size[d] <= 0) break;
    ++rank;
    if (self->nDimension > d) {
      if (size[d] != self->size[d]) same = false;
      if (stride && stride[d] >= 0 && stride[d] != self->stride[d]) same = false;
    }
  }
  if (rank != self->nDimension) same = false;
  if (same) return;

  if (rank == 0) {
    self->nDimension = 0;
    return;
  }
  if (rank != self->nDimension) {
    self->size = (long*)realloc(self->size, sizeof(long) * rank);
    self->stride = (long*)realloc(self->stride, sizeof(long) * rank);
    self->nDimension = rank;
  }
  ptrdiff_t extent = 1;
  for (int d = rank - 1; d >= 0; --d) {
    self->size[d] = size[d];
    if (stride && stride[d] >= 0)
      self->stride[d] = stride[d];
    else
      self->stride[d] = (d == rank - 1) ? 1 : self->size[d + 1] * self->stride[d + 1];
    extent += (self->size[d] - 1) * self->stride[d];
  }
  if (extent + self->storageOffset > 0) {
    if (!self->storage) self->storage = storage_new(s, dt, 0);
    if (extent + self->storageOffset > self->storage->size)
      storage_resize(s, self->storage, extent + self->storageOffset, dt);
  }
}

void tensor_set_storage_nd(THCState* s, AnyTensor* self, AnyStorage* st, ptrdiff_t off, int nd,
                           const long* size, const long* stride, DType dt) {
  if (self->storage != st) {
    if (self->storage) storage_free(s, self->storage);
    self->storage = st;
    if (st) storage_retain(st);
  }
  if (off < 0) raise_error("Tensor: invalid storage offset");
  self->storageOffset = off;
  tensor_resize_nd(s, self, nd, size, stride, dt);
}

void tensor_set(THCState* s, AnyTensor* self, AnyTensor* src, DType dt) {
  if (self != src)
    tensor_set_storage_nd(s, self, src->storage, src->storageOffset, src->nDimension, src->size,
                          src->stride, dt);
}

AnyTensor* tensor_new_with_tensor(THCState* s, AnyTensor* src, DType dt) {
  TensorRef t(s, tensor_new(s));
  tensor_set_storage_nd(s, t.t, src->storage, src->storageOffset, src->nDimension, src->size,
                        src->stride, dt);
  return t.release();
}

AnyTensor* tensor_new_with_size(THCState* s, int nd, const long* size, DType dt) {
  TensorRef t(s, tensor_new(s));
  tensor_resize_nd(s, t.t, nd, size, nullptr, dt);
  return t.release();
}

void tensor_resize_as(THCState* s, AnyTensor* self, AnyTensor* src, DType dt) {
  bool same = self->nDimension == src->nDimension;
  for (int d = 0; same && d < self->nDimension; ++d) same = self->size[d] == src->size[d];
  if (!same) tensor_resize_nd(s, self, src->nDimension, src->size, nullptr, dt);
}

void tensor_narrow(THCState* s, AnyTensor* self, AnyTensor* src, int dim, long first, long size,
                   DType dt) {
  if (!src) src = self;
  THC_ARG_CHECK(dim >= 0 && dim < src->nDimension, 3, "out of range");
  THC_ARG_CHECK(first >= 0 && first < src->size[dim], 4, "out of range");
  THC_ARG_CHECK(size > 0 && first + size <= src->size[dim], 5, "out of range");
  tensor_set(s, self, src, dt);
  if (first > 0) self->storageOffset += first * self->stride[dim];
  self->size[dim] = size;
}

void tensor_select(THCState* s, AnyTensor* self, AnyTensor* src, int dim, long idx, DType dt) {
  if (!src) src = self;
  THC_ARG_CHECK(src->nDimension > 1, 1, "cannot select on a vector");
  THC_ARG_CHECK(dim >= 0 && dim < src->nDimension, 3, "out of range");
  THC_ARG_CHECK(idx >= 0 && idx < src->size[dim], 4, "out of range");
  tensor_set(s, self, src, dt);
  tensor_narrow(s, self, nullptr, dim, idx, 1, dt);
  for (int d = dim; d < self->nDimension - 1; ++d) {
    self->size[d] = self->size[d + 1];
    self->stride[d] = self->stride[d + 1];
  }
  self->nDimension--;
}

void tensor_transpose(THCState* s, AnyTensor* self, AnyTensor* src, int d1, int d2, DType dt) {
  if (!src) src = self;
  THC_ARG_CHECK(d1 >= 0 && d1 < src->nDimension, 1, "out of range");
  THC_ARG_CHECK(d2 >= 0 && d2 < src->nDimension, 2, "out of range");
  tensor_set(s, self, src, dt);
  if (d1 == d2) return;
  std::swap(self->stride[d1], self->stride[d2]);
  std::swap(self->size[d1], self->size[d2]);
}

void tensor_squeeze(THCState* s, AnyTensor* self, AnyTensor* src, DType dt) {
  if (!src) src = self;
  tensor_set(s, self, src, dt);
  int nd = 0;
  const int srcDims = src->nDimension;
  for (int d = 0; d < srcDims; ++d) {
    if (self->size[d] != 1) {
      self->size[nd] = self->size[d];
      self->stride[nd] = self->stride[d];
      ++nd;
    }
  }
  if (nd == 0 && srcDims > 0) {  // all ones: stays a one-element vector
    self->size[0] = 1;
    self->stride[0] = 1;
    nd = 1;
  }
  self->nDimension = nd;
}

void tensor_squeeze1d(THCState* s, AnyTensor* self, AnyTensor* src, int dim, DType dt) {
  if (!src) src = self;
  THC_ARG_CHECK(dim < src->nDimension, 3, "dimension out of range");
  tensor_set(s, self, src, dt);
  if (self->size[dim] == 1 && self->nDimension > 1) {
    for (int d = dim; d < self->nDimension - 1; ++d) {
      self->size[d] = self->size[d + 1];
      self->stride[d] = self->stride[d + 1];
    }
    self->nDimension--;
  }
}

void tensor_unsqueeze1d(THCState* s, AnyTensor* self, AnyTensor* src, int dim, DType dt) {
  if (!src) src = self;
  THC_ARG_CHECK(dim >= 0 && dim <= src->nDimension, 3, "dimension out of range");
  THC_ARG_CHECK(src->nDimension > 0, 3, "cannot unsqueeze empty tensor");
  tensor_set(s, self, src, dt);
  const int nd = self->nDimension + 1;
  self->size = (long*)realloc(self->size, sizeof(long) * nd);
  self->stride = (long*)realloc(self->stride, sizeof(long) * nd);
  self->nDimension = nd;
  for (int d = nd - 1; d > dim; --d) {
    self->size[d] = self->size[d - 1];
    self->stride[d] = self->stride[d - 1];
  }
  self->stride[dim] = (dim + 1 < nd) ? self->size[dim + 1] * self->stride[dim + 1] : 1;
  self->size[dim] = 1;
}

int tensor_is_contiguous(const AnyTensor* t) {
  long z = 1;
  for (int d = t->nDimension - 1; d >= 0; --d) {
    if (t->size[d] == 1) continue;
    if (t->stride[d] != z) return 0;
    z *= t->size[d];
  }
  return 1;
}

AnyTensor* tensor_new_clone(THCState* s, AnyTensor* t, DType dt) {
  TensorRef r(s, tensor_new(s));
  tensor_resize_as(s, r.t, t, dt);
  copy_tensor(s, dt, r.t, t, false);
  return r.release();
}

AnyTensor* tensor_new_contiguous(THCState* s, AnyTensor* t, DType dt) {
  if (!tensor_is_contiguous(t)) return tensor_new_clone(s, t, dt);
  tensor_retain(t);
  return t;
}

void tensor_free_copy_to(THCState* s, AnyTensor* self, AnyTensor* dst, DType dt) {
  TensorRef hold(s, self);
  if (self != dst) copy_tensor(s, dt, dst, self, false);
}

// Host <-> device staging in logical (row-major) order.
static void tensor_copy_from_host(THCState* s, AnyTensor* self, const void* src, DType dt) {
  const ptrdiff_t n = tensor_numel(self);
  if (n == 0) return;
  const size_t bytes = (size_t)n * dtype_size(dt);
  // The copies below run on the null stream: work queued on the current stream
  // (a non-blocking one does not order itself against the null stream) may still
  // read the destination, or the block a fresh temporary was recycled from.
  THC_CHECK(hipStreamSynchronize(current_stream(s)));
  if (tensor_is_contiguous(self)) {
    THC_CHECK(hipMemcpy(tensor_data(self, dt), src, bytes, hipMemcpyHostToDevice));
    return;
  }
  TensorRef tmp(s, tensor_new_with_size(s, self->nDimension, self->size, dt));
  THC_CHECK(hipMemcpy(tensor_data(tmp.t, dt), src, bytes, hipMemcpyHostToDevice));
  copy_tensor(s, dt, self, tmp.t, false);
  THC_CHECK(hipStreamSynchronize(current_stream(s)));
}

static void tensor_copy_to_host(THCState* s, void* dst, AnyTensor* src, DType dt) {
  const ptrdiff_t n = tensor_numel(src);
  if (n == 0) return;
  TensorRef c(s, tensor_new_contiguous(s, src, dt));
  THC_CHECK(hipStreamSynchronize(current_stream(s)));
  THC_CHECK(hipMemcpy(dst, tensor_data(c.t, dt), (size_t)n * dtype_size(dt), hipMemcpyDeviceToHost));
}

// Asynchronous copies between a contiguous device tensor and host memory of the same element count,
// queued on the current stream without waiting (generic/THCTensorCopy.c:104-164, copyAsyncCPU /
// copyAsyncCuda; those take a TH tensor, which must be contiguous too: here the caller passes its
// data pointer). The host memory should be pinned for the copy to overlap with anything; the caller
// keeps it alive and untouched until the stream has passed the copy.
static void tensor_copy_async(THCState* s, AnyTensor* dev, void* host, ptrdiff_t hostElements, DType dt,
                              bool toDevice) {
  const ptrdiff_t n = tensor_numel(dev);
  THC_ARG_CHECK(n == hostElements, 2, "sizes do not match");
  THC_ARG_CHECK(n == 0 || tensor_is_contiguous(dev), toDevice ? 2 : 3,
                toDevice ? "Target tensor must be contiguous" : "Source tensor must be contiguous");
  THC_ARG_CHECK(n == 0 || host != nullptr, toDevice ? 3 : 2, "no host memory");
  if (n == 0) return;
  note_stream_use(s, {dev});
  const size_t bytes = (size_t)n * dtype_size(dt);
  if (toDevice)
    THC_CHECK(hipMemcpyAsync(tensor_data(dev, dt), host, bytes, hipMemcpyHostToDevice, current_stream(s)));
  else
    THC_CHECK(hipMemcpyAsync(host, tensor_data(dev, dt), bytes, hipMemcpyDeviceToHost, current_stream(s)));
}

}  // namespace thc

using namespace thc;

// ---------------------------------------------------------------- C ABI --
#define ST(x) ((AnyStorage*)(x))
#define TN(x) ((AnyTensor*)(x))

#define THC_AMD_DEFINE_TENSOR_API(Storage, Tensor, real, DT)                                       \
  THC_API real* Storage##_data(THCState*, const Storage* st) { return st->data; }                  \
  THC_API ptrdiff_t Storage##_size(THCState*, const Storage* st) { return st->size; }              \
  THC_API int Storage##_elementSize(THCState*) { return (int)sizeof(real); }                       \
  THC_API void Storage##_set(THCState* s, Storage* st, ptrdiff_t i, real v) {                      \
    THC_GUARD_VOID({                                                                               \
      THC_ARG_CHECK(i >= 0 && i < st->size, 2, "index out of bounds");                             \
      THC_CHECK(hipStreamSynchronize(current_stream(s)));                                          \
      THC_CHECK(hipMemcpy(st->data + i, &v, sizeof(real), hipMemcpyHostToDevice));                 \
    })                                                                                             \
  }                                                                                                \
  THC_API real Storage##_get(THCState* s, const Storage* st, ptrdiff_t i) {                        \
    real v{};                                                                                      \
    THC_GUARD_RET(v, {                                                                             \
      THC_ARG_CHECK(i >= 0 && i < st->size, 2, "index out of bounds");                             \
      THC_CHECK(hipStreamSynchronize(current_stream(s)));                                          \
      THC_CHECK(hipMemcpy(&v, st->data + i, sizeof(real), hipMemcpyDeviceToHost));                 \
    })                                                                                             \
  }                                                                                                \
  THC_API Storage* Storage##_new(THCState* s) {                                                    \
    THC_GUARD_RET(nullptr, return (Storage*)storage_new(s, DT, 0))                                 \
  }                                                                                                \
  THC_API Storage* Storage##_newWithSize(THCState* s, ptrdiff_t n) {                               \
    THC_GUARD_RET(nullptr, return (Storage*)storage_new(s, DT, n))                                 \
  }                                                                                                \
  THC_API void Storage##_retain(THCState*, Storage* st) { storage_retain(ST(st)); }                \
  THC_API void Storage##_free(THCState* s, Storage* st) { THC_GUARD_VOID(storage_free(s, ST(st))) } \
  THC_API void Storage##_resize(THCState* s, Storage* st, ptrdiff_t n) {                           \
    THC_GUARD_VOID(storage_resize(s, ST(st), n, DT))                                               \
  }                                                                                                \
  THC_API int Storage##_getDevice(THCState*, const Storage* st) { return st->device; }             \
  THC_API void Storage##_copyFromHost(THCState* s, Storage* st, const real* src, ptrdiff_t n) {    \
    THC_GUARD_VOID({                                                                               \
      THC_ARG_CHECK(n >= 0 && n <= st->size, 2, "size does not match");                            \
      THC_CHECK(hipStreamSynchronize(current_stream(s)));                                          \
      if (n) THC_CHECK(hipMemcpy(st->data, src, n * sizeof(real), hipMemcpyHostToDevice));         \
    })                                                                                             \
  }                                                                                                \
  THC_API void Storage##_copyToHost(THCState* s, real* dst, const Storage* st, ptrdiff_t n) {      \
    THC_GUARD_VOID({                                                                               \
      THC_ARG_CHECK(n >= 0 && n <= st->size, 2, "size does not match");                            \
      THC_CHECK(hipStreamSynchronize(current_stream(s)));                                          \
      if (n) THC_CHECK(hipMemcpy(dst, st->data, n * sizeof(real), hipMemcpyDeviceToHost));         \
    })                                                                                             \
  }                                                                                                \
  THC_API Storage* Tensor##_storage(THCState*, const Tensor* t) { return t->storage; }             \
  THC_API ptrdiff_t Tensor##_storageOffset(THCState*, const Tensor* t) {                           \
    return t->storageOffset;                                                                       \
  }                                                                                                \
  THC_API int Tensor##_nDimension(THCState*, const Tensor* t) { return t->nDimension; }            \
  THC_API long Tensor##_size(THCState*, const Tensor* t, int d) {                                  \
    THC_GUARD_RET(0, {                                                                             \
      THC_ARG_CHECK(d >= 0 && d < t->nDimension, 2, "out of range");                               \
      return t->size[d];                                                                           \
    })                                                                                             \
  }                                                                                                \
  THC_API long Tensor##_stride(THCState*, const Tensor* t, int d) {                                \
    THC_GUARD_RET(0, {                                                                             \
      THC_ARG_CHECK(d >= 0 && d < t->nDimension, 2, "out of range");                               \
      return t->stride[d];                                                                         \
    })                                                                                             \
  }                                                                                                \
  THC_API real* Tensor##_data(THCState*, const Tensor* t) {                                        \
    return (real*)tensor_data(TN(t), DT);                                                          \
  }                                                                                                \
  THC_API Tensor* Tensor##_new(THCState* s) { return (Tensor*)tensor_new(s); }                     \
  THC_API Tensor* Tensor##_newWithTensor(THCState* s, Tensor* t) {                                 \
    THC_GUARD_RET(nullptr, return (Tensor*)tensor_new_with_tensor(s, TN(t), DT))                   \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithStorage4d(THCState* s, Storage* st, ptrdiff_t off, long s0,      \
                                            long t0, long s1, long t1, long s2, long t2, long s3,  \
                                            long t3) {                                             \
    THC_GUARD_RET(nullptr, {                                                                       \
      long sz[4] = {s0, s1, s2, s3};                                                               \
      long sd[4] = {t0, t1, t2, t3};                                                               \
      TensorRef t(s, tensor_new(s));                                                               \
      tensor_set_storage_nd(s, t.t, ST(st), off, 4, sz, sd, DT);                                   \
      return (Tensor*)t.release();                                                                 \
    })                                                                                             \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithStorage1d(THCState* s, Storage* st, ptrdiff_t off, long s0,      \
                                            long t0) {                                             \
    return Tensor##_newWithStorage4d(s, st, off, s0, t0, -1, -1, -1, -1, -1, -1);                  \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithStorage2d(THCState* s, Storage* st, ptrdiff_t off, long s0,      \
                                            long t0, long s1, long t1) {                           \
    return Tensor##_newWithStorage4d(s, st, off, s0, t0, s1, t1, -1, -1, -1, -1);                  \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithStorage3d(THCState* s, Storage* st, ptrdiff_t off, long s0,      \
                                            long t0, long s1, long t1, long s2, long t2) {         \
    return Tensor##_newWithStorage4d(s, st, off, s0, t0, s1, t1, s2, t2, -1, -1);                  \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithSize4d(THCState* s, long s0, long s1, long s2, long s3) {        \
    THC_GUARD_RET(nullptr, {                                                                       \
      long sz[4] = {s0, s1, s2, s3};                                                               \
      return (Tensor*)tensor_new_with_size(s, 4, sz, DT);                                          \
    })                                                                                             \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithSize1d(THCState* s, long s0) {                                   \
    return Tensor##_newWithSize4d(s, s0, -1, -1, -1);                                              \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithSize2d(THCState* s, long s0, long s1) {                          \
    return Tensor##_newWithSize4d(s, s0, s1, -1, -1);                                              \
  }                                                                                                \
  THC_API Tensor* Tensor##_newWithSize3d(THCState* s, long s0, long s1, long s2) {                 \
    return Tensor##_newWithSize4d(s, s0, s1, s2, -1);                                              \
  }                                                                                                \
  THC_API Tensor* Tensor##_newClone(THCState* s, Tensor* t) {                                      \
    THC_GUARD_RET(nullptr, return (Tensor*)tensor_new_clone(s, TN(t), DT))                         \
  }                                                                                                \
  THC_API Tensor* Tensor##_newContiguous(THCState* s, Tensor* t) {                                 \
    THC_GUARD_RET(nullptr, return (Tensor*)tensor_new_contiguous(s, TN(t), DT))                    \
  }                                                                                                \
  THC_API Tensor* Tensor##_newSelect(THCState* s, Tensor* t, int d, long i) {                      \
    THC_GUARD_RET(nullptr, {                                                                       \
      TensorRef r(s, tensor_new_with_tensor(s, TN(t), DT));                                        \
      tensor_select(s, r.t, nullptr, d, i, DT);                                                    \
      return (Tensor*)r.release();                                                                 \
    })                                                                                             \
  }                                                                                                \
  THC_API Tensor* Tensor##_newNarrow(THCState* s, Tensor* t, int d, long first, long n) {          \
    THC_GUARD_RET(nullptr, {                                                                       \
      TensorRef r(s, tensor_new_with_tensor(s, TN(t), DT));                                        \
      tensor_narrow(s, r.t, nullptr, d, first, n, DT);                                             \
      return (Tensor*)r.release();                                                                 \
    })                                                                                             \
  }                                                                                                \
  THC_API Tensor* Tensor##_newTranspose(THCState* s, Tensor* t, int d1, int d2) {                  \
    THC_GUARD_RET(nullptr, {                                                                       \
      TensorRef r(s, tensor_new_with_tensor(s, TN(t), DT));                                        \
      tensor_transpose(s, r.t, nullptr, d1, d2, DT);                                               \
      return (Tensor*)r.release();                                                                 \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_resizeAs(THCState* s, Tensor* t, Tensor* src) {                            \
    THC_GUARD_VOID(tensor_resize_as(s, TN(t), TN(src), DT))                                        \
  }                                                                                                \
  THC_API void Tensor##_resize4d(THCState* s, Tensor* t, long s0, long s1, long s2, long s3) {     \
    THC_GUARD_VOID({                                                                               \
      long sz[4] = {s0, s1, s2, s3};                                                               \
      tensor_resize_nd(s, TN(t), 4, sz, nullptr, DT);                                              \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_resize1d(THCState* s, Tensor* t, long s0) {                                \
    Tensor##_resize4d(s, t, s0, -1, -1, -1);                                                       \
  }                                                                                                \
  THC_API void Tensor##_resize2d(THCState* s, Tensor* t, long s0, long s1) {                       \
    Tensor##_resize4d(s, t, s0, s1, -1, -1);                                                       \
  }                                                                                                \
  THC_API void Tensor##_resize3d(THCState* s, Tensor* t, long s0, long s1, long s2) {              \
    Tensor##_resize4d(s, t, s0, s1, s2, -1);                                                       \
  }                                                                                                \
  THC_API void Tensor##_resizeNd(THCState* s, Tensor* t, int nd, long* size, long* stride) {       \
    THC_GUARD_VOID(tensor_resize_nd(s, TN(t), nd, size, stride, DT))                               \
  }                                                                                                \
  THC_API void Tensor##_set(THCState* s, Tensor* t, Tensor* src) {                                 \
    THC_GUARD_VOID(tensor_set(s, TN(t), TN(src), DT))                                              \
  }                                                                                                \
  THC_API void Tensor##_setStorageNd(THCState* s, Tensor* t, Storage* st, ptrdiff_t off, int nd,   \
                                     long* size, long* stride) {                                   \
    THC_GUARD_VOID(tensor_set_storage_nd(s, TN(t), ST(st), off, nd, size, stride, DT))             \
  }                                                                                                \
  THC_API void Tensor##_narrow(THCState* s, Tensor* t, Tensor* src, int d, long first, long n) {   \
    THC_GUARD_VOID(tensor_narrow(s, TN(t), TN(src), d, first, n, DT))                              \
  }                                                                                                \
  THC_API void Tensor##_select(THCState* s, Tensor* t, Tensor* src, int d, long i) {               \
    THC_GUARD_VOID(tensor_select(s, TN(t), TN(src), d, i, DT))                                     \
  }                                                                                                \
  THC_API void Tensor##_transpose(THCState* s, Tensor* t, Tensor* src, int d1, int d2) {           \
    THC_GUARD_VOID(tensor_transpose(s, TN(t), TN(src), d1, d2, DT))                                \
  }                                                                                                \
  THC_API void Tensor##_squeeze(THCState* s, Tensor* t, Tensor* src) {                             \
    THC_GUARD_VOID(tensor_squeeze(s, TN(t), TN(src), DT))                                          \
  }                                                                                                \
  THC_API void Tensor##_squeeze1d(THCState* s, Tensor* t, Tensor* src, int d) {                    \
    THC_GUARD_VOID(tensor_squeeze1d(s, TN(t), TN(src), d, DT))                                     \
  }                                                                                                \
  THC_API void Tensor##_unsqueeze1d(THCState* s, Tensor* t, Tensor* src, int d) {                  \
    THC_GUARD_VOID(tensor_unsqueeze1d(s, TN(t), TN(src), d, DT))                                   \
  }                                                                                                \
  THC_API int Tensor##_isContiguous(THCState*, const Tensor* t) {                                  \
    return tensor_is_contiguous(TN(t));                                                            \
  }                                                                                                \
  THC_API int Tensor##_isSameSizeAs(THCState*, const Tensor* a, const Tensor* b) {                 \
    if (a->nDimension != b->nDimension) return 0;                                                  \
    for (int d = 0; d < a->nDimension; ++d)                                                        \
      if (a->size[d] != b->size[d]) return 0;                                                      \
    return 1;                                                                                      \
  }                                                                                                \
  THC_API int Tensor##_isSetTo(THCState*, const Tensor* a, const Tensor* b) {                      \
    if (a->storage != b->storage || a->storageOffset != b->storageOffset ||                        \
        a->nDimension != b->nDimension)                                                            \
      return 0;                                                                                    \
    for (int d = 0; d < a->nDimension; ++d)                                                        \
      if (a->size[d] != b->size[d] || a->stride[d] != b->stride[d]) return 0;                      \
    return 1;                                                                                      \
  }                                                                                                \
  THC_API ptrdiff_t Tensor##_nElement(THCState*, const Tensor* t) { return tensor_numel(TN(t)); }  \
  THC_API void Tensor##_retain(THCState*, Tensor* t) { tensor_retain(TN(t)); }                     \
  THC_API void Tensor##_free(THCState* s, Tensor* t) { THC_GUARD_VOID(tensor_free(s, TN(t))) }     \
  THC_API void Tensor##_freeCopyTo(THCState* s, Tensor* t, Tensor* dst) {                          \
    THC_GUARD_VOID(tensor_free_copy_to(s, TN(t), TN(dst), DT))                                     \
  }                                                                                                \
  THC_API int Tensor##_getDevice(THCState*, const Tensor* t) {                                     \
    return t->storage ? t->storage->device : -1;                                                   \
  }                                                                                                \
  THC_API void Tensor##_copy(THCState* s, Tensor* dst, Tensor* src) {                              \
    THC_GUARD_VOID({                                                                               \
      if (dst != src) copy_tensor(s, DT, TN(dst), TN(src), false);                                 \
    })                                                                                             \
  }                                                                                                \
  THC_API void Tensor##_copyIgnoringOverlaps(THCState* s, Tensor* dst, Tensor* src) {              \
    THC_GUARD_VOID(copy_tensor(s, DT, TN(dst), TN(src), true))                                     \
  }                                                                                                \
  THC_API void Tensor##_copyFromHost(THCState* s, Tensor* self, const real* src) {                 \
    THC_GUARD_VOID(tensor_copy_from_host(s, TN(self), src, DT))                                    \
  }                                                                                                \
  THC_API void Tensor##_copyToHost(THCState* s, real* dst, Tensor* src) {                          \
    THC_GUARD_VOID(tensor_copy_to_host(s, dst, TN(src), DT))                                       \
  }                                                                                                \
  THC_API void Tensor##_copyAsyncFromHost(THCState* s, Tensor* self, const real* src, ptrdiff_t n) { \
    THC_GUARD_VOID(tensor_copy_async(s, TN(self), const_cast<real*>(src), n, DT, true))            \
  }                                                                                                \
  THC_API void Tensor##_copyAsyncToHost(THCState* s, real* dst, ptrdiff_t n, Tensor* src) {        \
    THC_GUARD_VOID(tensor_copy_async(s, TN(src), dst, n, DT, false))                               \
  }

THC_AMD_DEFINE_TENSOR_API(THCudaStorage, THCudaTensor, float, DType::F32)
THC_AMD_DEFINE_TENSOR_API(THCudaHalfStorage, THCudaHalfTensor, THHalf, DType::F16)
THC_AMD_DEFINE_TENSOR_API(THCudaLongStorage, THCudaLongTensor, long, DType::I64)

THC_AMD_DEFINE_TENSOR_API(THCudaByteStorage, THCudaByteTensor, unsigned char, DType::U8)
THC_AMD_DEFINE_TENSOR_API(THCudaCharStorage, THCudaCharTensor, char, DType::I8)
THC_AMD_DEFINE_TENSOR_API(THCudaShortStorage, THCudaShortTensor, short, DType::I16)
THC_AMD_DEFINE_TENSOR_API(THCudaIntStorage, THCudaIntTensor, int, DType::I32)
THC_AMD_DEFINE_TENSOR_API(THCudaDoubleStorage, THCudaDoubleTensor, double, DType::F64)

#define THC_AMD_DEFINE_COPY_API(Tensor, DT)                                                        \
  THC_API void Tensor##_copyCudaByte(THCState* s, Tensor* self, THCudaByteTensor* src) {           \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::U8, TN(src)))                              \
  }                                                                                                \
  THC_API void Tensor##_copyCudaChar(THCState* s, Tensor* self, THCudaCharTensor* src) {           \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::I8, TN(src)))                              \
  }                                                                                                \
  THC_API void Tensor##_copyCudaShort(THCState* s, Tensor* self, THCudaShortTensor* src) {         \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::I16, TN(src)))                             \
  }                                                                                                \
  THC_API void Tensor##_copyCudaInt(THCState* s, Tensor* self, THCudaIntTensor* src) {             \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::I32, TN(src)))                             \
  }                                                                                                \
  THC_API void Tensor##_copyCudaLong(THCState* s, Tensor* self, THCudaLongTensor* src) {           \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::I64, TN(src)))                             \
  }                                                                                                \
  THC_API void Tensor##_copyCudaFloat(THCState* s, Tensor* self, THCudaTensor* src) {              \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::F32, TN(src)))                             \
  }                                                                                                \
  THC_API void Tensor##_copyCudaDouble(THCState* s, Tensor* self, THCudaDoubleTensor* src) {       \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::F64, TN(src)))                             \
  }                                                                                                \
  THC_API void Tensor##_copyCudaHalf(THCState* s, Tensor* self, THCudaHalfTensor* src) {           \
    THC_GUARD_VOID(convert_copy(s, DT, TN(self), DType::F16, TN(src)))                             \
  }
THC_AMD_DEFINE_COPY_API(THCudaByteTensor, DType::U8)
THC_AMD_DEFINE_COPY_API(THCudaCharTensor, DType::I8)
THC_AMD_DEFINE_COPY_API(THCudaShortTensor, DType::I16)
THC_AMD_DEFINE_COPY_API(THCudaIntTensor, DType::I32)
THC_AMD_DEFINE_COPY_API(THCudaLongTensor, DType::I64)
THC_AMD_DEFINE_COPY_API(THCudaTensor, DType::F32)
THC_AMD_DEFINE_COPY_API(THCudaDoubleTensor, DType::F64)
THC_AMD_DEFINE_COPY_API(THCudaHalfTensor, DType::F16)

THC_API void THCudaHalfTensor_copyCuda(THCState* s, THCudaHalfTensor* self, THCudaTensor* src) {
  THC_GUARD_VOID(convert_copy(s, DType::F16, TN(self), DType::F32, TN(src)))
}
