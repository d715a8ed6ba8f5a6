// THGPUTensor: strided views over THGPUStorage.  Metadata logic follows
// gputorch/lib/THC/THCTensor.cpp (rawResize :623-688, rawSet :597-621,
// isContiguous :510-525, newContiguous :186-195); the strided device copy
// replaces THGPUTensor_kernel_copy (THCTensorCopy.cpp:170-290).
#include "common.h"

#include <cstdlib>
#include <cstring>
#include <vector>

using namespace thgpu;

#define THGPU_MAX_DIMS 8

namespace {

struct StridedDesc {
    int nd;
    long size[THGPU_MAX_DIMS];
    long dst_stride[THGPU_MAX_DIMS];
    long src_stride[THGPU_MAX_DIMS];
};

// One thread per element, linear index decomposed over the (common) sizes;
// innermost dimension fastest so that contiguous sides coalesce.
__global__ void strided_copy_kernel(float *__restrict__ dst, const float *__restrict__ src, StridedDesc d, long n) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long step = (long)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        long rem = i, od = 0, os = 0;
        for (int k = d.nd - 1; k >= 0; --k) {
            long q = rem / d.size[k];
            long r = rem - q * d.size[k];
            od += r * d.dst_stride[k];
            os += r * d.src_stride[k];
            rem = q;
        }
        dst[od] = src[os];
    }
}

void raw_resize(THGPUTensor *self, int nDimension, const long *size, const long *stride) {
    int d, nd = 0;
    bool same = true;
    for (d = 0; d < nDimension; d++) {
        if (size[d] > 0) {
            nd++;
            if ((self->nDimension > d) && (size[d] != self->size[d])) same = false;
            if ((self->nDimension > d) && stride && (stride[d] >= 0) && (stride[d] != self->stride[d])) same = false;
        } else
            break;
    }
    nDimension = nd;
    if (nDimension != self->nDimension) same = false;
    if (same) return;

    if (nDimension > 0) {
        // Transactional: work out the new strides and extent, grow the storage first, and commit the new
        // shape only when that succeeded.  A failed allocation (the error handler may return) leaves the
        // tensor exactly as it was, so no caller can be left holding a shape its storage does not back.
        if (nDimension > THGPU_MAX_DIMS * 4) {
            raise("Tensor: too many dimensions (%d)", nDimension);
            return;
        }
        long new_stride[THGPU_MAX_DIMS * 4];
        long total = 1;
        for (d = nDimension - 1; d >= 0; d--) {
            if (stride && (stride[d] >= 0))
                new_stride[d] = stride[d];
            else
                new_stride[d] = (d == nDimension - 1) ? 1 : size[d + 1] * new_stride[d + 1];
            total += (size[d] - 1) * new_stride[d];
        }
        // Storage only ever grows here (THCTensor.cpp:677-683).
        if (total + self->storageOffset > 0) {
            if (!self->storage) self->storage = THGPUStorage_new();
            if (!self->storage) return;
            if (total + self->storageOffset > self->storage->size) {
                if (!(self->storage->flag & TH_STORAGE_RESIZABLE)) {
                    raise("Tensor: the storage is too small for the new shape and is not resizable");
                    return;
                }
                THGPUStorage_resize(self->storage, total + self->storageOffset);
                if (total + self->storageOffset > self->storage->size) return;  // the allocation failed (reported)
            }
        }
        if (nDimension != self->nDimension) {
            self->size = static_cast<long *>(std::realloc(self->size, sizeof(long) * nDimension));
            self->stride = static_cast<long *>(std::realloc(self->stride, sizeof(long) * nDimension));
            self->nDimension = nDimension;
        }
        for (d = 0; d < nDimension; d++) {
            self->size[d] = size[d];
            self->stride[d] = new_stride[d];
        }
    } else
        self->nDimension = 0;
}

void raw_set(THGPUTensor *self, THGPUStorage *storage, long storageOffset, int nDimension, const long *size,
             const long *stride) {
    if (self->storage != storage) {
        if (self->storage) THGPUStorage_free(self->storage);
        if (storage) {
            self->storage = storage;
            THGPUStorage_retain(storage);
        } else
            self->storage = nullptr;
    }
    if (storageOffset < 0) {
        raise("Tensor: invalid storage offset");
        return;
    }
    self->storageOffset = storageOffset;
    raw_resize(self, nDimension, size, stride);
}

long elem_offset(const THGPUTensor *t, int nd, const long *x) {
    long off = t->storageOffset;
    for (int d = 0; d < nd; d++) off += x[d] * t->stride[d];
    return off;
}

template <typename HostTensor>
long host_nelement(const HostTensor *t) {
    if (t->nDimension == 0) return 0;
    long n = 1;
    for (int d = 0; d < t->nDimension; d++) n *= t->size[d];
    return n;
}

template <typename HostTensor>
bool host_contiguous(const HostTensor *t) {
    long z = 1;
    for (int d = t->nDimension - 1; d >= 0; d--) {
        if (t->size[d] != 1) {
            if (t->stride[d] == z)
                z *= t->size[d];
            else
                return false;
        }
    }
    return true;
}

// Gathers a (possibly strided) host tensor into a dense float vector.
template <typename HostTensor>
void host_gather(const HostTensor *t, std::vector<float> &out) {
    long n = host_nelement(t);
    out.resize((size_t)n);
    for (long i = 0; i < n; i++) {
        long rem = i, off = t->storageOffset;
        for (int d = t->nDimension - 1; d >= 0; d--) {
            off += (rem % t->size[d]) * t->stride[d];
            rem /= t->size[d];
        }
        out[(size_t)i] = (float)t->storage->data[off];
    }
}

template <typename HostTensor, typename T>
void host_scatter(HostTensor *t, const std::vector<float> &in) {
    long n = host_nelement(t);
    for (long i = 0; i < n; i++) {
        long rem = i, off = t->storageOffset;
        for (int d = t->nDimension - 1; d >= 0; d--) {
            off += (rem % t->size[d]) * t->stride[d];
            rem /= t->size[d];
        }
        t->storage->data[off] = (T)in[(size_t)i];
    }
}

}  // namespace

extern "C" {

THGPUStorage *THGPUTensor_storage(const THGPUTensor *self) { return self->storage; }
long THGPUTensor_storageOffset(const THGPUTensor *self) { return self->storageOffset; }
int THGPUTensor_nDimension(const THGPUTensor *self) { return self->nDimension; }

long THGPUTensor_size(const THGPUTensor *self, int dim) {
    THGPU_ARGCHECK((dim >= 0) && (dim < self->nDimension), 2, "out of range", 0);
    return self->size[dim];
}

long THGPUTensor_stride(const THGPUTensor *self, int dim) {
    THGPU_ARGCHECK((dim >= 0) && (dim < self->nDimension), 2, "out of range", 0);
    return self->stride[dim];
}

static THLongStorage *long_storage_from(const long *v, int n) {
    THLongStorage *s = static_cast<THLongStorage *>(std::calloc(1, sizeof(THLongStorage)));
    s->data = static_cast<long *>(std::malloc(sizeof(long) * (n > 0 ? n : 1)));
    if (n > 0) std::memcpy(s->data, v, sizeof(long) * n);
    s->size = n;
    s->refcount = 1;
    s->flag = TH_STORAGE_REFCOUNTED | TH_STORAGE_RESIZABLE | TH_STORAGE_FREEMEM;
    return s;
}

/* The returned THLongStorage is malloc'ed with the TH layout; release with
 * free(s->data); free(s) (or THLongStorage_free where TH is linked). */
THLongStorage *THGPUTensor_newSizeOf(THGPUTensor *self) { return long_storage_from(self->size, self->nDimension); }
THLongStorage *THGPUTensor_newStrideOf(THGPUTensor *self) { return long_storage_from(self->stride, self->nDimension); }

float *THGPUTensor_data(const THGPUTensor *self) {
    return self->storage ? self->storage->data + self->storageOffset : nullptr;
}

void THGPUTensor_setFlag(THGPUTensor *self, const char flag) { self->flag |= flag; }
void THGPUTensor_clearFlag(THGPUTensor *self, const char flag) { self->flag &= ~flag; }

THGPUTensor *THGPUTensor_new(void) {
    THGPUTensor *t = static_cast<THGPUTensor *>(std::calloc(1, sizeof(THGPUTensor)));
    if (!t) {
        raise("out of host memory");
        return nullptr;
    }
    t->refcount = 1;
    t->flag = TH_TENSOR_REFCOUNTED;
    return t;
}

THGPUTensor *THGPUTensor_newWithTensor(THGPUTensor *tensor) {
    THGPUTensor *self = THGPUTensor_new();
    raw_set(self, tensor->storage, tensor->storageOffset, tensor->nDimension, tensor->size, tensor->stride);
    return self;
}

THGPUTensor *THGPUTensor_newWithStorage(THGPUStorage *storage, long storageOffset, THLongStorage *size,
                                        THLongStorage *stride) {
    THGPUTensor *self = THGPUTensor_new();
    if (size && stride) THGPU_ARGCHECK(size->size == stride->size, 4, "inconsistent size", self);
    raw_set(self, storage, storageOffset, size ? (int)size->size : (stride ? (int)stride->size : 0),
            size ? size->data : nullptr, stride ? stride->data : nullptr);
    return self;
}

THGPUTensor *THGPUTensor_newWithStorage4d(THGPUStorage *storage, long storageOffset, long size0, long stride0,
                                          long size1, long stride1, long size2, long stride2, long size3,
                                          long stride3) {
    long size[4] = {size0, size1, size2, size3};
    long stride[4] = {stride0, stride1, stride2, stride3};
    THGPUTensor *self = THGPUTensor_new();
    raw_set(self, storage, storageOffset, 4, size, stride);
    return self;
}
THGPUTensor *THGPUTensor_newWithStorage1d(THGPUStorage *storage, long storageOffset, long size0, long stride0) {
    return THGPUTensor_newWithStorage4d(storage, storageOffset, size0, stride0, -1, -1, -1, -1, -1, -1);
}
THGPUTensor *THGPUTensor_newWithStorage2d(THGPUStorage *storage, long storageOffset, long size0, long stride0,
                                          long size1, long stride1) {
    return THGPUTensor_newWithStorage4d(storage, storageOffset, size0, stride0, size1, stride1, -1, -1, -1, -1);
}
THGPUTensor *THGPUTensor_newWithStorage3d(THGPUStorage *storage, long storageOffset, long size0, long stride0,
                                          long size1, long stride1, long size2, long stride2) {
    return THGPUTensor_newWithStorage4d(storage, storageOffset, size0, stride0, size1, stride1, size2, stride2, -1,
                                        -1);
}

THGPUTensor *THGPUTensor_newWithSize(THLongStorage *size, THLongStorage *stride) {
    return THGPUTensor_newWithStorage(nullptr, 0, size, stride);
}
THGPUTensor *THGPUTensor_newWithSize4d(long size0, long size1, long size2, long size3) {
    long size[4] = {size0, size1, size2, size3};
    THGPUTensor *self = THGPUTensor_new();
    raw_resize(self, 4, size, nullptr);
    return self;
}
THGPUTensor *THGPUTensor_newWithSize1d(long size0) { return THGPUTensor_newWithSize4d(size0, -1, -1, -1); }
THGPUTensor *THGPUTensor_newWithSize2d(long size0, long size1) { return THGPUTensor_newWithSize4d(size0, size1, -1, -1); }
THGPUTensor *THGPUTensor_newWithSize3d(long size0, long size1, long size2) {
    return THGPUTensor_newWithSize4d(size0, size1, size2, -1);
}

THGPUTensor *THGPUTensor_newClone(THGPUTensor *self) {
    THGPUTensor *t = THGPUTensor_new();
    THGPUTensor_resizeAs(t, self);
    THGPUTensor_copy(t, self);
    return t;
}

THGPUTensor *THGPUTensor_newContiguous(THGPUTensor *self) {
    if (!THGPUTensor_isContiguous(self)) return THGPUTensor_newClone(self);
    THGPUTensor_retain(self);
    return self;
}

THGPUTensor *THGPUTensor_newSelect(THGPUTensor *tensor, int dimension, long sliceIndex) {
    THGPUTensor *self = THGPUTensor_newWithTensor(tensor);
    THGPUTensor_select(self, nullptr, dimension, sliceIndex);
    return self;
}
THGPUTensor *THGPUTensor_newNarrow(THGPUTensor *tensor, int dimension, long firstIndex, long size) {
    THGPUTensor *self = THGPUTensor_newWithTensor(tensor);
    THGPUTensor_narrow(self, nullptr, dimension, firstIndex, size);
    return self;
}
THGPUTensor *THGPUTensor_newTranspose(THGPUTensor *tensor, int dimension1, int dimension2) {
    THGPUTensor *self = THGPUTensor_newWithTensor(tensor);
    THGPUTensor_transpose(self, nullptr, dimension1, dimension2);
    return self;
}

void THGPUTensor_resize(THGPUTensor *self, THLongStorage *size, THLongStorage *stride) {
    THGPU_ARGCHECK(size != nullptr, 2, "invalid size", );
    if (stride) THGPU_ARGCHECK(stride->size == size->size, 3, "invalid stride", );
    raw_resize(self, (int)size->size, size->data, stride ? stride->data : nullptr);
}

void THGPUTensor_resizeAs(THGPUTensor *self, THGPUTensor *src) {
    bool same = self->nDimension == src->nDimension;
    for (int d = 0; same && d < self->nDimension; d++) same = self->size[d] == src->size[d];
    if (!same) raw_resize(self, src->nDimension, src->size, nullptr);
}

void THGPUTensor_resize4d(THGPUTensor *self, long size0, long size1, long size2, long size3) {
    long size[4] = {size0, size1, size2, size3};
    raw_resize(self, 4, size, nullptr);
}
void THGPUTensor_resize1d(THGPUTensor *t, long size0) { THGPUTensor_resize4d(t, size0, -1, -1, -1); }
void THGPUTensor_resize2d(THGPUTensor *t, long size0, long size1) { THGPUTensor_resize4d(t, size0, size1, -1, -1); }
void THGPUTensor_resize3d(THGPUTensor *t, long size0, long size1, long size2) {
    THGPUTensor_resize4d(t, size0, size1, size2, -1);
}
void THGPUTensor_resize5d(THGPUTensor *self, long size0, long size1, long size2, long size3, long size4) {
    long size[5] = {size0, size1, size2, size3, size4};
    raw_resize(self, 5, size, nullptr);
}

void THGPUTensor_set(THGPUTensor *self, THGPUTensor *src) {
    if (self != src) raw_set(self, src->storage, src->storageOffset, src->nDimension, src->size, src->stride);
}

void THGPUTensor_setStorage(THGPUTensor *self, THGPUStorage *storage, long storageOffset, THLongStorage *size,
                            THLongStorage *stride) {
    if (size && stride) THGPU_ARGCHECK(size->size == stride->size, 5, "inconsistent size/stride sizes", );
    raw_set(self, storage, storageOffset, size ? (int)size->size : (stride ? (int)stride->size : 0),
            size ? size->data : nullptr, stride ? stride->data : nullptr);
}

void THGPUTensor_setStorage4d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0,
                              long size1, long stride1, long size2, long stride2, long size3, long stride3) {
    long size[4] = {size0, size1, size2, size3};
    long stride[4] = {stride0, stride1, stride2, stride3};
    raw_set(self, storage, storageOffset, 4, size, stride);
}
void THGPUTensor_setStorage1d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0) {
    THGPUTensor_setStorage4d(self, storage, storageOffset, size0, stride0, -1, -1, -1, -1, -1, -1);
}
void THGPUTensor_setStorage2d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0,
                              long size1, long stride1) {
    THGPUTensor_setStorage4d(self, storage, storageOffset, size0, stride0, size1, stride1, -1, -1, -1, -1);
}
void THGPUTensor_setStorage3d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0,
                              long size1, long stride1, long size2, long stride2) {
    THGPUTensor_setStorage4d(self, storage, storageOffset, size0, stride0, size1, stride1, size2, stride2, -1, -1);
}

void THGPUTensor_narrow(THGPUTensor *self, THGPUTensor *src, int dimension, long firstIndex, long size) {
    if (!src) src = self;
    THGPU_ARGCHECK((dimension >= 0) && (dimension < src->nDimension), 3, "out of range", );
    THGPU_ARGCHECK((firstIndex >= 0) && (firstIndex < src->size[dimension]), 4, "out of range", );
    THGPU_ARGCHECK((size > 0) && (firstIndex + size <= src->size[dimension]), 5, "out of range", );
    THGPUTensor_set(self, src);
    if (firstIndex > 0) self->storageOffset += firstIndex * self->stride[dimension];
    self->size[dimension] = size;
}

void THGPUTensor_select(THGPUTensor *self, THGPUTensor *src, int dimension, long sliceIndex) {
    if (!src) src = self;
    THGPU_ARGCHECK(src->nDimension > 1, 1, "cannot select on a vector", );
    THGPU_ARGCHECK((dimension >= 0) && (dimension < src->nDimension), 3, "out of range", );
    THGPU_ARGCHECK((sliceIndex >= 0) && (sliceIndex < src->size[dimension]), 4, "out of range", );
    THGPUTensor_set(self, src);
    THGPUTensor_narrow(self, nullptr, dimension, sliceIndex, 1);
    for (int d = dimension; d < self->nDimension - 1; d++) {
        self->size[d] = self->size[d + 1];
        self->stride[d] = self->stride[d + 1];
    }
    self->nDimension--;
}

void THGPUTensor_transpose(THGPUTensor *self, THGPUTensor *src, int dimension1, int dimension2) {
    if (!src) src = self;
    THGPU_ARGCHECK((dimension1 >= 0) && (dimension1 < src->nDimension), 1, "out of range", );
    THGPU_ARGCHECK((dimension2 >= 0) && (dimension2 < src->nDimension), 2, "out of range", );
    THGPUTensor_set(self, src);
    if (dimension1 == dimension2) return;
    long z = self->stride[dimension1];
    self->stride[dimension1] = self->stride[dimension2];
    self->stride[dimension2] = z;
    z = self->size[dimension1];
    self->size[dimension1] = self->size[dimension2];
    self->size[dimension2] = z;
}

// A new last dimension of length `size` walks along `dimension` with its stride; `dimension`
// itself keeps every `step`-th start (TH/generic/THTensor.c:418-460).
void THGPUTensor_unfold(THGPUTensor *self, THGPUTensor *src, int dimension, long size, long step) {
    if (!src) src = self;
    THGPU_ARGCHECK(src->nDimension > 0, 1, "cannot unfold an empty tensor", );
    THGPU_ARGCHECK(dimension >= 0 && dimension < src->nDimension, 2, "out of range", );
    THGPU_ARGCHECK(size <= src->size[dimension], 3, "out of range", );
    THGPU_ARGCHECK(step > 0, 4, "invalid step", );
    THGPUTensor_set(self, src);
    const int nd = self->nDimension;
    std::vector<long> new_size(nd + 1), new_stride(nd + 1);
    new_size[nd] = size;
    new_stride[nd] = self->stride[dimension];
    for (int d = 0; d < nd; d++) {
        if (d == dimension) {
            new_size[d] = (self->size[d] - size) / step + 1;
            new_stride[d] = step * self->stride[d];
        } else {
            new_size[d] = self->size[d];
            new_stride[d] = self->stride[d];
        }
    }
    self->size = static_cast<long *>(std::realloc(self->size, sizeof(long) * (nd + 1)));
    self->stride = static_cast<long *>(std::realloc(self->stride, sizeof(long) * (nd + 1)));
    for (int d = 0; d <= nd; d++) {
        self->size[d] = new_size[d];
        self->stride[d] = new_stride[d];
    }
    self->nDimension = nd + 1;
}

THGPUTensor *THGPUTensor_newUnfold(THGPUTensor *tensor, int dimension, long size, long step) {
    THGPUTensor *self = THGPUTensor_newWithTensor(tensor);
    THGPUTensor_unfold(self, nullptr, dimension, size, step);
    return self;
}

// Drops the dimensions of length one (all of them: TH/generic/THTensor.c:462-493; one: :495-513).
void THGPUTensor_squeeze(THGPUTensor *self, THGPUTensor *src) {
    if (!src) src = self;
    THGPUTensor_set(self, src);
    int ndim = 0;
    for (int d = 0; d < src->nDimension; d++) {
        if (src->size[d] != 1) {
            if (d != ndim) {
                self->size[ndim] = src->size[d];
                self->stride[ndim] = src->stride[d];
            }
            ndim++;
        }
    }
    if (ndim == 0 && src->nDimension > 0) {  // no 0-dimensional tensors
        self->size[0] = 1;
        self->stride[0] = 1;
        ndim = 1;
    }
    self->nDimension = ndim;
}

void THGPUTensor_squeeze1d(THGPUTensor *self, THGPUTensor *src, int dimension) {
    if (!src) src = self;
    THGPU_ARGCHECK(dimension >= 0 && dimension < src->nDimension, 3, "dimension out of range", );
    THGPUTensor_set(self, src);
    if (src->size[dimension] == 1 && src->nDimension > 1) {
        for (int d = dimension; d < self->nDimension - 1; d++) {
            self->size[d] = self->size[d + 1];
            self->stride[d] = self->stride[d + 1];
        }
        self->nDimension--;
    }
}

int THGPUTensor_isContiguous(const THGPUTensor *self) {
    long z = 1;
    for (int d = self->nDimension - 1; d >= 0; d--) {
        if (self->size[d] != 1) {
            if (self->stride[d] == z)
                z *= self->size[d];
            else
                return 0;
        }
    }
    return 1;
}

int THGPUTensor_isSameSizeAs(const THGPUTensor *self, const THGPUTensor *src) {
    if (self->nDimension != src->nDimension) return 0;
    for (int d = 0; d < self->nDimension; ++d)
        if (self->size[d] != src->size[d]) return 0;
    return 1;
}

long THGPUTensor_nElement(const THGPUTensor *self) {
    if (self->nDimension == 0) return 0;
    long n = 1;
    for (int d = 0; d < self->nDimension; d++) n *= self->size[d];
    return n;
}

void THGPUTensor_retain(THGPUTensor *self) {
    if (self->flag & TH_TENSOR_REFCOUNTED) ++self->refcount;
}

void THGPUTensor_free(THGPUTensor *self) {
    if (!self) return;
    if (self->flag & TH_TENSOR_REFCOUNTED) {
        if (--self->refcount == 0) {
            std::free(self->size);
            std::free(self->stride);
            if (self->storage) THGPUStorage_free(self->storage);
            std::free(self);
        }
    }
}

void THGPUTensor_freeCopyTo(THGPUTensor *self, THGPUTensor *dst) {
    if (self != dst) THGPUTensor_copy(dst, self);
    THGPUTensor_free(self);
}

#define THGPU_GETSET(ND, ARGS, IDX, CHECKS)                                                       \
    void THGPUTensor_set##ND##d(THGPUTensor *tensor, ARGS, float value) {                         \
        THGPU_ARGCHECK(tensor->nDimension == ND, 1, "tensor must have " #ND " dimension(s)", );   \
        long x[] = IDX;                                                                           \
        THGPU_ARGCHECK(CHECKS, 2, "out of range", );                                              \
        THGPUStorage_set(tensor->storage, elem_offset(tensor, ND, x), value);                     \
    }                                                                                             \
    float THGPUTensor_get##ND##d(const THGPUTensor *tensor, ARGS) {                               \
        THGPU_ARGCHECK(tensor->nDimension == ND, 1, "tensor must have " #ND " dimension(s)", 0);  \
        long x[] = IDX;                                                                           \
        THGPU_ARGCHECK(CHECKS, 2, "out of range", 0);                                             \
        return THGPUStorage_get(tensor->storage, elem_offset(tensor, ND, x));                     \
    }
#define THGPU_COMMA ,
#define THGPU_IN(i) ((x##i >= 0) && (x##i < tensor->size[i]))
THGPU_GETSET(1, long x0, {x0}, THGPU_IN(0))
THGPU_GETSET(2, long x0 THGPU_COMMA long x1, {x0 THGPU_COMMA x1}, THGPU_IN(0) && THGPU_IN(1))
THGPU_GETSET(3, long x0 THGPU_COMMA long x1 THGPU_COMMA long x2, {x0 THGPU_COMMA x1 THGPU_COMMA x2},
             THGPU_IN(0) && THGPU_IN(1) && THGPU_IN(2))
THGPU_GETSET(4, long x0 THGPU_COMMA long x1 THGPU_COMMA long x2 THGPU_COMMA long x3,
             {x0 THGPU_COMMA x1 THGPU_COMMA x2 THGPU_COMMA x3},
             THGPU_IN(0) && THGPU_IN(1) && THGPU_IN(2) && THGPU_IN(3))

void THGPUTensor_fill(THGPUTensor *self, float value) {
    long n = THGPUTensor_nElement(self);
    if (n == 0) return;
    if (THGPUTensor_isContiguous(self)) {
        if (fill_device(THGPUTensor_data(self), n, value)) raise("%s", thgpu_last_error());
        return;
    }
    // Non-contiguous view: fill a dense clone and copy it back over the view.
    THGPUTensor *dense = THGPUTensor_new();
    raw_resize(dense, self->nDimension, self->size, nullptr);
    if (fill_device(THGPUTensor_data(dense), n, value)) raise("%s", thgpu_last_error());
    THGPUTensor_freeCopyTo(dense, self);
}

void THGPUTensor_zero(THGPUTensor *self) { THGPUTensor_fill(self, 0.0f); }

void THGPUTensor_copy(THGPUTensor *self, THGPUTensor *src) {
    long n = THGPUTensor_nElement(self);
    THGPU_ARGCHECK(n == THGPUTensor_nElement(src), 2, "sizes do not match", );
    if (n == 0) return;
    if (THGPUTensor_isContiguous(self) && THGPUTensor_isContiguous(src)) {
        if (copy_d2d(THGPUTensor_data(self), THGPUTensor_data(src), n)) raise("%s", thgpu_last_error());
        return;
    }
    // Element i (row-major over each tensor's own shape) of src goes to
    // element i of self; with different shapes the copy walks both index
    // spaces through a common refinement only when the shapes agree, else it
    // densifies the source first.
    THGPUTensor *s = src;
    bool same_shape = THGPUTensor_isSameSizeAs(self, src);
    if (!same_shape) {
        if (!THGPUTensor_isContiguous(src)) {
            s = THGPUTensor_newClone(src);
        }
        if (THGPUTensor_isContiguous(self)) {
            if (copy_d2d(THGPUTensor_data(self), THGPUTensor_data(s), n)) raise("%s", thgpu_last_error());
            if (s != src) THGPUTensor_free(s);
            return;
        }
    }
    if (self->nDimension > THGPU_MAX_DIMS) {
        if (s != src) THGPUTensor_free(s);
        raise("bad argument #1: too many dimensions");
        return;
    }
    StridedDesc d;
    d.nd = self->nDimension;
    long dense = 1;
    for (int k = self->nDimension - 1; k >= 0; --k) {
        d.size[k] = self->size[k];
        d.dst_stride[k] = self->stride[k];
        d.src_stride[k] = same_shape ? s->stride[k] : dense;
        dense *= self->size[k];
    }
    hipStream_t st = stream();
    if (!st) {
        if (s != src) THGPUTensor_free(s);
        raise("%s", thgpu_last_error());
        return;
    }
    long blocks = (n + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    {
        LaunchScope scope("strided_copy", 0.0, 8.0 * n);
        hipLaunchKernelGGL(strided_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, st, THGPUTensor_data(self),
                           THGPUTensor_data(s), d, n);
    }
    if (check_launch("strided_copy")) raise("%s", thgpu_last_error());
    if (s != src) THGPUTensor_free(s);
}

void THGPUTensor_copyGPU(THGPUTensor *self, THGPUTensor *src) { THGPUTensor_copy(self, src); }

// Host -> device: densify on the host if needed, upload into a contiguous
// device tensor, then a device-side strided copy if self is a view
// (THCTensorCopy.cpp:20-36).
#define THGPU_TENSOR_COPY_FROM_HOST(Name)                                                         \
    void THGPUTensor_copy##Name(THGPUTensor *self, TH##Name##Tensor *src) {                       \
        long n = THGPUTensor_nElement(self);                                                      \
        THGPU_ARGCHECK(n == host_nelement(src), 2, "sizes do not match", );                       \
        if (n == 0) return;                                                                       \
        std::vector<float> buf;                                                                   \
        host_gather(src, buf);                                                                    \
        THGPUTensor *selfc = THGPUTensor_newContiguous(self);                                     \
        if (copy_h2d(THGPUTensor_data(selfc), buf.data(), n)) raise("%s", thgpu_last_error());    \
        THGPUTensor_freeCopyTo(selfc, self);                                                      \
    }
THGPU_TENSOR_COPY_FROM_HOST(Byte)
THGPU_TENSOR_COPY_FROM_HOST(Char)
THGPU_TENSOR_COPY_FROM_HOST(Short)
THGPU_TENSOR_COPY_FROM_HOST(Int)
THGPU_TENSOR_COPY_FROM_HOST(Long)
THGPU_TENSOR_COPY_FROM_HOST(Double)

void THGPUTensor_copyFloat(THGPUTensor *self, THFloatTensor *src) {
    long n = THGPUTensor_nElement(self);
    THGPU_ARGCHECK(n == host_nelement(src), 2, "sizes do not match", );
    if (n == 0) return;
    THGPUTensor *selfc = THGPUTensor_newContiguous(self);
    int rc;
    if (host_contiguous(src)) {
        rc = copy_h2d(THGPUTensor_data(selfc), src->storage->data + src->storageOffset, n);
    } else {
        std::vector<float> buf;
        host_gather(src, buf);
        rc = copy_h2d(THGPUTensor_data(selfc), buf.data(), n);
    }
    if (rc) raise("%s", thgpu_last_error());
    THGPUTensor_freeCopyTo(selfc, self);
}

// Device -> host (THCTensorCopy.cpp:64-80).
void THFloatTensor_copyGPU(THFloatTensor *self, THGPUTensor *src) {
    long n = host_nelement(self);
    THGPU_ARGCHECK(n == THGPUTensor_nElement(src), 2, "sizes do not match", );
    if (n == 0) return;
    THGPUTensor *srcc = THGPUTensor_newContiguous(src);
    if (host_contiguous(self)) {
        if (copy_d2h(self->storage->data + self->storageOffset, THGPUTensor_data(srcc), n))
            raise("%s", thgpu_last_error());
    } else {
        std::vector<float> buf((size_t)n);
        if (copy_d2h(buf.data(), THGPUTensor_data(srcc), n)) raise("%s", thgpu_last_error());
        host_scatter<THFloatTensor, float>(self, buf);
    }
    THGPUTensor_free(srcc);
}

#define THGPU_TENSOR_COPY_TO_HOST(Name, ctype)                                                    \
    void TH##Name##Tensor_copyGPU(TH##Name##Tensor *self, THGPUTensor *src) {                     \
        long n = host_nelement(self);                                                             \
        THGPU_ARGCHECK(n == THGPUTensor_nElement(src), 2, "sizes do not match", );                \
        if (n == 0) return;                                                                       \
        THGPUTensor *srcc = THGPUTensor_newContiguous(src);                                       \
        std::vector<float> buf((size_t)n);                                                        \
        if (copy_d2h(buf.data(), THGPUTensor_data(srcc), n)) raise("%s", thgpu_last_error());     \
        host_scatter<TH##Name##Tensor, ctype>(self, buf);                                         \
        THGPUTensor_free(srcc);                                                                   \
    }
THGPU_TENSOR_COPY_TO_HOST(Byte, unsigned char)
THGPU_TENSOR_COPY_TO_HOST(Char, char)
THGPU_TENSOR_COPY_TO_HOST(Short, short)
THGPU_TENSOR_COPY_TO_HOST(Int, int)
THGPU_TENSOR_COPY_TO_HOST(Long, long)
THGPU_TENSOR_COPY_TO_HOST(Double, double)

}  // extern "C"
