// THGPUStorage on hipMalloc memory with hipMemcpyAsync copies on the library
// stream.  Semantics follow gputorch/lib/THC/THCStorage.cpp and
// THCStorageCopy.cpp; the device buffer replaces the array_view that the
// reference kept in allocatorContext.
#include "common.h"
#include "kernels.h"

#include <cstdlib>
#include <cstring>
#include <unordered_map>
#include <vector>

using namespace thgpu;

namespace thgpu {

__global__ void fill_kernel(float *__restrict__ p, long n, float v) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long stride = (long)gridDim.x * blockDim.x;
    // 16-byte stores over the aligned body, scalar head/tail.
    long head = ((16 - ((uintptr_t)p & 15)) & 15) / 4;
    if (head > n) head = n;
    if (i < head) p[i] = v;
    float4 *p4 = reinterpret_cast<float4 *>(p + head);
    long n4 = (n - head) / 4;
    float4 v4 = make_float4(v, v, v, v);
    for (long j = i; j < n4; j += stride) p4[j] = v4;
    long tail = head + n4 * 4;
    if (i < n - tail) p[tail + i] = v;
}

int fill_device(float *p, long n, float v) {
    if (n <= 0) return 0;
    hipStream_t s = stream();
    if (!s) return 1;
    long blocks = (n / 4 + 255) / 256;
    if (blocks < 1) blocks = 1;
    if (blocks > 8192) blocks = 8192;
    {
        LaunchScope scope("fill", 0.0, 4.0 * n);
        hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, s, p, n, v);
    }
    return check_launch("fill");
}

// One launch that fills several buffers (a network's gradient tensors): entry e owns the virtual index range
// [start[e], start[e+1]) of the concatenation.
constexpr int kFillManyMax = 32;
struct FillMany {
    float *p[kFillManyMax];
    long start[kFillManyMax + 1];
    int count;
};

__global__ __launch_bounds__(256) void fill_many_kernel(const FillMany f, float v) {
    const long total = f.start[f.count];
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        int e = 0;
        while (i >= f.start[e + 1]) ++e;  // at most 32 ranges
        f.p[e][i - f.start[e]] = v;
    }
}

// Blocking host<->device copies: stage through the caller's pageable memory
// with hipMemcpyAsync on the library stream, then drain the stream, which is
// what a blocking clEnqueue{Read,Write}Buffer gave the reference's callers
// (gputorch/lib/THC/copyHelpers.cpp:14-85).
int copy_h2d(float *dst, const float *src, long n) {
    if (n <= 0) return 0;
    hipStream_t s = stream();
    if (!s) return 1;
    THGPU_HIP_TRY(hipMemcpyAsync(dst, src, sizeof(float) * (size_t)n, hipMemcpyHostToDevice, s));
    THGPU_HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int copy_d2h(float *dst, const float *src, long n) {
    if (n <= 0) return 0;
    hipStream_t s = stream();
    if (!s) return 1;
    THGPU_HIP_TRY(hipMemcpyAsync(dst, src, sizeof(float) * (size_t)n, hipMemcpyDeviceToHost, s));
    THGPU_HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int copy_d2d(float *dst, const float *src, long n) {
    if (n <= 0 || dst == src) return 0;
    hipStream_t s = stream();
    if (!s) return 1;
    THGPU_HIP_TRY(hipMemcpyAsync(dst, src, sizeof(float) * (size_t)n, hipMemcpyDeviceToDevice, s));
    return 0;
}

}  // namespace thgpu

// ---- device blocks ------------------------------------------------------------------------------------
// A released block goes to a free list keyed by its size and is handed out again to the next request of that
// size, without draining the stream and without hipFree / hipMalloc: everything the library enqueues runs on
// its one in-order stream, so whatever still uses the block was enqueued before its release and whatever the
// next owner enqueues runs after it.  Shapes recur in this workload (the same modules resize the same buffers
// every step), so exact-size reuse hits.  The cache is dropped (after a stream drain) when it holds more than
// kCacheLimit bytes or when hipMalloc fails.
namespace {

constexpr size_t kCacheLimit = size_t(8) << 30;
std::unordered_map<size_t, std::vector<float *>> g_free_blocks;
size_t g_cached_bytes = 0;

void drop_cached_blocks_impl() {
    if (g_free_blocks.empty()) return;
    hipStream_t s = thgpu::stream();
    if (s) (void)hipStreamSynchronize(s);
    for (auto &kv : g_free_blocks)
        for (float *p : kv.second) device_free(p);
    g_free_blocks.clear();
    g_cached_bytes = 0;
}

// hipSuccess and a block of `floats` floats, or the error of the failed hipMalloc (cleared from the runtime's
// sticky state: the failure is reported by the caller, later launch checks must not see it again).
hipError_t acquire_block(long floats, float **out) {
    const size_t bytes = sizeof(float) * (size_t)floats;
    auto it = g_free_blocks.find(bytes);
    if (it != g_free_blocks.end() && !it->second.empty()) {
        *out = it->second.back();
        it->second.pop_back();
        g_cached_bytes -= bytes;
        return hipSuccess;
    }
    hipError_t e = device_malloc(reinterpret_cast<void **>(out), bytes);
    if (e != hipSuccess && !g_free_blocks.empty()) {
        (void)hipGetLastError();
        drop_cached_blocks_impl();
        e = device_malloc(reinterpret_cast<void **>(out), bytes);
    }
    if (e != hipSuccess) (void)hipGetLastError();
    return e;
}

void release_block(float *p, long floats) {
    if (!p) return;
    thgpu::conv_forget_buffer(p);  // whatever was known about its contents ends with this owner
    const size_t bytes = sizeof(float) * (size_t)floats;
    if (floats <= 0 || g_cached_bytes + bytes > kCacheLimit) {
        hipStream_t s = thgpu::stream();
        if (s) (void)hipStreamSynchronize(s);  // work enqueued earlier may still use the buffer
        device_free(p);
        if (g_cached_bytes + bytes > kCacheLimit) drop_cached_blocks_impl();
        return;
    }
    g_free_blocks[bytes].push_back(p);
    g_cached_bytes += bytes;
}

}  // namespace

namespace thgpu {
// For the library's other allocations (the split-reduction workspace, the offset tables): the kept blocks go back to
// the device, so that a hipMalloc that has just failed can be tried once more.  Returns whether anything was freed.
bool drop_cached_blocks() {
    const bool had = !g_free_blocks.empty();
    drop_cached_blocks_impl();
    return had;
}
}  // namespace thgpu

static void release_buffer(THGPUStorage *self) {
    release_block(self->data, self->size);
    self->data = nullptr;
    self->size = 0;
}

extern "C" {

float *THGPUStorage_data(const THGPUStorage *self) { return self->data; }
long THGPUStorage_size(const THGPUStorage *self) { return self->size; }

void THGPUStorage_set(THGPUStorage *self, long index, float value) {
    THGPU_ARGCHECK((index >= 0) && (index < self->size), 2, "index out of bounds", );
    if (copy_h2d(self->data + index, &value, 1)) raise("%s", thgpu_last_error());
}

float THGPUStorage_get(const THGPUStorage *self, long index) {
    float value = 0;
    THGPU_ARGCHECK((index >= 0) && (index < self->size), 2, "index out of bounds", 0.0f);
    if (copy_d2h(&value, self->data + index, 1)) raise("%s", thgpu_last_error());
    return value;
}

THGPUStorage *THGPUStorage_new(void) {
    THGPUStorage *s = static_cast<THGPUStorage *>(std::calloc(1, sizeof(THGPUStorage)));
    if (!s) {
        raise("out of host memory");
        return nullptr;
    }
    s->refcount = 1;
    s->flag = TH_STORAGE_REFCOUNTED | TH_STORAGE_RESIZABLE | TH_STORAGE_FREEMEM;
    return s;
}

THGPUStorage *THGPUStorage_newWithSize(long size) {
    THGPU_ARGCHECK(size >= 0, 2, "invalid size", nullptr);
    THGPUStorage *s = THGPUStorage_new();
    if (!s || size == 0) return s;
    if (!stream()) {
        std::free(s);
        raise("%s", thgpu_last_error());
        return nullptr;
    }
    hipError_t e = acquire_block(size, &s->data);
    if (e != hipSuccess) {
        std::free(s);
        raise("hipMalloc of %ld floats failed: %s", size, hipGetErrorString(e));
        return nullptr;
    }
    s->size = size;
    return s;
}

THGPUStorage *THGPUStorage_newWithSize1(float d0) {
    float v[1] = {d0};
    return THGPUStorage_newWithData(v, 1);
}
THGPUStorage *THGPUStorage_newWithSize2(float d0, float d1) {
    float v[2] = {d0, d1};
    return THGPUStorage_newWithData(v, 2);
}
THGPUStorage *THGPUStorage_newWithSize3(float d0, float d1, float d2) {
    float v[3] = {d0, d1, d2};
    return THGPUStorage_newWithData(v, 3);
}
THGPUStorage *THGPUStorage_newWithSize4(float d0, float d1, float d2, float d3) {
    float v[4] = {d0, d1, d2, d3};
    return THGPUStorage_newWithData(v, 4);
}

THGPUStorage *THGPUStorage_newWithMapping(const char *, long, int) {
    raise("not available yet for THGPUStorage");
    return nullptr;
}

THGPUStorage *THGPUStorage_newWithData(float *data, long size) {
    THGPUStorage *s = THGPUStorage_newWithSize(size);
    if (!s) return nullptr;
    if (size > 0 && copy_h2d(s->data, data, size)) {
        raise("%s", thgpu_last_error());
    }
    return s;
}

void THGPUStorage_setFlag(THGPUStorage *self, const char flag) { self->flag |= flag; }
void THGPUStorage_clearFlag(THGPUStorage *self, const char flag) { self->flag &= ~flag; }

void THGPUStorage_retain(THGPUStorage *self) {
    if (self && (self->flag & TH_STORAGE_REFCOUNTED)) ++self->refcount;
}

void THGPUStorage_free(THGPUStorage *self) {
    if (!self || !(self->flag & TH_STORAGE_REFCOUNTED)) return;
    if (--(self->refcount) <= 0) {
        if (self->flag & TH_STORAGE_FREEMEM) release_buffer(self);
        std::free(self);
    }
}

void THGPUStorage_fill(THGPUStorage *self, float value) {
    if (fill_device(self->data, self->size, value)) raise("%s", thgpu_last_error());
}

void THGPUStorage_resize(THGPUStorage *self, long size) {
    THGPU_ARGCHECK(size >= 0, 2, "invalid size", );
    if (!(self->flag & TH_STORAGE_RESIZABLE)) return;
    if (size == 0) {
        if (self->flag & TH_STORAGE_FREEMEM) release_buffer(self);
        self->data = nullptr;
        self->size = 0;
        return;
    }
    if (self->size == size) return;
    float *fresh = nullptr;
    if (!stream()) {
        raise("%s", thgpu_last_error());
        return;
    }
    hipError_t e = acquire_block(size, &fresh);
    if (e != hipSuccess) {
        raise("hipMalloc of %ld floats failed: %s", size, hipGetErrorString(e));
        return;
    }
    // The first min(old,new) elements survive a resize (THCStorage.cpp:188-189).
    if (self->data) {
        long keep = self->size < size ? self->size : size;
        if (copy_d2d(fresh, self->data, keep)) raise("%s", thgpu_last_error());
        release_buffer(self);
    }
    self->data = fresh;
    self->size = size;
}

void THGPUStorage_rawCopy(THGPUStorage *self, float *src) {
    if (copy_d2d(self->data, src, self->size)) raise("%s", thgpu_last_error());
}

void THGPUStorage_copy(THGPUStorage *self, THGPUStorage *src) {
    THGPU_ARGCHECK(self->size == src->size, 2, "size does not match", );
    if (copy_d2d(self->data, src->data, self->size)) raise("%s", thgpu_last_error());
}

void THGPUStorage_copyGPU(THGPUStorage *self, THGPUStorage *src) { THGPUStorage_copy(self, src); }

void THGPUStorage_copyFloat(THGPUStorage *self, struct THFloatStorage *src) {
    THGPU_ARGCHECK(self->size == src->size, 2, "size does not match", );
    if (copy_h2d(self->data, src->data, self->size)) raise("%s", thgpu_last_error());
}

void THFloatStorage_copyGPU(THFloatStorage *self, struct THGPUStorage *src) {
    THGPU_ARGCHECK(self->size == src->size, 2, "size does not match", );
    if (copy_d2h(self->data, src->data, self->size)) raise("%s", thgpu_last_error());
}

// Other element types convert through a host float buffer, as the reference
// does (THCStorageCopy.cpp:12-29, 37-54).
#define THGPU_STORAGE_COPY_VIA_FLOAT(Name, ctype)                                             \
    void THGPUStorage_copy##Name(THGPUStorage *self, struct TH##Name##Storage *src) {         \
        THGPU_ARGCHECK(self->size == src->size, 2, "size does not match", );                  \
        std::vector<float> buf((size_t)src->size);                                            \
        for (long i = 0; i < src->size; i++) buf[(size_t)i] = (float)src->data[i];            \
        if (copy_h2d(self->data, buf.data(), self->size)) raise("%s", thgpu_last_error());    \
    }                                                                                         \
    void TH##Name##Storage_copyGPU(TH##Name##Storage *self, struct THGPUStorage *src) {       \
        THGPU_ARGCHECK(self->size == src->size, 2, "size does not match", );                  \
        std::vector<float> buf((size_t)src->size);                                            \
        if (copy_d2h(buf.data(), src->data, src->size)) {                                     \
            raise("%s", thgpu_last_error());                                                  \
            return;                                                                           \
        }                                                                                     \
        for (long i = 0; i < src->size; i++) self->data[i] = (ctype)buf[(size_t)i];           \
    }
THGPU_STORAGE_COPY_VIA_FLOAT(Byte, unsigned char)
THGPU_STORAGE_COPY_VIA_FLOAT(Char, char)
THGPU_STORAGE_COPY_VIA_FLOAT(Short, short)
THGPU_STORAGE_COPY_VIA_FLOAT(Int, int)
THGPU_STORAGE_COPY_VIA_FLOAT(Long, long)
THGPU_STORAGE_COPY_VIA_FLOAT(Double, double)

int thgpu_empty_cache(void) {
    drop_cached_blocks();
    return 0;
}

long thgpu_cached_bytes(void) { return (long)g_cached_bytes; }

int thgpu_memcpy_h2d(float *dst_device, const float *src_host, long n) {
    if (n < 0) return fail("thgpu_memcpy_h2d: negative count");
    if (n == 0) return 0;
    if (!dst_device || !src_host) return fail("thgpu_memcpy_h2d: null pointer");
    return copy_h2d(dst_device, src_host, n);
}

int thgpu_memcpy_d2h(float *dst_host, const float *src_device, long n) {
    if (n < 0) return fail("thgpu_memcpy_d2h: negative count");
    if (n == 0) return 0;
    if (!dst_host || !src_device) return fail("thgpu_memcpy_d2h: null pointer");
    return copy_d2h(dst_host, src_device, n);
}

}  // extern "C"

extern "C" int thgpu_fill_many(THGPUTensor **tensors, int count, float value) {
    if (count < 0 || (count > 0 && !tensors)) return fail("thgpu_fill_many: invalid arguments");
    hipStream_t s = stream();
    if (!s) return 1;
    for (int i = 0; i < count; ++i) {  // every tensor is checked before anything is launched
        THGPUTensor *t = tensors[i];
        if (!t) return fail("thgpu_fill_many: null tensor");
        if (THGPUTensor_nElement(t) > 0 && (!THGPUTensor_isContiguous(t) || !tensor_backed(t)))
            return fail("thgpu_fill_many: tensor %d is not contiguous or exceeds its storage", i);
    }
    for (int first = 0; first < count; first += kFillManyMax) {
        FillMany f;
        f.count = 0;
        f.start[0] = 0;
        for (int i = first; i < count && i < first + kFillManyMax; ++i) {
            const long n = THGPUTensor_nElement(tensors[i]);
            if (n == 0) continue;
            f.p[f.count] = THGPUTensor_data(tensors[i]);
            f.start[f.count + 1] = f.start[f.count] + n;
            ++f.count;
        }
        const long total = f.start[f.count];
        if (total == 0) continue;
        long blocks = (total + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        {
            LaunchScope scope("fill", 0.0, 4.0 * total);
            hipLaunchKernelGGL(fill_many_kernel, dim3((unsigned)blocks), dim3(256), 0, s, f, value);
        }
        if (check_launch("fill")) return 1;
    }
    return 0;
}
