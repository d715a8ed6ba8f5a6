// Internal helpers shared by the libthgpu sources: error plumbing, the library
// stream, launch bracketing for per-kernel timing, magic-number division.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/thgpu.h"

namespace thgpu {

// ---- errors -----------------------------------------------------------------
// Records a message for thgpu_last_error(); returns a non-zero status so that
// `return fail(...)` reads naturally in the flat entry points.
int fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
// Records the message and calls the installed TH-style handler.
void raise(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define THGPU_HIP_TRY(expr)                                                                       \
    do {                                                                                          \
        hipError_t _e = (expr);                                                                   \
        if (_e != hipSuccess)                                                                     \
            return ::thgpu::fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, \
                                 __LINE__);                                                       \
    } while (0)

// For TH-named functions (void or value returning): raise through the handler
// and return `ret` if the handler comes back.
#define THGPU_ARGCHECK(cond, argn, msg, ret)                         \
    do {                                                             \
        if (!(cond)) {                                               \
            ::thgpu::raise("bad argument #%d: %s", (argn), (msg));   \
            return ret;                                              \
        }                                                            \
    } while (0)

#define THGPU_HIP_CHECK_RAISE(expr, ret)                                                           \
    do {                                                                                           \
        hipError_t _e = (expr);                                                                    \
        if (_e != hipSuccess) {                                                                    \
            ::thgpu::raise("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return ret;                                                                            \
        }                                                                                          \
    } while (0)

// ---- runtime ----------------------------------------------------------------
// Library stream (created on first use).  nullptr means initialisation failed
// and the error is recorded.
hipStream_t stream();
// Grow-only device scratch for split reductions; stream-ordered with the
// kernels that use it because everything runs on the one library stream.
float *workspace(size_t bytes);
int num_cus();
// Returns the storage block cache's kept buffers to the device (draining the stream first); true when there were
// any.  Every hipMalloc of the library that fails calls this and tries once more (storage.hip).
bool drop_cached_blocks();
// hipMalloc / hipFree as the library calls them: counted, so that a test can show that an entry point made neither
// (thgpu_device_alloc_calls).
hipError_t device_malloc(void **p, size_t bytes);
void device_free(void *p);
// The fixed device array behind the entry points that must not allocate (runtime.hip): its device
// address and size in floats once the library is initialised, nullptr before (never initialises).
float *static_scratch(size_t *floats);

// Testing and tuning switches.  Filled from the environment once, when the library initialises
// (THGPU_GEMM_TILE, THGPU_GEMM_SPLIT, THGPU_IM2COL_KERNEL, THGPU_IM2COL_PLAN, THGPU_COL2IM_GENERIC,
// THGPU_POOL_FWD_WAVE, THGPU_POOL_BWD_DIRECT, THGPU_POOL_BWD_TILE, THGPU_POOL_BWD_CELL, THGPU_CONV_NARROW_OFF), and changed afterwards only through thgpu_debug_set: no launch reads the
// environment.
struct Tuning {
    char gemm_tile[16] = "";      // a tile configuration by name; "" leaves the choice to the cost model
    int gemm_split = 0;           // reduction split count; 0 leaves it to the cost model
    char im2col_kernel[16] = "";  // unit | strip | direct
    int im2col_plan[3] = {0, 0, 0};  // strip shape "v,PL,TG"
    bool col2im_generic = false;
    bool pool_fwd_wave = false;   // the wavefront-level tile kernel instead of the direct forward kernel
    bool pool_bwd_direct = false; // the one-lane-per-pixel backward kernel
    bool pool_bwd_tile = false;   // the LDS tile backward kernel where the staged kernel would run
    bool pool_bwd_cell = false;   // the cell backward kernel (no LDS) where the staged kernel would run
    int pool_bwd_pixels = 0;      // pixels a workgroup of the staged backward kernel takes; 0 leaves it to the planner
    bool gradbias_separate = false;  // the two-stage bias-gradient sum even where the gradWeight product could do it
    bool conv_narrow_off = false;    // the tiled GEMM kernels where the kernels for layers with a handful of taps would run
};
const Tuning &tuning();

// Brackets one kernel launch with events when per-kernel timing is enabled.
struct LaunchScope {
    LaunchScope(const char *name, double flops, double bytes);
    ~LaunchScope();
    int slot;
};

// Per-kernel timing on?  And a label for one record that is formatted only then (interned; the
// report groups records by label), so that e.g. every GEMM shape of a network is listed on its own.
bool prof_enabled();
const char *prof_label(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// Checks the launch itself (bad configuration shows up here, not at sync).
int check_launch(const char *name);

// ---- raw device helpers (storage.hip) -----------------------------------------
int fill_device(float *p, long n, float v);           // async on the library stream
int copy_h2d(float *dst, const float *src, long n);   // blocking
int copy_d2h(float *dst, const float *src, long n);   // blocking
int copy_d2d(float *dst, const float *src, long n);   // async on the library stream

// ---- tensors as kernel operands -------------------------------------------------
// Whether every element the tensor's shape addresses lies inside its storage: the check an operator
// makes on each tensor it has resized, and on the caller's, before any kernel is given its pointer.
inline bool tensor_backed(const THGPUTensor *t) {
    if (!t) return false;
    long extent = t->nDimension > 0 ? 1 : 0;
    for (int d = 0; d < t->nDimension; ++d) {
        if (t->size[d] <= 0) return true;  // no elements: nothing to back
        if (t->stride[d] < 0) return false;
        extent += (t->size[d] - 1) * t->stride[d];
    }
    if (extent == 0) return true;
    return t->storage && t->storage->data && t->storageOffset >= 0 &&
           t->storageOffset + extent <= t->storage->size;
}
// A dense tensor of exactly n elements with memory behind all of them.
inline bool tensor_ready(const THGPUTensor *t, long n) {
    return t && THGPUTensor_isContiguous(t) && THGPUTensor_nElement(t) == n && tensor_backed(t);
}

// ---- unsigned division by a run-time constant ---------------------------------
// q = n / d for 0 <= n < 2^31, 1 <= d < 2^31 via one mul-hi and a shift.
struct FastDiv {
    uint32_t d, mul, shr;
    FastDiv() : d(1), mul(0), shr(0) {}
    explicit FastDiv(uint32_t div) : d(div) {
        if (div == 1) { mul = 0; shr = 0; return; }
        uint32_t l = 0;
        while ((1ull << l) < div) ++l;                      // ceil(log2 d), >= 1 here
        // Round-up method: the 33-bit multiplier ceil(2^(32+l)/d) lies in
        // [2^32, 2^33); its low 32 bits are kept and the implicit top bit is
        // folded into the (n - t)/2 + t step of div().
        uint64_t mm = ((1ull << (32 + l)) + div - 1) / div;
        mul = (uint32_t)(mm - (1ull << 32));
        shr = l;
    }
    __host__ __device__ inline uint32_t div(uint32_t n) const {
        if (d == 1) return n;
#if defined(__HIP_DEVICE_COMPILE__)
        uint32_t t = __umulhi(n, mul);
#else
        uint32_t t = (uint32_t)(((uint64_t)n * mul) >> 32);
#endif
        // (n + t) may overflow 32 bits: use the standard overflow-free form
        return (((n - t) >> 1) + t) >> (shr - 1);
    }
    __host__ __device__ inline void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
        q = div(n);
        r = n - q * d;
    }
};

}  // namespace thgpu
