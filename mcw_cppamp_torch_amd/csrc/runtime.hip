// Runtime plumbing of libthgpu: error reporting, the library stream, the
// split-reduction workspace, event timing and per-kernel profiling.
#include "common.h"
#include "kernels.h"

#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace thgpu {

static char g_last_error[1024] = "";

static void default_handler(const char *msg, void *) {
    // TH's default handlers print and exit (TH/THGeneral.c:7-11,40-47).
    std::fprintf(stderr, "$ Error: %s\n", msg);
    std::exit(-1);
}
static THGPUErrorHandler g_handler = default_handler;
static void *g_handler_data = nullptr;

int fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return 1;
}

void raise(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    g_handler(g_last_error, g_handler_data);
}

// ---- tuning switches -----------------------------------------------------------
static Tuning g_tuning;
static bool g_tuning_read = false;

static int tuning_set(const char *name, const char *value) {
    const char *v = value ? value : "";
    if (!std::strcmp(name, "gemm_tile")) {
        std::snprintf(g_tuning.gemm_tile, sizeof(g_tuning.gemm_tile), "%s", v);
    } else if (!std::strcmp(name, "gemm_split")) {
        g_tuning.gemm_split = std::atoi(v);
    } else if (!std::strcmp(name, "im2col_kernel")) {
        std::snprintf(g_tuning.im2col_kernel, sizeof(g_tuning.im2col_kernel), "%s", v);
    } else if (!std::strcmp(name, "im2col_plan")) {
        g_tuning.im2col_plan[0] = g_tuning.im2col_plan[1] = g_tuning.im2col_plan[2] = 0;
        std::sscanf(v, "%d,%d,%d", &g_tuning.im2col_plan[0], &g_tuning.im2col_plan[1], &g_tuning.im2col_plan[2]);
    } else if (!std::strcmp(name, "col2im_generic")) {
        g_tuning.col2im_generic = v[0] == '1';
    } else if (!std::strcmp(name, "pool_fwd_wave")) {
        g_tuning.pool_fwd_wave = v[0] == '1';
    } else if (!std::strcmp(name, "pool_bwd_direct")) {
        g_tuning.pool_bwd_direct = v[0] == '1';
    } else if (!std::strcmp(name, "pool_bwd_tile")) {
        g_tuning.pool_bwd_tile = v[0] == '1';
    } else if (!std::strcmp(name, "pool_bwd_cell")) {
        g_tuning.pool_bwd_cell = v[0] == '1';
    } else if (!std::strcmp(name, "pool_bwd_pixels")) {
        g_tuning.pool_bwd_pixels = std::atoi(v);
    } else if (!std::strcmp(name, "gradbias_separate")) {
        g_tuning.gradbias_separate = v[0] == '1';
    } else if (!std::strcmp(name, "conv_narrow_off")) {
        g_tuning.conv_narrow_off = v[0] == '1';
    } else {
        return fail("thgpu_debug_set: unknown switch '%s'", name);
    }
    return 0;
}

const Tuning &tuning() {
    if (!g_tuning_read) {
        g_tuning_read = true;
        static const char *const kEnv[][2] = {
            {"THGPU_GEMM_TILE", "gemm_tile"},           {"THGPU_GEMM_SPLIT", "gemm_split"},
            {"THGPU_IM2COL_KERNEL", "im2col_kernel"},   {"THGPU_IM2COL_PLAN", "im2col_plan"},
            {"THGPU_COL2IM_GENERIC", "col2im_generic"}, {"THGPU_POOL_FWD_WAVE", "pool_fwd_wave"},
            {"THGPU_POOL_BWD_DIRECT", "pool_bwd_direct"}, {"THGPU_GRADBIAS_SEPARATE", "gradbias_separate"},
            {"THGPU_POOL_BWD_TILE", "pool_bwd_tile"}, {"THGPU_POOL_BWD_CELL", "pool_bwd_cell"},
            {"THGPU_POOL_BWD_PIXELS", "pool_bwd_pixels"}, {"THGPU_CONV_NARROW_OFF", "conv_narrow_off"}};
        for (auto &e : kEnv)
            if (const char *v = std::getenv(e[0])) (void)tuning_set(e[1], v);
    }
    return g_tuning;
}

// ---- the array behind the entry points that must not allocate --------------------
// Device memory the library holds from the moment its code object is loaded until the process
// ends (64 MiB on every GPU the process uses).  `scratch` is only a host-side handle of the
// symbol: the device address comes from hipGetSymbolAddress at initialisation and is the only
// thing ever passed to a kernel.
constexpr size_t kStaticScratchFloats = (size_t)THGPU_GEMM_NOALLOC_MAX_ELEMENTS;
static __device__ __align__(256) float scratch[kStaticScratchFloats];
static float *g_scratch_ptr = nullptr;  // device address of scratch[] on device 0, the one device the library runs on

// ---- stream / device ----------------------------------------------------------
static hipStream_t g_stream = nullptr;
static bool g_init_done = false, g_init_ok = false;
static int g_cus = 0;

static int init_once() {
    if (g_init_done) return g_init_ok ? 0 : 1;
    g_init_done = true;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n < 1)
        return fail("no HIP device available (%s)", e == hipSuccess ? "device count 0" : hipGetErrorString(e));
    THGPU_HIP_TRY(hipSetDevice(0));
    hipDeviceProp_t prop;
    THGPU_HIP_TRY(hipGetDeviceProperties(&prop, 0));
    g_cus = prop.multiProcessorCount;
    // Default priority; non-blocking with respect to the legacy null stream.
    THGPU_HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    // Device 0 is current: resolve where this device keeps its copy of scratch[].
    void *sp = nullptr;
    THGPU_HIP_TRY(hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)));
    g_scratch_ptr = static_cast<float *>(sp);
    (void)tuning();
    g_init_ok = true;
    return 0;
}

float *static_scratch(size_t *floats) {
    if (floats) *floats = kStaticScratchFloats;
    return g_init_ok ? g_scratch_ptr : nullptr;
}

hipStream_t stream() {
    if (init_once() != 0) return nullptr;
    return g_stream;
}

int num_cus() {
    init_once();
    return g_cus > 0 ? g_cus : 256;
}

static long g_alloc_calls = 0;

hipError_t device_malloc(void **p, size_t bytes) {
    ++g_alloc_calls;
    return hipMalloc(p, bytes);
}

void device_free(void *p) {
    ++g_alloc_calls;
    (void)hipFree(p);
}

static float *g_ws = nullptr;
static size_t g_ws_bytes = 0;

float *workspace(size_t bytes) {
    if (bytes <= g_ws_bytes) return g_ws;
    if (!stream()) return nullptr;
    if (g_ws) {
        // Kernels still in flight may read the old buffer.
        if (hipStreamSynchronize(g_stream) != hipSuccess) return nullptr;
        device_free(g_ws);
        g_ws = nullptr;
        g_ws_bytes = 0;
    }
    size_t want = bytes + bytes / 4;
    hipError_t e = device_malloc(reinterpret_cast<void **>(&g_ws), want);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        // freed storage buffers may be sitting in the block cache: give them back and try once more
        if (drop_cached_blocks()) e = device_malloc(reinterpret_cast<void **>(&g_ws), want);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();  // or the next launch check would report this failure as its own
        fail("workspace allocation of %zu bytes failed: %s", want, hipGetErrorString(e));
        g_ws = nullptr;
        return nullptr;
    }
    g_ws_bytes = want;
    return g_ws;
}

int check_launch(const char *name) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("launch of %s failed: %s", name, hipGetErrorString(e));
    return 0;
}

// ---- events -------------------------------------------------------------------
static std::vector<hipEvent_t> g_events;

// ---- per-kernel profiling -------------------------------------------------------
struct ProfRecord {
    const char *name;
    hipEvent_t start, stop;
    double flops, bytes;
};
static bool g_prof_on = false;
static std::vector<ProfRecord> g_prof;
static std::vector<hipEvent_t> g_prof_pool;

static hipEvent_t pool_event() {
    if (!g_prof_pool.empty()) {
        hipEvent_t e = g_prof_pool.back();
        g_prof_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

bool prof_enabled() { return g_prof_on; }

const char *prof_label(const char *fmt, ...) {
    static std::set<std::string> labels;  // node addresses stay valid: the returned pointer lives as long as the process
    char buf[256];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    return labels.insert(buf).first->c_str();
}

LaunchScope::LaunchScope(const char *name, double flops, double bytes) : slot(-1) {
    if (!g_prof_on || !stream()) return;
    ProfRecord r{name, pool_event(), pool_event(), flops, bytes};
    if (!r.start || !r.stop) return;
    (void)hipEventRecord(r.start, g_stream);
    slot = static_cast<int>(g_prof.size());
    g_prof.push_back(r);
}

LaunchScope::~LaunchScope() {
    if (slot >= 0) (void)hipEventRecord(g_prof[slot].stop, g_stream);
}

}  // namespace thgpu

using namespace thgpu;

extern "C" {

void THGPUSetErrorHandler(THGPUErrorHandler handler, void *data) {
    g_handler = handler ? handler : default_handler;
    g_handler_data = data;
}

const char *thgpu_last_error(void) { return g_last_error; }

int thgpu_init(void) { return init_once(); }

int thgpu_debug_set(const char *name, const char *value) {
    if (!name) return fail("thgpu_debug_set: null name");
    (void)tuning();  // the environment is read first, so that it never overrides a later call
    return tuning_set(name, value);
}

int thgpu_synchronize(void) {
    if (!stream()) return 1;
    THGPU_HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

int thgpu_device_info(char *name, long name_cap, int *compute_units, long *total_mem_bytes) {
    if (!stream()) return 1;
    hipDeviceProp_t prop;
    THGPU_HIP_TRY(hipGetDeviceProperties(&prop, 0));
    if (name && name_cap > 0) {
        std::snprintf(name, static_cast<size_t>(name_cap), "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem_bytes) *total_mem_bytes = static_cast<long>(prop.totalGlobalMem);
    return 0;
}

int thgpu_event_create(void) {
    if (!stream()) return -1;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) {
        fail("hipEventCreate failed");
        return -1;
    }
    g_events.push_back(e);
    return static_cast<int>(g_events.size()) - 1;
}

int thgpu_event_record(int ev) {
    if (!stream()) return 1;
    if (ev < 0 || ev >= static_cast<int>(g_events.size())) return fail("bad event handle %d", ev);
    THGPU_HIP_TRY(hipEventRecord(g_events[ev], g_stream));
    return 0;
}

int thgpu_event_elapsed_ms(int ev_start, int ev_stop, float *ms) {
    int n = static_cast<int>(g_events.size());
    if (ev_start < 0 || ev_start >= n || ev_stop < 0 || ev_stop >= n || !ms)
        return fail("bad event handle (%d, %d)", ev_start, ev_stop);
    THGPU_HIP_TRY(hipEventSynchronize(g_events[ev_stop]));
    THGPU_HIP_TRY(hipEventElapsedTime(ms, g_events[ev_start], g_events[ev_stop]));
    return 0;
}

long thgpu_selftest_index_math(void) {
    long bad = 0;
    const uint32_t divisors[] = {1, 2, 3, 4, 5, 6, 7, 9, 11, 12, 13, 16, 25, 27, 36, 49, 55, 63, 75, 121, 144,
                                 169, 196, 363, 576, 729, 784, 825, 1600, 3025, 3136, 12544, 50176, 65535, 65536,
                                 1000003, 16777216, 2147483647u};
    for (uint32_t d : divisors) {
        FastDiv f(d);
        auto probe = [&](uint32_t n) {
            uint32_t q, r;
            f.divmod(n, q, r);
            if (q != n / d || r != n % d) ++bad;
        };
        for (uint32_t n = 0; n < 5000; ++n) probe(n);
        for (uint64_t n = 1; n < (1ull << 32); n = n * 3 + 1) {
            probe((uint32_t)n);
            probe((uint32_t)n - 1);
        }
        for (uint32_t k = 1; k < 4000; ++k) {
            uint64_t m = (uint64_t)k * d;
            if (m < (1ull << 32)) {
                probe((uint32_t)m);
                probe((uint32_t)m - 1);
            }
        }
        probe(0x7fffffffu);
        probe(0xffffffffu);
    }
    return bad;
}

long thgpu_device_alloc_calls(void) { return g_alloc_calls; }

long thgpu_selftest_launch_plans(void) { return im2col_plan_selftest() + pool_plan_selftest(); }

int thgpu_prof_enable(int on) {
    g_prof_on = on != 0;
    return 0;
}

int thgpu_prof_reset(void) {
    if (g_stream) (void)hipStreamSynchronize(g_stream);
    for (auto &r : g_prof) {
        g_prof_pool.push_back(r.start);
        g_prof_pool.push_back(r.stop);
    }
    g_prof.clear();
    return 0;
}

long thgpu_prof_report(char *buf, long cap) {
    struct Agg {
        long calls = 0;
        double ms = 0, flops = 0, bytes = 0;
    };
    std::map<std::string, Agg> agg;
    if (g_stream) (void)hipStreamSynchronize(g_stream);
    for (auto &r : g_prof) {
        float ms = 0;
        if (hipEventElapsedTime(&ms, r.start, r.stop) != hipSuccess) continue;
        Agg &a = agg[r.name];
        a.calls += 1;
        a.ms += ms;
        a.flops += r.flops;
        a.bytes += r.bytes;
    }
    std::string out = "{";
    bool first = true;
    for (auto &kv : agg) {
        char line[512];
        std::snprintf(line, sizeof(line), "%s\"%s\": {\"calls\": %ld, \"ms\": %.6f, \"flops\": %.1f, \"bytes\": %.1f}",
                      first ? "" : ", ", kv.first.c_str(), kv.second.calls, kv.second.ms, kv.second.flops,
                      kv.second.bytes);
        out += line;
        first = false;
    }
    out += "}";
    if (buf && cap > 0) {
        std::strncpy(buf, out.c_str(), static_cast<size_t>(cap) - 1);
        buf[cap - 1] = 0;
    }
    return static_cast<long>(out.size()) + 1;
}

}  // extern "C"
