/*
 * thgpu.h -- C ABI of libthgpu, the MI355X (gfx950) implementation of the
 * gputorch/gpunn convolution hot path: THGPUStorage / THGPUTensor on hipMalloc
 * memory, THGPUBlas_gemm on fp32 MFMA, batched im2col / col2im,
 * nn.SpatialConvolutionMM, nn.SpatialMaxPooling and nn.Threshold forward and
 * backward.
 *
 * Plain C: pointers, sizes and the two TH structs whose layout LuaJIT FFI code
 * reads directly (gputorch/FFI.lua:5-29).  Every declaration cites the
 * reference interface it replaces (paths relative to the reference tree).
 *
 * Conventions
 *  - `data` of a THGPUStorage is a DEVICE pointer (hipMalloc); `allocator` and
 *    `allocatorContext` are unused and NULL.
 *  - All device work is enqueued on one library-owned HIP stream.  Functions
 *    that hand data to the host (get, copies to host, thgpu_synchronize)
 *    block until the stream has drained; everything else returns as soon as
 *    the work is enqueued.  Not thread-safe, like the reference.
 *  - TH-named functions return void/values as in the reference and report
 *    errors through the installable handler (THGPUSetErrorHandler), which
 *    mirrors THSetErrorHandler / THSetArgErrorHandler (TH/THGeneral.c:7-65).
 *    thgpu_* functions return 0 on success or a non-zero status and leave a
 *    message in thgpu_last_error(); they never call the handler.
 */
#ifndef THGPU_H
#define THGPU_H

#ifdef __cplusplus
extern "C" {
#endif

/* ---- struct layouts (ABI) ------------------------------------------------ */

typedef struct THAllocator THAllocator; /* opaque, never dereferenced here */

#define TH_STORAGE_REFCOUNTED 1 /* TH/generic/THStorage.h:19-21 */
#define TH_STORAGE_RESIZABLE 2
#define TH_STORAGE_FREEMEM 4
#define TH_TENSOR_REFCOUNTED 1 /* gputorch/lib/THC/THCTensor.h:16 */

/* TH/generic/THStorage.h:23-31 instantiated with real=float, Real=GPU by
 * gputorch/lib/THC/THCStorage.h:10-20; FFI view gputorch/FFI.lua:6-14. */
typedef struct THGPUStorage {
    float *data; /* device pointer */
    long size;
    int refcount;
    char flag;
    THAllocator *allocator;
    void *allocatorContext;
} THGPUStorage;

/* gputorch/lib/THC/THCTensor.h:18-50 (data members only); FFI view
 * gputorch/FFI.lua:16-28. */
typedef struct THGPUTensor {
    long *size;
    long *stride;
    int nDimension;
    THGPUStorage *storage;
    long storageOffset;
    int refcount;
    char flag;
} THGPUTensor;

/* Host-side TH types that appear in the copy signatures.  Same layouts
 * (TH/generic/THStorage.h:23-31, TH/generic/THTensor.h), host pointers.  A translation unit that has included
 * Torch's own TH.h (the luaT bindings do) already has them and skips these declarations. */
#ifndef TH_INC
#define THGPU_DECLARE_HOST_TYPES(Name, ctype)                                              \
    typedef struct TH##Name##Storage {                                                     \
        ctype *data;                                                                       \
        long size;                                                                         \
        int refcount;                                                                      \
        char flag;                                                                         \
        THAllocator *allocator;                                                            \
        void *allocatorContext;                                                            \
    } TH##Name##Storage;                                                                   \
    typedef struct TH##Name##Tensor {                                                      \
        long *size;                                                                        \
        long *stride;                                                                      \
        int nDimension;                                                                    \
        TH##Name##Storage *storage;                                                        \
        long storageOffset;                                                                \
        int refcount;                                                                      \
        char flag;                                                                         \
    } TH##Name##Tensor;
THGPU_DECLARE_HOST_TYPES(Byte, unsigned char)
THGPU_DECLARE_HOST_TYPES(Char, char)
THGPU_DECLARE_HOST_TYPES(Short, short)
THGPU_DECLARE_HOST_TYPES(Int, int)
THGPU_DECLARE_HOST_TYPES(Long, long)
THGPU_DECLARE_HOST_TYPES(Float, float)
THGPU_DECLARE_HOST_TYPES(Double, double)
#endif /* TH_INC */

/* ---- runtime --------------------------------------------------------------- */

/* Error handler, replacing THSetErrorHandler/THSetArgErrorHandler
 * (TH/THGeneral.c:16-65) and __THGPUCheck (gputorch/lib/THC/THCGeneral.cpp:
 * 17-24).  The default handler prints the message and exits, as TH's default
 * does (TH/THGeneral.c:7-11,40-47).  A handler that returns makes the failing
 * TH-named function return early without touching its arguments. */
typedef void (*THGPUErrorHandler)(const char *msg, void *data);
void THGPUSetErrorHandler(THGPUErrorHandler handler, void *data);

/* Message of the most recent failure (empty string if none). */
const char *thgpu_last_error(void);

/* Selects device 0, creates the library stream.  Called lazily by everything
 * else; explicit call returns non-zero if no usable GPU is present. */
int thgpu_init(void);

/* Testing and tuning switches (no counterpart in the reference).  name: gemm_tile (a tile configuration such
 * as "128x128"), gemm_split (a reduction split count), im2col_kernel (unit | strip | direct), im2col_plan
 * ("v,PL,TG"), col2im_generic ("1"), pool_fwd_wave ("1"), pool_bwd_direct ("1"), pool_bwd_tile ("1"),
 * pool_bwd_cell ("1"), pool_bwd_pixels (pixels per workgroup of the staged max-pool backward kernel, which it also
 * pins), gradbias_separate ("1"), conv_narrow_off ("1": the tiled GEMM kernels where the kernels for layers with at
 * most 32 taps would run); value NULL or "" restores the library's own choice.  The environment variables
 * THGPU_GEMM_TILE, THGPU_GEMM_SPLIT, THGPU_IM2COL_KERNEL, THGPU_IM2COL_PLAN, THGPU_COL2IM_GENERIC,
 * THGPU_POOL_FWD_WAVE, THGPU_POOL_BWD_DIRECT, THGPU_POOL_BWD_TILE, THGPU_POOL_BWD_CELL, THGPU_POOL_BWD_PIXELS,
 * THGPU_GRADBIAS_SEPARATE and THGPU_CONV_NARROW_OFF give the initial values and are read once, when the library
 * initialises; no operator call reads the environment. */
int thgpu_debug_set(const char *name, const char *value);

/* Real stream synchronisation, replacing the no-op gputorch.synchronize
 * (gputorch/init.cpp:10-14). */
int thgpu_synchronize(void);
/* Storage buffers that are released (free, resize) are kept and handed out again to the next request of the
 * same size instead of going through hipFree / hipMalloc and a stream drain (everything runs on the library's
 * one in-order stream, so reuse is ordered).  thgpu_empty_cache returns the kept blocks to the device (it
 * drains the stream first); thgpu_cached_bytes says how much is kept.  The cache empties itself above 8 GiB
 * and when an allocation fails.  No counterpart in the reference, whose array_views freed eagerly. */
int thgpu_empty_cache(void);
long thgpu_cached_bytes(void);
/* How many times the library has called hipMalloc or hipFree since it was loaded (storage blocks, the split-reduction
 * workspace, the offset tables of the gathered convolutions: every allocation it makes).  A caller that must not
 * allocate can verify an entry point against it; no counterpart in the reference. */
long thgpu_device_alloc_calls(void);

/* Device name / compute-unit count / total memory, replacing the stubbed
 * getDeviceProperties (gputorch/init.cpp:40-66). */
int thgpu_device_info(char *name, long name_cap, int *compute_units, long *total_mem_bytes);

/* Timing on the library stream (the reference brackets ops with torch.Timer
 * around the no-op synchronize, gpunn/test/test.lua:2823-2831).  Events are
 * small integer handles. */
int thgpu_event_create(void);
int thgpu_event_record(int ev);
int thgpu_event_elapsed_ms(int ev_start, int ev_stop, float *ms); /* synchronises on ev_stop */

/* Per-kernel timing: while enabled every kernel launch of the library is
 * bracketed by HIP events on the library stream.  The report is a JSON object
 * {"kernel name": {"calls": n, "ms": total, "flops": total, "bytes": total}}
 * with the algorithmic flops/bytes the launch sites declare. */
int thgpu_prof_enable(int on);
int thgpu_prof_reset(void);
long thgpu_prof_report(char *buf, long cap); /* returns the length needed */

/* Host-only self check of the index arithmetic the kernels rely on (magic-number
 * division against the C operators over a sweep of divisors and dividends).
 * Needs no GPU.  Returns the number of mismatches. */
long thgpu_selftest_index_math(void);
/* Host-only check of the im2col strip planner and the max-pool backward tile planner over a grid of
 * geometries (LDS budgets, coverage, index ranges); returns the number of violations (no counterpart in the
 * reference). */
long thgpu_selftest_launch_plans(void);

/* ---- THGPUStorage: TH/generic/THStorage.h:33-65 instantiated for GPU,
 *      implementation replaced: gputorch/lib/THC/THCStorage.cpp:7-198 -------- */
float *THGPUStorage_data(const THGPUStorage *self);
long THGPUStorage_size(const THGPUStorage *self);
void THGPUStorage_set(THGPUStorage *self, long index, float value);  /* THCStorage.cpp:7-12, blocking */
float THGPUStorage_get(const THGPUStorage *self, long index);        /* THCStorage.cpp:14-21, blocking */
THGPUStorage *THGPUStorage_new(void);                                 /* THCStorage.cpp:23-34 */
THGPUStorage *THGPUStorage_newWithSize(long size);                    /* THCStorage.cpp:36-57 */
THGPUStorage *THGPUStorage_newWithSize1(float);                       /* THCStorage.cpp:59-64 */
THGPUStorage *THGPUStorage_newWithSize2(float, float);                /* THCStorage.cpp:66-72 */
THGPUStorage *THGPUStorage_newWithSize3(float, float, float);         /* THCStorage.cpp:74-81 */
THGPUStorage *THGPUStorage_newWithSize4(float, float, float, float);  /* THCStorage.cpp:83-91 */
THGPUStorage *THGPUStorage_newWithMapping(const char *filename, long size, int shared); /* error, THCStorage.cpp:93-97 */
/* `data` is a HOST pointer (THCStorage.cpp:99-110); its contents are uploaded. */
THGPUStorage *THGPUStorage_newWithData(float *data, long size);
void THGPUStorage_setFlag(THGPUStorage *self, const char flag);
void THGPUStorage_clearFlag(THGPUStorage *self, const char flag);
void THGPUStorage_retain(THGPUStorage *self);                         /* THCStorage.cpp:112-116 */
void THGPUStorage_free(THGPUStorage *self);                           /* THCStorage.cpp:118-140 */
void THGPUStorage_resize(THGPUStorage *self, long size);              /* THCStorage.cpp:154-198: new buffer, D2D copy of min(old,new) */
void THGPUStorage_fill(THGPUStorage *self, float value);              /* THCStorage.cpp:142-152 */

/* Blocking copies of n floats between a host buffer and device memory, replacing gpuMemcpy
 * (gputorch/lib/THC/copyHelpers.cpp:14-85) where a binding moves raw data itself: GPUStorage:write / :read stage the
 * floats through host memory around THFile_writeFloatRaw / readFloatRaw (gputorch/Storage.cpp:15-31). */
int thgpu_memcpy_h2d(float *dst_device, const float *src_host, long n);
int thgpu_memcpy_d2h(float *dst_host, const float *src_device, long n);

/* gputorch/lib/THC/THCStorageCopy.h:9-26, THCStorageCopy.cpp:5-75 */
void THGPUStorage_rawCopy(THGPUStorage *self, float *src); /* src is a DEVICE pointer (THCStorageCopy.cpp:56-62) */
void THGPUStorage_copy(THGPUStorage *self, THGPUStorage *src);
void THGPUStorage_copyGPU(THGPUStorage *self, THGPUStorage *src);
void THGPUStorage_copyByte(THGPUStorage *self, struct THByteStorage *src);
void THGPUStorage_copyChar(THGPUStorage *self, struct THCharStorage *src);
void THGPUStorage_copyShort(THGPUStorage *self, struct THShortStorage *src);
void THGPUStorage_copyInt(THGPUStorage *self, struct THIntStorage *src);
void THGPUStorage_copyLong(THGPUStorage *self, struct THLongStorage *src);
void THGPUStorage_copyFloat(THGPUStorage *self, struct THFloatStorage *src);
void THGPUStorage_copyDouble(THGPUStorage *self, struct THDoubleStorage *src);
void THByteStorage_copyGPU(THByteStorage *self, struct THGPUStorage *src);
void THCharStorage_copyGPU(THCharStorage *self, struct THGPUStorage *src);
void THShortStorage_copyGPU(THShortStorage *self, struct THGPUStorage *src);
void THIntStorage_copyGPU(THIntStorage *self, struct THGPUStorage *src);
void THLongStorage_copyGPU(THLongStorage *self, struct THGPUStorage *src);
void THFloatStorage_copyGPU(THFloatStorage *self, struct THGPUStorage *src);
void THDoubleStorage_copyGPU(THDoubleStorage *self, struct THGPUStorage *src);

/* ---- THGPUTensor: gputorch/lib/THC/THCTensor.h:53-152,
 *      implementation replaced: gputorch/lib/THC/THCTensor.cpp ---------------- */
THGPUStorage *THGPUTensor_storage(const THGPUTensor *self);
long THGPUTensor_storageOffset(const THGPUTensor *self);
int THGPUTensor_nDimension(const THGPUTensor *self);
long THGPUTensor_size(const THGPUTensor *self, int dim);
long THGPUTensor_stride(const THGPUTensor *self, int dim);
THLongStorage *THGPUTensor_newSizeOf(THGPUTensor *self);
THLongStorage *THGPUTensor_newStrideOf(THGPUTensor *self);
float *THGPUTensor_data(const THGPUTensor *self); /* device pointer incl. storageOffset */
void THGPUTensor_setFlag(THGPUTensor *self, const char flag);
void THGPUTensor_clearFlag(THGPUTensor *self, const char flag);

THGPUTensor *THGPUTensor_new(void);
THGPUTensor *THGPUTensor_newWithTensor(THGPUTensor *tensor);
THGPUTensor *THGPUTensor_newWithStorage(THGPUStorage *storage, long storageOffset, THLongStorage *size,
                                        THLongStorage *stride); /* stride may be NULL */
THGPUTensor *THGPUTensor_newWithStorage1d(THGPUStorage *storage, long storageOffset, long size0, long stride0);
THGPUTensor *THGPUTensor_newWithStorage2d(THGPUStorage *storage, long storageOffset, long size0, long stride0,
                                          long size1, long stride1);
THGPUTensor *THGPUTensor_newWithStorage3d(THGPUStorage *storage, long storageOffset, long size0, long stride0,
                                          long size1, long stride1, long size2, long stride2);
THGPUTensor *THGPUTensor_newWithStorage4d(THGPUStorage *storage, long storageOffset, long size0, long stride0,
                                          long size1, long stride1, long size2, long stride2, long size3,
                                          long stride3);
THGPUTensor *THGPUTensor_newWithSize(THLongStorage *size, THLongStorage *stride);
THGPUTensor *THGPUTensor_newWithSize1d(long size0);
THGPUTensor *THGPUTensor_newWithSize2d(long size0, long size1);
THGPUTensor *THGPUTensor_newWithSize3d(long size0, long size1, long size2);
THGPUTensor *THGPUTensor_newWithSize4d(long size0, long size1, long size2, long size3);
THGPUTensor *THGPUTensor_newClone(THGPUTensor *self);                 /* THCTensor.cpp:178-184 */
THGPUTensor *THGPUTensor_newContiguous(THGPUTensor *tensor);          /* THCTensor.cpp:186-195: self retained if contiguous */
THGPUTensor *THGPUTensor_newSelect(THGPUTensor *tensor, int dimension, long sliceIndex);
THGPUTensor *THGPUTensor_newNarrow(THGPUTensor *tensor, int dimension, long firstIndex, long size);
THGPUTensor *THGPUTensor_newTranspose(THGPUTensor *tensor, int dimension1, int dimension2);
THGPUTensor *THGPUTensor_newUnfold(THGPUTensor *tensor, int dimension, long size, long step);

void THGPUTensor_resize(THGPUTensor *tensor, THLongStorage *size, THLongStorage *stride);
void THGPUTensor_resizeAs(THGPUTensor *tensor, THGPUTensor *src);
void THGPUTensor_resize1d(THGPUTensor *tensor, long size0);
void THGPUTensor_resize2d(THGPUTensor *tensor, long size0, long size1);
void THGPUTensor_resize3d(THGPUTensor *tensor, long size0, long size1, long size2);
void THGPUTensor_resize4d(THGPUTensor *tensor, long size0, long size1, long size2, long size3);
void THGPUTensor_resize5d(THGPUTensor *tensor, long size0, long size1, long size2, long size3, long size4);

void THGPUTensor_set(THGPUTensor *self, THGPUTensor *src);
void THGPUTensor_setStorage(THGPUTensor *self, THGPUStorage *storage, long storageOffset, THLongStorage *size,
                            THLongStorage *stride);
void THGPUTensor_setStorage1d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0);
void THGPUTensor_setStorage2d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0,
                              long size1, long stride1);
void THGPUTensor_setStorage3d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0,
                              long size1, long stride1, long size2, long stride2);
void THGPUTensor_setStorage4d(THGPUTensor *self, THGPUStorage *storage, long storageOffset, long size0, long stride0,
                              long size1, long stride1, long size2, long stride2, long size3, long stride3);
void THGPUTensor_narrow(THGPUTensor *self, THGPUTensor *src, int dimension, long firstIndex, long size);
void THGPUTensor_select(THGPUTensor *self, THGPUTensor *src, int dimension, long sliceIndex);
void THGPUTensor_transpose(THGPUTensor *self, THGPUTensor *src, int dimension1, int dimension2);
void THGPUTensor_unfold(THGPUTensor *self, THGPUTensor *src, int dimension, long size, long step);   /* THCTensor.h:92; TH/generic/THTensor.c:418-460 */
void THGPUTensor_squeeze(THGPUTensor *self, THGPUTensor *src);                                         /* TH/generic/THTensor.c:462-493 */
void THGPUTensor_squeeze1d(THGPUTensor *self, THGPUTensor *src, int dimension);                        /* TH/generic/THTensor.c:495-513 */

int THGPUTensor_isContiguous(const THGPUTensor *self);                /* THCTensor.cpp:510-525 */
int THGPUTensor_isSameSizeAs(const THGPUTensor *self, const THGPUTensor *src);
long THGPUTensor_nElement(const THGPUTensor *self);
void THGPUTensor_retain(THGPUTensor *self);
void THGPUTensor_free(THGPUTensor *self);
void THGPUTensor_freeCopyTo(THGPUTensor *self, THGPUTensor *dst);

void THGPUTensor_set1d(THGPUTensor *tensor, long x0, float value);
void THGPUTensor_set2d(THGPUTensor *tensor, long x0, long x1, float value);
void THGPUTensor_set3d(THGPUTensor *tensor, long x0, long x1, long x2, float value);
void THGPUTensor_set4d(THGPUTensor *tensor, long x0, long x1, long x2, long x3, float value);
float THGPUTensor_get1d(const THGPUTensor *tensor, long x0);
float THGPUTensor_get2d(const THGPUTensor *tensor, long x0, long x1);
float THGPUTensor_get3d(const THGPUTensor *tensor, long x0, long x1, long x2);
float THGPUTensor_get4d(const THGPUTensor *tensor, long x0, long x1, long x2, long x3);

/* gputorch/lib/THC/THCTensorMath.h:7-8, THCTensorMath.cpp:15-42 */
void THGPUTensor_fill(THGPUTensor *self, float value);
void THGPUTensor_zero(THGPUTensor *self);

/* THGPUTensor_fill for `count` contiguous tensors in one kernel launch (no counterpart in the reference, where a
 * network's gradients are zeroed tensor by tensor, mcw_nn/Module.lua:66-73, or flattened into one storage by
 * getParameters first): what nn.Sequential:zeroGradParameters amounts to on a stack of small layers.  Returns 0
 * or a status with thgpu_last_error() set; nothing is written when a tensor is rejected. */
int thgpu_fill_many(THGPUTensor **tensors, int count, float value);

/* gputorch/lib/THC/THCTensorCopy.h:7-23.  copy handles any strides
 * (THCTensorCopy.cpp:170-290); host<->device copies are blocking
 * (THCTensorCopy.cpp:20-36,64-80). */
void THGPUTensor_copy(THGPUTensor *self, THGPUTensor *src);
void THGPUTensor_copyGPU(THGPUTensor *self, THGPUTensor *src);
void THGPUTensor_copyByte(THGPUTensor *self, THByteTensor *src);
void THGPUTensor_copyChar(THGPUTensor *self, THCharTensor *src);
void THGPUTensor_copyShort(THGPUTensor *self, THShortTensor *src);
void THGPUTensor_copyInt(THGPUTensor *self, THIntTensor *src);
void THGPUTensor_copyLong(THGPUTensor *self, THLongTensor *src);
void THGPUTensor_copyFloat(THGPUTensor *self, THFloatTensor *src);
void THGPUTensor_copyDouble(THGPUTensor *self, THDoubleTensor *src);
void THByteTensor_copyGPU(THByteTensor *self, THGPUTensor *src);
void THCharTensor_copyGPU(THCharTensor *self, THGPUTensor *src);
void THShortTensor_copyGPU(THShortTensor *self, THGPUTensor *src);
void THIntTensor_copyGPU(THIntTensor *self, THGPUTensor *src);
void THLongTensor_copyGPU(THLongTensor *self, THGPUTensor *src);
void THFloatTensor_copyGPU(THFloatTensor *self, THGPUTensor *src);
void THDoubleTensor_copyGPU(THDoubleTensor *self, THGPUTensor *src);

/* ---- tensor math on the GEMM (the classifier layers after a conv stack) ------ */

/* self = src + value / src * value / src / value, self resized to src
 * (gputorch/lib/THC/THCTensorMath.cpp:67-101). */
void THGPUTensor_add(THGPUTensor *self, THGPUTensor *src, float value);
void THGPUTensor_mul(THGPUTensor *self, THGPUTensor *src, float value);
void THGPUTensor_div(THGPUTensor *self, THGPUTensor *src, float value);
/* self = src1 + value * src2 (THCTensorMath.cpp:103-131). */
void THGPUTensor_cadd(THGPUTensor *self, THGPUTensor *src1, float value, THGPUTensor *src2);
/* self = beta*t + alpha * mat*vec, mat1*mat2, vec1 (x) vec2; self is resized to t and
 * takes its values when they differ; views contiguous along either dimension are used
 * in place (THCTensorMath.cpp:624-829; CPU twin TH/generic/THTensorMath.c:458-620). */
void THGPUTensor_addmv(THGPUTensor *self, float beta, THGPUTensor *t, float alpha, THGPUTensor *mat, THGPUTensor *vec);
void THGPUTensor_addmm(THGPUTensor *self, float beta, THGPUTensor *t, float alpha, THGPUTensor *mat1,
                       THGPUTensor *mat2);
void THGPUTensor_addr(THGPUTensor *self, float beta, THGPUTensor *t, float alpha, THGPUTensor *vec1,
                      THGPUTensor *vec2);

/* gputorch/lib/THC/THCTensorMath.h:28,91-93 (THCTensorMath.cpp:269-280,1331-1465): the rest of what Torch's generic
 * tensor binding calls (torch/generic/Tensor.c:405-454 `index`, `indexCopy`, `indexFill`; TensorOperator.c:120 `*`).
 * dot sums in two fixed-shape stages (reruns are bit-identical) and blocks; the index operations take a HOST vector of
 * 1-based indices and work slice by slice, like TH/generic/THTensorMath.c:69-176. */
float THGPUTensor_dot(THGPUTensor *self, THGPUTensor *src);
void THGPUTensor_indexCopy(THGPUTensor *res_, int dim, struct THLongTensor *indices, THGPUTensor *src);
void THGPUTensor_indexFill(THGPUTensor *tensor, int dim, struct THLongTensor *index, float val);
void THGPUTensor_indexSelect(THGPUTensor *tensor, THGPUTensor *src, int dim, struct THLongTensor *index);

/* ---- BLAS ------------------------------------------------------------------ */

/* Level-1 / level-2 BLAS on device pointers with strided vectors: the generic TH signatures
 * (mcw_torch7_core/lib/TH/generic/THBlas.h) in place of the array_view + offset ones of
 * gputorch/lib/THC/THCBlas.h:29-48 (called from THCTensorMath.cpp:122,671-688,835-852 and
 * gpunn-impl/SpatialConvolutionMM.cpp:413).  Column-major, semantics and degenerate-dimension fix-ups of
 * TH/generic/THBlas.c:68-100,182-264; gemv 'n', ger and axpy add in TH's own order (bit-identical to its
 * fallback loops), gemv 't' sums each column with a fixed-shape tree.  THGPUTensor_addmv / addr keep riding
 * the GEMM. */
void THGPUBlas_axpy(long n, float a, float *x, long incx, float *y, long incy);
void THGPUBlas_ger(long m, long n, float alpha, float *x, long incx, float *y, long incy, float *a, long lda);
void THGPUBlas_gemv(char trans, long m, long n, float alpha, float *a, long lda, float *x, long incx, float beta,
                    float *y, long incy);

/* Column-major C = beta*C + alpha*op(A)*op(B) on DEVICE pointers: the generic
 * THBlas signature (TH/generic/THBlas.h:17 instantiated by gputorch/lib/THC/
 * THCBlas.h:6-14); replaces the array_view overload THCBlas.h:35-39 and its
 * kernels THCBlas.cpp:10-288 (offsets fold into the pointers).  All four
 * transpose variants honour lda/ldb/ldc.  Quick returns as THCBlas.cpp:257. */
void THGPUBlas_gemm(char transa, char transb, long m, long n, long k, float alpha, float *a, long lda, float *b,
                    long ldb, float beta, float *c, long ldc);

/* The same product for `batch` problems whose operands and results are `stride_*` floats apart
 * (stride 0 shares an operand).  New: the reference multiplies image by image (gpunn-impl/
 * SpatialConvolutionMM.cpp:168-217 calls THGPUBlas_gemm once per image); here a shared op(B) with
 * transa == 'n' -- the convolution's forward and gradInput products -- runs as one launch.  Returns
 * 0 or a status with thgpu_last_error() set. */
int thgpu_gemm_strided_batched(char transa, char transb, long m, long n, long k, float alpha, const float *a, long lda,
                               long stride_a, const float *b, long ldb, long stride_b, float beta, float *c, long ldc,
                               long stride_c, long batch);

/* THGPUBlas_gemm for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments
 * and result as THGPUBlas_gemm, status returned instead of the error handler being called.  The call
 * allocates nothing: the partial sums of a split reduction, which THGPUBlas_gemm keeps in a workspace
 * that grows with hipMalloc, go to a fixed array of THGPU_GEMM_NOALLOC_MAX_ELEMENTS floats (64 MiB) that
 * the library holds on the GPU from load to exit, and the split is chosen among those whose partial sums
 * fit it.  Limits: thgpu_init() must have been called (outside any capture; this call sets nothing up and
 * fails otherwise); a result of more than THGPU_GEMM_NOALLOC_MAX_ELEMENTS elements (m * n) is rejected.
 * Every call on the GPU shares the one array: calls that overlap in time (other streams or threads) race;
 * calls through the library stream, which is what this function enqueues on, are ordered. */
#define THGPU_GEMM_NOALLOC_MAX_ELEMENTS (16L << 20)
int thgpu_gemm_noalloc(char transa, char transb, long m, long n, long k, float alpha, const float *a, long lda,
                       const float *b, long ldb, float beta, float *c, long ldc);

/* ---- flat operator entry points -------------------------------------------- */

/* Batched im2col: im [B,C,H,W] -> col [B, C*kH*kW, Ho*Wo] (device pointers).
 * Replaces the per-image kernel gputorch/lib/THC/gpunn-impl/
 * SpatialConvolutionMM.cpp:10-52; output layout and zero padding as the CPU
 * nn_(unfolded_copy), mcw_nn/generic/SpatialConvolutionMM.c:52-96. */
int thgpu_im2col(const float *im, long B, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                 float *col);

/* Batched col2im gather: col [B, C*kH*kW, Ho*Wo] -> im [B,C,H,W], overwriting
 * im.  Replaces gpunn-impl/SpatialConvolutionMM.cpp:54-108; every pixel is
 * summed from 0 in kh-ascending, kw-ascending order, bit-matching the CPU
 * nn_(unfolded_acc), mcw_nn/generic/SpatialConvolutionMM.c:6-50. */
int thgpu_col2im(const float *col, long B, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                 float *im);

/* nn.SpatialConvolutionMM.  Replace gpunn_SpatialConvolutionMM_updateOutput /
 * _updateGradInput / _accGradParameters (gpunn-impl/SpatialConvolutionMM.cpp:
 * 110-225, 227-311, 313-429); arguments are the module fields those read by
 * name (:116-128) with the single `padding` split into padW/padH.  input is
 * [C,H,W] or [B,C,H,W] contiguous and is never modified; weight is
 * [M, C*kH*kW].  Buffer shapes follow the CPU module, the parity target
 * (mcw_nn/generic/SpatialConvolutionMM.c:179,243): finput is resized to
 * [B,K,N] and keeps the whole batch of columns, fgradInput likewise holds the
 * column gradients.  accGradParameters rebuilds finput from its `input`
 * argument on every call, as the reference GPU code does (:388-396), so its
 * result depends on its arguments alone: finput and fgradInput may be shared
 * between modules, and `input` need not be the last forward pass's (see
 * thgpu_conv_set_finput_reuse for the CPU module's behaviour). */
int thgpu_SpatialConvolutionMM_updateOutput(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
                                            THGPUTensor *finput, THGPUTensor *fgradInput, THGPUTensor *output,
                                            int kW, int kH, int dW, int dH, int padW, int padH);
int thgpu_SpatialConvolutionMM_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                               THGPUTensor *finput, THGPUTensor *fgradInput,
                                               THGPUTensor *gradInput, int kW, int kH, int dW, int dH, int padW,
                                               int padH);
int thgpu_SpatialConvolutionMM_accGradParameters(THGPUTensor *input, THGPUTensor *gradOutput,
                                                 THGPUTensor *gradWeight, THGPUTensor *gradBias,
                                                 THGPUTensor *finput, THGPUTensor *fgradInput, int kW, int kH,
                                                 int dW, int dH, int padW, int padH, float scale);

/* nn.Threshold fused into its neighbours (no counterpart in the reference, where gpunn_Threshold_updateOutput /
 * _updateGradInput, gpunn-impl/Threshold.cpp:16-81, always run as passes of their own).
 * updateOutputFused, THGPU_FUSE_THRESHOLD: output = y > threshold ? y : val for every y = conv(input) + bias, applied
 *   as the value is stored; bit-identical to updateOutput followed by thgpu_Threshold_updateOutput in place.
 * updateGradInputFused, THGPU_FUSE_INPUT_MASK: gradInput = input > threshold ? g : 0 for every g of updateGradInput,
 *   applied as the value is stored -- the backward of a Threshold in front of this module, whose output `input` is
 *   (value <= threshold assumed, so that its output exceeds the threshold exactly where its input did);
 *   bit-identical to updateGradInput followed by thgpu_Threshold_updateGradInput.
 *
 * The padded image without a copy.  On the gathered route (thgpu_conv_set_mode) updateOutput and accGradParameters
 * read a copy of the input with a zero border of padH rows and padW columns.  A producer can write that image
 * itself: SpatialConvolutionMM_updateOutput* and SpatialMaxPooling_updateOutput leave an `output` tensor that
 * already has the right sizes as it is, also when it is a view with contiguous rows into a larger buffer (strides
 * (C*P, P, pitch, 1)), and store into it.  With THGPU_INPUT_IN_PADDED_BUFFER the caller states that `input` is
 * such a view: the interior of a [B, C, H + 2 padH, W + 2 padW] buffer whose border holds zeros.  The layout is
 * checked, the zeros are the caller's word; no copy is made and finput stays untouched (a layer that does not
 * gather copies the view into dense form first).  updateGradInputFused takes its mask from such a view as well. */
#define THGPU_FUSE_THRESHOLD 1          /* updateOutputFused */
#define THGPU_FUSE_INPUT_MASK 1         /* updateGradInputFused */
#define THGPU_INPUT_IN_PADDED_BUFFER 2  /* updateOutputFused, accGradParametersFused */
int thgpu_SpatialConvolutionMM_updateOutputFused(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
                                                 THGPUTensor *finput, THGPUTensor *fgradInput, THGPUTensor *output,
                                                 int kW, int kH, int dW, int dH, int padW, int padH, int flags,
                                                 float threshold, float val);
int thgpu_SpatialConvolutionMM_updateGradInputFused(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                                    THGPUTensor *finput, THGPUTensor *fgradInput,
                                                    THGPUTensor *gradInput, int kW, int kH, int dW, int dH, int padW,
                                                    int padH, int flags, float threshold);
int thgpu_SpatialConvolutionMM_accGradParametersFused(THGPUTensor *input, THGPUTensor *gradOutput,
                                                      THGPUTensor *gradWeight, THGPUTensor *gradBias,
                                                      THGPUTensor *finput, THGPUTensor *fgradInput, int kW, int kH,
                                                      int dW, int dH, int padW, int padH, float scale, int flags);
/* The padded gradient without a copy (no counterpart in the reference).  On the gathered route updateGradInput reads
 * gradOutput from a zero-bordered copy at the head of fgradInput.  Inside a container that knows which module
 * produces a layer's gradOutput, that producer can store its result there as well while it stores it densely:
 *   1. thgpu_SpatialConvolutionMM_gradOutputTwin (the layer's own input, weight, fgradInput and geometry): sizes
 *      fgradInput for the gathered gradInput product, zeroes its padded region unless it is known to be zero-bordered
 *      for this geometry already, and makes `twin` a [B,] M, Ho, Wo view of gradOutput's place in it.  *available is 0
 *      (and nothing is touched) when the layer's gradInput does not take the gathered route.
 *   2. the producer's updateGradInput -- thgpu_SpatialMaxPooling_updateGradInputTwin or
 *      thgpu_SpatialConvolutionMM_updateGradInputTwin with that `twin` -- stores every value of its gradInput a second
 *      time through the view; *wrote_twin says whether the kernel that ran could (the max-pooling kernels for 3x3 and 2x2
 *      windows at stride 2 and the unit-stride gathered gradInput product can; otherwise only the dense result is
 *      written).
 *   3. the layer's thgpu_SpatialConvolutionMM_updateGradInputTwin with THGPU_GRADOUTPUT_IN_TWIN, called with that
 *      dense gradInput as gradOutput before anything else touches either tensor: no padded copy is made.  The flag
 *      is the caller's word for the contents; it is ignored (the copy is made) unless fgradInput is still the buffer
 *      step 1 prepared for this geometry.
 * Results are bit-identical to the plain entry points'.  `twin` may be NULL in the *Twin entry points (no second
 * copy); flags also take THGPU_FUSE_INPUT_MASK with `threshold` as in updateGradInputFused / ...Masked. */
#define THGPU_GRADOUTPUT_IN_TWIN 8 /* SpatialConvolutionMM_updateGradInputTwin */
int thgpu_SpatialConvolutionMM_gradOutputTwin(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *fgradInput,
                                              THGPUTensor *twin, int kW, int kH, int dW, int dH, int padW, int padH,
                                              int *available);
int thgpu_SpatialConvolutionMM_updateGradInputTwin(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                                   THGPUTensor *finput, THGPUTensor *fgradInput,
                                                   THGPUTensor *gradInput, int kW, int kH, int dW, int dH, int padW,
                                                   int padH, int flags, float threshold, THGPUTensor *twin,
                                                   int *wrote_twin);
/* 1 when updateOutput / accGradParameters of a layer with these sizes would gather from the padded image in the
 * current mode (and so profit from an input that already lies in a padded buffer), 0 otherwise. */
int thgpu_conv_gathers(long B, int C, int H, int W, int M, int kW, int kH, int dW, int dH, int padW, int padH);

/* How the three entry points above compute (no counterpart in the reference, whose only route is
 * im2col + sgemm + col2im, gpunn-impl/SpatialConvolutionMM.cpp:110-429).
 *   mode 0: that route; finput and fgradInput hold the K x N columns as in the reference.
 *   mode 1 (initial): per layer and pass, the GEMM gathers its second operand from a zero-padded copy
 *           of the image and no columns exist, where the shape allows it and it is the faster route
 *           (forward and gradWeight: wherever a tiled kernel takes the product; gradInput: layers whose input
 *           planes fill the 64-row tiles and that are padded, or strided ones); the column route otherwise.
 *   mode 2: gathered wherever the shape allows it.
 * On the gathered route finput holds the padded input ([B,] C, H+2padH, W+2padW) and fgradInput the
 * padded gradOutput followed by the flipped kernels; outputs and gradients are the same sums of the
 * same products, equal to the column route's to fp32 rounding.  The environment variable THGPU_CONV
 * (columns | auto | gathered) sets the initial mode.  set returns 0, or an error for any other mode. */
int thgpu_conv_set_mode(int mode);
int thgpu_conv_get_mode(void);

/* on != 0: accGradParameters takes a finput that has the shape the forward pass gives it to BE the forward
 * pass's and does not rebuild it -- the CPU module's behaviour (mcw_nn/generic/SpatialConvolutionMM.c:318,
 * 336), which saves one pass over the input per call and is wrong when `input` is not what the last
 * updateOutput of this module saw or when another module wrote the shared buffer in between (no
 * counterpart in the reference GPU code, which always rebuilds).  Initially off.  Returns 0. */
int thgpu_conv_set_finput_reuse(int on);
int thgpu_conv_get_finput_reuse(void);

/* nn.SpatialMaxPooling.  Replace gpunn_SpatialMaxPooling_updateOutput /
 * _updateGradInput (gpunn-impl/SpatialMaxPooling.cpp:205-281, 283-383).
 * indices is resized to [2,(B,)C,Ho,Wo] floats, plane 0 = ky+1, plane 1 = kx+1
 * (mcw_nn/generic/SpatialMaxPooling.c:51-52,133-134).  Backward accepts
 * overlapping windows (the reference GPU code rejects dW!=kW, :293-294) and
 * adds in the CPU order (mcw_nn/generic/SpatialMaxPooling.c:165-174). */
int thgpu_SpatialMaxPooling_updateOutput(THGPUTensor *input, THGPUTensor *output, THGPUTensor *indices, int kW,
                                         int kH, int dW, int dH);
int thgpu_SpatialMaxPooling_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                            THGPUTensor *indices, int kW, int kH, int dW, int dH);

/* updateGradInput with the backward of a Threshold in front of the pooling layer applied as gradInput is stored:
 * gradInput = input > threshold ? g : 0 (see thgpu_SpatialConvolutionMM_updateGradInputFused). */
/* ... and with a second copy of gradInput stored through `twin` (see thgpu_SpatialConvolutionMM_gradOutputTwin). */
int thgpu_SpatialMaxPooling_updateGradInputTwin(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                                THGPUTensor *indices, int kW, int kH, int dW, int dH, int flags,
                                                float threshold, THGPUTensor *twin, int *wrote_twin);
int thgpu_SpatialMaxPooling_updateGradInputMasked(THGPUTensor *input, THGPUTensor *gradOutput,
                                                  THGPUTensor *gradInput, THGPUTensor *indices, int kW, int kH,
                                                  int dW, int dH, float threshold);

/* nn.Threshold / nn.ReLU.  Replace gpunn_Threshold_updateOutput /
 * _updateGradInput (gpunn-impl/Threshold.cpp:16-38, 53-81). */
int thgpu_Threshold_updateOutput(THGPUTensor *input, THGPUTensor *output, float threshold, float val);
int thgpu_Threshold_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                    float threshold);

/* nn.SpatialAveragePooling.  Replace gpunn_SpatialAveragePooling_updateOutput /
 * _updateGradInput (gpunn-impl/SpatialAveragePooling.cpp:67-124, 185-233; CPU twin
 * mcw_nn/generic/SpatialAveragePooling.c:5-94, 96-174).  Despite the name the
 * module returns the window SUM (neither implementation divides).  No padding,
 * Ho = (H - kH) / dH + 1.  Results are bit-identical to the CPU module's;
 * backward accepts overlapping windows (the reference GPU code requires
 * dW == kW and dH == kH, :194-195). */
int thgpu_SpatialAveragePooling_updateOutput(THGPUTensor *input, THGPUTensor *output, int kW, int kH, int dW, int dH);
int thgpu_SpatialAveragePooling_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                                int kW, int kH, int dW, int dH);

/* nn.SpatialSubSampling: output = bias[k] + weight[k] * sum(window), one weight
 * and one bias per plane.  Replace gpunn_SpatialSubSampling_updateOutput /
 * _updateGradInput / _accGradParameters (gpunn-impl/SpatialSubSampling.cpp:246-317,
 * 319-373, 375-440; CPU twin mcw_nn/generic/SpatialSubSampling.c:5-100, 102-185,
 * 187-275).  weight, bias, gradWeight, gradBias: contiguous vectors of
 * nInputPlane elements.  output and gradInput are bit-identical to the CPU
 * module's; gradWeight and gradBias are deterministic and agree to rounding. */
int thgpu_SpatialSubSampling_updateOutput(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
                                          THGPUTensor *output, int kW, int kH, int dW, int dH);
int thgpu_SpatialSubSampling_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                             THGPUTensor *gradInput, int kW, int kH, int dW, int dH);
int thgpu_SpatialSubSampling_accGradParameters(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradWeight,
                                               THGPUTensor *gradBias, int kW, int kH, int dW, int dH, float scale);

/* nn.LogSoftMax on a vector or a matrix of frames.  Replace gpunn_LogSoftMax_updateOutput /
 * _updateGradInput (gpunn-impl/LogSoftMax.cpp:115-146, 148-181).  The arithmetic is the CPU
 * module's (mcw_nn/generic/LogSoftMax.c:37-53, 85-97: double accumulation and the polynomial
 * THExpMinusApprox of TH/THLogAdd.c:56-86 in the forward sum), so results agree with it to the
 * rounding of the float output.  updateGradInput reads the module's output, not its input. */
int thgpu_LogSoftMax_updateOutput(THGPUTensor *input, THGPUTensor *output);
int thgpu_LogSoftMax_updateGradInput(THGPUTensor *gradOutput, THGPUTensor *output, THGPUTensor *gradInput);

/* nn.ClassNLLCriterion without class weights.  Replace gpunn_ClassNLLCriterion_updateOutput /
 * _updateGradInput (gpunn-impl/ClassNLLCriterion.cpp:96-135, 137-184).  target holds 1-based class
 * numbers as floats, one per frame ([nframe] or [nframe, ntarget]); outputTensor is the module's
 * one-element tensor and receives -(sum of input[i][target[i]-1]) [/ nframe when sizeAverage and the
 * input is a matrix].  updateGradInput writes -1 [/ nframe] at the target positions of gradInput, which
 * the caller has sized like the input and zeroed (mcw_nn/ClassNLLCriterion.lua:43-51).  Targets outside
 * 1..ndim are skipped. */
int thgpu_ClassNLLCriterion_updateOutput(THGPUTensor *input, THGPUTensor *target, THGPUTensor *outputTensor,
                                         int sizeAverage);
int thgpu_ClassNLLCriterion_updateGradInput(THGPUTensor *input, THGPUTensor *target, THGPUTensor *gradInput,
                                            int sizeAverage);

#ifdef __cplusplus
}
#endif
#endif /* THGPU_H */
