// THGPUTensor BLAS-level math on the MFMA GEMM: addmm, addmv, addr, and the
// scalar/axpy elementwise operations nn.Linear is written with
// (mcw_nn/Linear.lua:34-101).  The view handling follows the reference
// dispatcher (gputorch/lib/THC/THCTensorMath.cpp:624-829, the same logic as
// TH/generic/THTensorMath.c:458-561): a result or operand that is contiguous
// along either of its two dimensions is used in place through the transpose
// flags of THGPUBlas_gemm, anything else goes through a dense copy.
#include "common.h"

#include <vector>

using namespace thgpu;

namespace {

// op 0: out = in + v; 1: out = in * v; 2: out = in / v; 3: out = out + v * in (axpy)
__global__ __launch_bounds__(256) void scalar_op_kernel(const float *__restrict__ in, float *__restrict__ out, long n,
                                                        float v, int op) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float x = in[i];
        // the axpy keeps the two roundings of y[i] += a*x[i] (TH/generic/THBlas.c:96-99): no fused multiply-add
        out[i] = op == 0 ? x + v : op == 1 ? x * v : op == 2 ? x / v : __fadd_rn(out[i], __fmul_rn(v, x));
    }
}

int scalar_op(const float *in, float *out, long n, float v, int op, const char *tag) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (n == 0) return 0;
    long blocks = (n + 255) / 256;
    if (blocks > 8L * 4 * num_cus()) blocks = 8L * 4 * num_cus();
    {
        LaunchScope scope(tag, 0.0, (op == 3 ? 12.0 : 8.0) * n);
        hipLaunchKernelGGL(scalar_op_kernel, dim3((unsigned)blocks), dim3(256), 0, s, in, out, n, v, op);
    }
    return check_launch(tag);
}

// self = op(src, value) with the reference's resize / densify / copy-back sequence
// (THCTensorMath.cpp:67-101).
void unary_scalar(THGPUTensor *self_, THGPUTensor *src_, float value, int op, const char *tag) {
    THGPUTensor_resizeAs(self_, src_);
    THGPUTensor *self = THGPUTensor_newContiguous(self_);
    THGPUTensor *src = THGPUTensor_newContiguous(src_);
    if (scalar_op(THGPUTensor_data(src), THGPUTensor_data(self), THGPUTensor_nElement(self), value, op, tag))
        raise("%s", thgpu_last_error());
    THGPUTensor_free(src);
    THGPUTensor_freeCopyTo(self, self_);
}

// ---- level-1 / level-2 BLAS with strided vectors, in the loop order of TH's own routines ---------------------

// y[i*incy] += a * x[i*incx]   (TH/generic/THBlas.c:96-99)
__global__ __launch_bounds__(256) void axpy_kernel(long n, float a, const float *__restrict__ x, long incx,
                                                   float *__restrict__ y, long incy) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        y[i * incy] = __fadd_rn(y[i * incy], __fmul_rn(a, x[i * incx]));
}

// a[i + j*lda] += (alpha * y[j*incy]) * x[i*incx]   (TH/generic/THBlas.c:254-262)
__global__ __launch_bounds__(256) void ger_kernel(long m, long n, float alpha, const float *__restrict__ x, long incx,
                                                  const float *__restrict__ y, long incy, float *__restrict__ a,
                                                  long lda) {
    const long total = m * n;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
        const long j = e / m, i = e - j * m;
        const float z = __fmul_rn(alpha, y[j * incy]);
        a[i + j * lda] = __fadd_rn(a[i + j * lda], __fmul_rn(z, x[i * incx]));
    }
}

// 'n': y[i] = beta*y[i], then += (alpha*x[j]) * a[i + j*lda] for j ascending: one lane per row i, rows coalesced
// (TH/generic/THBlas.c:229-240; beta == 1 leaves y as it is, any other beta scales it first, as scal does).
__global__ __launch_bounds__(256) void gemv_n_kernel(long m, long n, float alpha, const float *__restrict__ a, long lda,
                                                     const float *__restrict__ x, long incx, float beta,
                                                     float *__restrict__ y, long incy) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= m) return;
    float acc = beta == 1.0f ? y[i * incy] : __fmul_rn(beta, y[i * incy]);
    for (long j = 0; j < n; ++j) acc = __fadd_rn(acc, __fmul_rn(__fmul_rn(alpha, x[j * incx]), a[i + j * lda]));
    y[i * incy] = acc;
}

// 't': y[i] = beta*y[i] + alpha * sum_j x[j] * a[j + i*lda]: one wavefront per output, lanes along the column, then a
// fixed-shape tree over the 64 lane sums (TH/generic/THBlas.c:216-226 adds j ascending: tolerance parity, not bit parity).
__global__ __launch_bounds__(256) void gemv_t_kernel(long m, long n, float alpha, const float *__restrict__ a, long lda,
                                                     const float *__restrict__ x, long incx, float beta,
                                                     float *__restrict__ y, long incy) {
    const long i = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (i >= n) return;
    const float *col = a + i * lda;
    float sum = 0.0f;
    for (long j = lane; j < m; j += 64) sum += x[j * incx] * col[j];
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
    if (lane == 0) y[i * incy] = beta * y[i * incy] + alpha * sum;
}

// dot product in two fixed-shape stages, so that reruns are bit-identical: every workgroup sums one contiguous chunk
// (lanes strided over it, then a tree over the 256 lane sums), a single workgroup adds the chunk sums the same way.
__global__ __launch_bounds__(256) void dot_partial_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                          long n, long chunk, float *__restrict__ part) {
    const long lo = (long)blockIdx.x * chunk;
    const long hi = lo + chunk < n ? lo + chunk : n;
    float sum = 0.0f;
    for (long i = lo + threadIdx.x; i < hi; i += 256) sum += a[i] * b[i];
    __shared__ float red[256];
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[blockIdx.x] = red[0];
}

__global__ __launch_bounds__(256) void dot_final_kernel(const float *__restrict__ part, int nparts,
                                                        float *__restrict__ out) {
    float sum = 0.0f;
    for (int i = threadIdx.x; i < nparts; i += 256) sum += part[i];
    __shared__ float red[256];
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = red[0];
}

// The 1-based entries of a host index vector, checked against the size they index.
bool host_indices(const THLongTensor *index, long limit, std::vector<long> &out, const char *who) {
    const long n = index->size[0];
    const long st = index->stride ? index->stride[0] : 1;
    if (n > 0 && (!index->storage || !index->storage->data)) {
        raise("%s: index tensor has no storage", who);
        return false;
    }
    out.resize((size_t)n);
    for (long i = 0; i < n; ++i) {
        const long v = index->storage->data[index->storageOffset + i * st];
        if (v < 1 || v > limit) {
            raise("%s: index %ld out of range [1, %ld]", who, v, limit);
            return false;
        }
        out[(size_t)i] = v - 1;
    }
    return true;
}

int launch_grid(long work) {
    long blocks = (work + 255) / 256;
    const long cap = 8L * 4 * num_cus();
    return (int)(blocks > cap ? cap : blocks < 1 ? 1 : blocks);
}

}  // namespace

extern "C" {

void THGPUBlas_axpy(long n, float a, float *x, long incx, float *y, long incy) {
    hipStream_t s = stream();
    if (!s) return raise("%s", thgpu_last_error());
    if (n <= 0) return;
    if (!x || !y) return raise("THGPUBlas_axpy: null operand");
    if (n == 1) incx = incy = 1;  // TH/generic/THBlas.c:72-76
    {
        LaunchScope scope("blas_axpy", 2.0 * n, 12.0 * n);
        hipLaunchKernelGGL(axpy_kernel, dim3(launch_grid(n)), dim3(256), 0, s, n, a, x, incx, y, incy);
    }
    if (check_launch("blas_axpy")) raise("%s", thgpu_last_error());
}

void THGPUBlas_ger(long m, long n, float alpha, float *x, long incx, float *y, long incy, float *a, long lda) {
    hipStream_t s = stream();
    if (!s) return raise("%s", thgpu_last_error());
    if (m <= 0 || n <= 0) return;
    if (!x || !y || !a) return raise("THGPUBlas_ger: null operand");
    if (n == 1) lda = m;  // TH/generic/THBlas.c:232-233
    {
        LaunchScope scope("blas_ger", 2.0 * m * n, 8.0 * m * n);
        hipLaunchKernelGGL(ger_kernel, dim3(launch_grid(m * n)), dim3(256), 0, s, m, n, alpha, x, incx, y, incy, a, lda);
    }
    if (check_launch("blas_ger")) raise("%s", thgpu_last_error());
}

void THGPUBlas_gemv(char trans, long m, long n, float alpha, float *a, long lda, float *x, long incx, float beta,
                    float *y, long incy) {
    hipStream_t s = stream();
    if (!s) return raise("%s", thgpu_last_error());
    if (n == 1) lda = m;  // TH/generic/THBlas.c:184-185
    const bool t = trans == 't' || trans == 'T';
    const long outs = t ? n : m;
    if (outs <= 0) return;
    if (!a || !x || !y) return raise("THGPUBlas_gemv: null operand");
    {
        LaunchScope scope("blas_gemv", 2.0 * m * n, 4.0 * m * n);
        if (t)
            hipLaunchKernelGGL(gemv_t_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, s, m, n, alpha, a, lda, x, incx,
                               beta, y, incy);
        else
            hipLaunchKernelGGL(gemv_n_kernel, dim3((unsigned)((m + 255) / 256)), dim3(256), 0, s, m, n, alpha, a, lda, x,
                               incx, beta, y, incy);
    }
    if (check_launch("blas_gemv")) raise("%s", thgpu_last_error());
}

void THGPUTensor_add(THGPUTensor *self, THGPUTensor *src, float value) { unary_scalar(self, src, value, 0, "tensor_add"); }
void THGPUTensor_mul(THGPUTensor *self, THGPUTensor *src, float value) { unary_scalar(self, src, value, 1, "tensor_mul"); }
void THGPUTensor_div(THGPUTensor *self, THGPUTensor *src, float value) { unary_scalar(self, src, value, 2, "tensor_div"); }

void THGPUTensor_cadd(THGPUTensor *self_, THGPUTensor *src1, float value, THGPUTensor *src2) {
    THGPUTensor_resizeAs(self_, src1);
    THGPU_ARGCHECK(THGPUTensor_nElement(src1) == THGPUTensor_nElement(src2), 3, "size do not match", );
    THGPUTensor *self = THGPUTensor_newContiguous(self_);
    if (self_ != src1) THGPUTensor_copy(self, src1);
    THGPUTensor *s2 = THGPUTensor_newContiguous(src2);
    if (scalar_op(THGPUTensor_data(s2), THGPUTensor_data(self), THGPUTensor_nElement(self), value, 3, "tensor_cadd"))
        raise("%s", thgpu_last_error());
    THGPUTensor_free(s2);
    THGPUTensor_freeCopyTo(self, self_);
}

void THGPUTensor_addmm(THGPUTensor *r_, float beta, THGPUTensor *t, float alpha, THGPUTensor *m1, THGPUTensor *m2) {
    if (m1->nDimension != 2 || m2->nDimension != 2) {
        raise("matrix and matrix expected");
        return;
    }
    if (t->nDimension != 2 || t->size[0] != m1->size[0] || t->size[1] != m2->size[1] || m1->size[1] != m2->size[0]) {
        raise("size mismatch");
        return;
    }
    if (t != r_) {
        THGPUTensor_resizeAs(r_, t);
        THGPUTensor_copy(r_, t);
    }
    // In column-major terms the result is used as it lies when its first
    // dimension is contiguous; when its second is, the product is formed
    // transposed (operands swapped); otherwise through a dense transposed copy.
    char tr;
    THGPUTensor *r__;
    if (r_->stride[0] == 1 && r_->stride[1] != 0) {
        tr = 'n';
        r__ = r_;
    } else if (r_->stride[1] == 1 && r_->stride[0] != 0) {
        THGPUTensor *swap = m2;
        m2 = m1;
        m1 = swap;
        tr = 't';
        r__ = r_;
    } else {
        tr = 'n';
        THGPUTensor *dense = THGPUTensor_newWithSize2d(r_->size[1], r_->size[0]);
        r__ = THGPUTensor_newTranspose(dense, 0, 1);  // shape of r_, first dimension contiguous
        THGPUTensor_free(dense);
        THGPUTensor_copy(r__, r_);
    }
    const int d0 = tr == 'n' ? 0 : 1, d1 = tr == 'n' ? 1 : 0;
    char t1, t2;
    THGPUTensor *m1_, *m2_;
    if (m1->stride[d0] == 1 && m1->stride[d1] != 0) {
        t1 = 'n';
        m1_ = m1;
    } else if (m1->stride[d1] == 1 && m1->stride[d0] != 0) {
        t1 = 't';
        m1_ = m1;
    } else {
        t1 = tr == 'n' ? 't' : 'n';
        m1_ = THGPUTensor_newClone(m1);
    }
    if (m2->stride[d0] == 1 && m2->stride[d1] != 0) {
        t2 = 'n';
        m2_ = m2;
    } else if (m2->stride[d1] == 1 && m2->stride[d0] != 0) {
        t2 = 't';
        m2_ = m2;
    } else {
        t2 = tr == 'n' ? 't' : 'n';
        m2_ = THGPUTensor_newClone(m2);
    }
    const long mm = r__->size[d0], nn = r__->size[d1], kk = m1_->size[d1];
    THGPUBlas_gemm(t1, t2, mm, nn, kk, alpha, THGPUTensor_data(m1_), t1 == 'n' ? m1_->stride[d1] : m1_->stride[d0],
                   THGPUTensor_data(m2_), t2 == 'n' ? m2_->stride[d1] : m2_->stride[d0], beta, THGPUTensor_data(r__),
                   r__->stride[d1]);
    if (m1_ != m1) THGPUTensor_free(m1_);
    if (m2_ != m2) THGPUTensor_free(m2_);
    if (r__ != r_) THGPUTensor_freeCopyTo(r__, r_);
}

void THGPUTensor_addmv(THGPUTensor *r_, float beta, THGPUTensor *t, float alpha, THGPUTensor *mat, THGPUTensor *vec) {
    if (mat->nDimension != 2 || vec->nDimension != 1) {
        raise("matrix and vector expected");
        return;
    }
    if (mat->size[1] != vec->size[0] || t->nDimension != 1 || t->size[0] != mat->size[0]) {
        raise("size mismatch");
        return;
    }
    if (r_ != t) {
        THGPUTensor_resizeAs(r_, t);
        THGPUTensor_copy(r_, t);
    }
    // y = beta*y + alpha*op(A)*x as a GEMM with one column; x and y must be dense for that.
    THGPUTensor *x = THGPUTensor_newContiguous(vec);
    THGPUTensor *y = THGPUTensor_newContiguous(r_);
    THGPUTensor *a = mat;
    char ta;
    long lda;
    if (mat->stride[0] == 1 && mat->stride[1] != 0) {
        ta = 'n';
        lda = mat->stride[1];
    } else if (mat->stride[1] == 1 && mat->stride[0] != 0) {
        ta = 't';
        lda = mat->stride[0];
    } else {
        a = THGPUTensor_newClone(mat);  // row-major dense: the transposed case
        ta = 't';
        lda = a->stride[0];
    }
    THGPUBlas_gemm(ta, 'n', mat->size[0], 1, mat->size[1], alpha, THGPUTensor_data(a), lda, THGPUTensor_data(x),
                   mat->size[1], beta, THGPUTensor_data(y), mat->size[0]);
    if (a != mat) THGPUTensor_free(a);
    THGPUTensor_free(x);
    THGPUTensor_freeCopyTo(y, r_);
}

void THGPUTensor_addr(THGPUTensor *r_, float beta, THGPUTensor *t, float alpha, THGPUTensor *vec1, THGPUTensor *vec2) {
    if (vec1->nDimension != 1 || vec2->nDimension != 1) {
        raise("vector and vector expected");
        return;
    }
    if (t->nDimension != 2 || t->size[0] != vec1->size[0] || t->size[1] != vec2->size[0]) {
        raise("size mismatch");
        return;
    }
    if (r_ != t) {
        THGPUTensor_resizeAs(r_, t);
        THGPUTensor_copy(r_, t);
    }
    // r = beta*r + alpha * vec1 (x) vec2: a GEMM with a reduction of length one on a dense row-major r.
    THGPUTensor *r = THGPUTensor_newContiguous(r_);
    THGPUTensor *x = THGPUTensor_newContiguous(vec1);
    THGPUTensor *y = THGPUTensor_newContiguous(vec2);
    const long m = vec1->size[0], n = vec2->size[0];
    // column-major view of row-major r is n x m: r'(j, i) = alpha * y(j) * x(i)
    THGPUBlas_gemm('n', 't', n, m, 1, alpha, THGPUTensor_data(y), n, THGPUTensor_data(x), m, beta, THGPUTensor_data(r),
                   n);
    THGPUTensor_free(x);
    THGPUTensor_free(y);
    THGPUTensor_freeCopyTo(r, r_);
}

// gputorch/lib/THC/THCTensorMath.cpp:269-280 (a Bolt inner product there).  Blocking: the value goes to the host.
float THGPUTensor_dot(THGPUTensor *self, THGPUTensor *src) {
    if (!self || !src) {
        raise("THGPUTensor_dot: null tensor");
        return 0.0f;
    }
    const long n = THGPUTensor_nElement(self);
    THGPU_ARGCHECK(n == THGPUTensor_nElement(src), 2, "size do not match", 0.0f);
    if (n == 0) return 0.0f;
    hipStream_t st = stream();
    if (!st) {
        raise("%s", thgpu_last_error());
        return 0.0f;
    }
    THGPUTensor *a = THGPUTensor_newContiguous(self);
    THGPUTensor *b = THGPUTensor_newContiguous(src);
    float result = 0.0f;
    long parts = (n + 4095) / 4096;
    if (parts > 1024) parts = 1024;
    const long chunk = (n + parts - 1) / parts;
    parts = (n + chunk - 1) / chunk;
    float *ws = a && b && tensor_backed(a) && tensor_backed(b) ? workspace(sizeof(float) * (size_t)(parts + 1)) : nullptr;
    if (ws) {
        {
            LaunchScope scope("dot", 2.0 * n, 8.0 * n);
            hipLaunchKernelGGL(dot_partial_kernel, dim3((unsigned)parts), dim3(256), 0, st, THGPUTensor_data(a),
                               THGPUTensor_data(b), n, chunk, ws);
            hipLaunchKernelGGL(dot_final_kernel, dim3(1), dim3(256), 0, st, ws, (int)parts, ws + parts);
        }
        if (check_launch("dot") || copy_d2h(&result, ws + parts, 1)) raise("%s", thgpu_last_error());
    } else {
        raise("THGPUTensor_dot: %s", a && b ? thgpu_last_error() : "could not make the operands contiguous");
    }
    if (a) THGPUTensor_free(a);
    if (b) THGPUTensor_free(b);
    return result;
}

// Index operations along one dimension with a host vector of 1-based indices, slice by slice like
// TH/generic/THTensorMath.c:69-176 (the reference's kernels: gputorch/lib/THC/THCTensorMath.cpp:1331-1465).
void THGPUTensor_indexSelect(THGPUTensor *res_, THGPUTensor *src, int dim, THLongTensor *index) {
    if (!res_ || !src || !index) return raise("THGPUTensor_indexSelect: null tensor");
    THGPU_ARGCHECK(index->nDimension == 1, 3, "expecting vector of indices", );
    THGPU_ARGCHECK(src->nDimension > 0, 2, "Source tensor is empty", );
    THGPU_ARGCHECK(dim >= 0 && dim < src->nDimension, 4, "Indexing dim is out of bounds", );
    std::vector<long> idx;
    if (!host_indices(index, src->size[dim], idx, "indexSelect")) return;
    std::vector<long> size(src->size, src->size + src->nDimension);
    size[(size_t)dim] = (long)idx.size();
    THLongStorage sz;
    sz.data = size.data();
    sz.size = (long)size.size();
    THGPUTensor_resize(res_, &sz, nullptr);
    for (size_t k = 0; k < idx.size(); ++k) {
        THGPUTensor *d = THGPUTensor_newNarrow(res_, dim, (long)k, 1);
        THGPUTensor *s = THGPUTensor_newNarrow(src, dim, idx[k], 1);
        if (d && s) THGPUTensor_copy(d, s);
        if (d) THGPUTensor_free(d);
        if (s) THGPUTensor_free(s);
    }
}

void THGPUTensor_indexCopy(THGPUTensor *res_, int dim, THLongTensor *index, THGPUTensor *src) {
    if (!res_ || !src || !index) return raise("THGPUTensor_indexCopy: null tensor");
    THGPU_ARGCHECK(index->nDimension == 1, 3, "expecting vector of indices", );
    THGPU_ARGCHECK(src->nDimension > 0, 2, "Source tensor is empty", );
    THGPU_ARGCHECK(dim >= 0 && dim < src->nDimension && dim < res_->nDimension, 4, "Indexing dim is out of bounds", );
    THGPU_ARGCHECK(index->size[0] == src->size[dim], 4, "length of src.size[dim] is not equal to length of indices", );
    std::vector<long> idx;
    if (!host_indices(index, res_->size[dim], idx, "indexCopy")) return;
    for (size_t k = 0; k < idx.size(); ++k) {
        THGPUTensor *d = THGPUTensor_newNarrow(res_, dim, idx[k], 1);
        THGPUTensor *s = THGPUTensor_newNarrow(src, dim, (long)k, 1);
        if (d && s) THGPUTensor_copy(d, s);
        if (d) THGPUTensor_free(d);
        if (s) THGPUTensor_free(s);
    }
}

void THGPUTensor_indexFill(THGPUTensor *res_, int dim, THLongTensor *index, float val) {
    if (!res_ || !index) return raise("THGPUTensor_indexFill: null tensor");
    THGPU_ARGCHECK(index->nDimension == 1, 3, "Index is supposed to be a vector", );
    THGPU_ARGCHECK(res_->nDimension > 0, 2, "Source tensor is empty", );
    THGPU_ARGCHECK(dim >= 0 && dim < res_->nDimension, 4, "Indexing dim is out of bounds", );
    std::vector<long> idx;
    if (!host_indices(index, res_->size[dim], idx, "indexFill")) return;
    for (size_t k = 0; k < idx.size(); ++k) {
        THGPUTensor *d = THGPUTensor_newNarrow(res_, dim, idx[k], 1);
        if (d) {
            THGPUTensor_fill(d, val);
            THGPUTensor_free(d);
        }
    }
}

}  // extern "C"
