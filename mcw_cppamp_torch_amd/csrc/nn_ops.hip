// Operator entry points on THGPUTensor arguments: nn.SpatialConvolutionMM,
// nn.SpatialMaxPooling, nn.Threshold.  These are what the luaT bindings of the
// reference do after unpacking the module table
// (gputorch/lib/THC/gpunn-impl/SpatialConvolutionMM.cpp:110-429,
//  SpatialMaxPooling.cpp:205-383, Threshold.cpp:16-81): check shapes, resize
// the module's buffers, launch.  One launch per kernel for the whole batch
// instead of the reference's per-image loops.
#include "gemm_mfma.h"
#include "kernels.h"

#include <map>

using namespace thgpu;

namespace {

struct ConvShape {
    long B;
    int C, H, W, M, K, Ho, Wo;
    long N;
    bool batched;
};

// Common argument checks.  Messages follow the reference's luaL_argcheck /
// THArgCheck texts where it has one.
int conv_shape(ConvShape &s, const THGPUTensor *input, const THGPUTensor *weight, int kW, int kH, int dW, int dH,
               int padW, int padH) {
    if (!input || !weight) return fail("SpatialConvolutionMM: null tensor");
    if (!(input->nDimension == 3 || input->nDimension == 4)) return fail("3D or 4D (batch mode) tensor is expected");
    if (kW <= 0 || kH <= 0 || dW <= 0 || dH <= 0 || padW < 0 || padH < 0)
        return fail("SpatialConvolutionMM: invalid kernel/stride/padding");
    if (weight->nDimension != 2) return fail("SpatialConvolutionMM: weight must be 2D [nOutputPlane, nInputPlane*kH*kW]");
    s.batched = input->nDimension == 4;
    const int o = s.batched ? 1 : 0;
    s.B = s.batched ? input->size[0] : 1;
    s.C = (int)input->size[o];
    s.H = (int)input->size[o + 1];
    s.W = (int)input->size[o + 2];
    s.M = (int)weight->size[0];
    s.K = s.C * kH * kW;
    if (weight->size[1] != s.K) return fail("input channels and nInputPlane dont match");
    if (s.H + 2 * padH < kH || s.W + 2 * padW < kW) return fail("SpatialConvolutionMM: input image smaller than kernel size");
    s.Ho = (s.H + 2 * padH - kH) / dH + 1;
    s.Wo = (s.W + 2 * padW - kW) / dW + 1;
    s.N = (long)s.Ho * s.Wo;
    if (s.B * s.N >= (1L << 31)) return fail("SpatialConvolutionMM: batch*outputHeight*outputWidth exceeds 2^31");
    return 0;
}

int require_contiguous(const THGPUTensor *t, const char *what) {
    if (!THGPUTensor_isContiguous(t)) return fail("SpatialConvolutionMM: %s must be contiguous", what);
    return 0;
}

int check_grad_output(const ConvShape &s, const THGPUTensor *gradOutput) {
    if (gradOutput->nDimension != (s.batched ? 4 : 3))
        return fail("SpatialConvolutionMM: gradOutput must have as many dimensions as the output");
    const int o = s.batched ? 1 : 0;
    if (gradOutput->size[o] != s.M) return fail("Number of output features is not equal to nOutputPlane");
    if ((s.batched && gradOutput->size[0] != s.B) || gradOutput->size[o + 1] != s.Ho || gradOutput->size[o + 2] != s.Wo)
        return fail("SpatialConvolutionMM: gradOutput size does not match the output size");
    return 0;
}

// Device pointer of element 0; tensors that reach a kernel are contiguous.
inline float *dptr(const THGPUTensor *t) { return THGPUTensor_data(t); }

// The padded input a module keeps in finput when it runs without the column buffer:
// [B,] C, H + 2 padH, W + 2 padW.
bool is_padded(const THGPUTensor *t, const ConvShape &s, int padH, int padW) {
    const int o = s.batched ? 1 : 0;
    return t->nDimension == 3 + o && (!s.batched || t->size[0] == s.B) && t->size[o] == s.C &&
           t->size[o + 1] == s.H + 2 * padH && t->size[o + 2] == s.W + 2 * padW && THGPUTensor_isContiguous(t);
}
// The forward's columns: [B,] K, N.
bool is_columns(const THGPUTensor *t, const ConvShape &s) {
    const int o = s.batched ? 1 : 0;
    return t->nDimension == 2 + o && (!s.batched || t->size[0] == s.B) && t->size[o] == s.K && t->size[o + 1] == s.N &&
           THGPUTensor_isContiguous(t);
}
bool g_finput_reuse = false;

int size_padded(THGPUTensor *t, const ConvShape &s, int padH, int padW) {
    if (s.batched)
        THGPUTensor_resize4d(t, s.B, s.C, s.H + 2 * padH, s.W + 2 * padW);
    else
        THGPUTensor_resize3d(t, s.C, s.H + 2 * padH, s.W + 2 * padW);
    if (!is_padded(t, s, padH, padW) || !tensor_backed(t)) return fail("SpatialConvolutionMM: could not size finput");
    return 0;
}

// An image tensor ([B,] C, H, W) whose rows are contiguous and whose planes follow each other at one fixed distance:
// the dense layout (pitch == W, plane == H*W) or the interior of a larger buffer, e.g. one with a zero border.
struct PlaneLayout {
    long pitch = 0;  // floats between rows
    long plane = 0;  // floats between planes; images are C planes apart
    bool dense = false;
};

bool plane_layout(const THGPUTensor *t, PlaneLayout &l) {
    if (!t || !(t->nDimension == 3 || t->nDimension == 4)) return false;
    const int o = t->nDimension == 4 ? 1 : 0;
    const long C = t->size[o], H = t->size[o + 1], W = t->size[o + 2];
    if (C <= 0 || H <= 0 || W <= 0) return false;
    if (W > 1 && t->stride[o + 2] != 1) return false;
    l.pitch = H > 1 ? t->stride[o + 1] : W;
    l.plane = C > 1 || o == 1 ? t->stride[o] : H * l.pitch;
    if (C == 1 && o == 1 && t->size[0] > 1) l.plane = t->stride[0];  // single-plane images: the image stride is the plane's
    if (l.pitch < W || l.plane < (H - 1) * l.pitch + W) return false;
    if (o == 1 && t->size[0] > 1 && t->stride[0] != C * l.plane) return false;
    l.dense = l.pitch == W && l.plane == H * W;
    return tensor_backed(t);
}

// Whether `input` lies inside a buffer that keeps padH rows above and below and padW columns left and right of
// every plane (the caller vouches for the zeros in them): then the buffer itself is the padded image.
bool interior_of_padded(const THGPUTensor *input, const ConvShape &s, int padH, int padW, PlaneLayout &l) {
    if (!plane_layout(input, l)) return false;
    const long Hp = s.H + 2L * padH, Wp = s.W + 2L * padW;
    if (l.pitch != Wp || l.plane != Hp * Wp) return false;
    const long lead = (long)padH * Wp + padW;  // from the buffer's first element to the interior's
    return input->storageOffset >= lead && input->storageOffset - lead + s.B * s.C * l.plane <= input->storage->size;
}

void set_output_layout(GemmProblem &p, const PlaneLayout &l, int planes_per_image, int width) {
    p.sC = l.plane;
    p.bsC = (long)planes_per_image * l.plane;
    if (!l.dense) {
        p.c_pitch = (int)l.pitch;
        p.c_w = width;
    }
}

// ---- gradOutput delivered in the padded layout of the gathered gradInput product ("the twin") --------------------
// Geometry of that layout for one layer, and the buffers (by device address of fgradInput's first element) whose
// padded region is known to have zero borders: zeroed here, or written whole by the padding kernel.  A buffer leaves
// the list when its memory is released (conv_forget_buffer) or when another route writes something else into it.
struct TwinGeom {
    long B;
    int M, Ho, Wo, top, left, Hq, Wq;
    bool operator==(const TwinGeom &o) const {
        return B == o.B && M == o.M && Ho == o.Ho && Wo == o.Wo && top == o.top && left == o.left && Hq == o.Hq &&
               Wq == o.Wq;
    }
};
std::map<const float *, TwinGeom> g_zero_bordered;

TwinGeom twin_geom(const ConvShape &s, int kH, int kW, int padH, int padW, int dH, int dW) {
    TwinGeom t;
    t.B = s.B;
    t.M = s.M;
    t.Ho = s.Ho;
    t.Wo = s.Wo;
    conv_implicit_q_layout(s.C, s.H, s.W, kH, kW, padH, padW, dH, dW, &t.top, &t.left, &t.Hq, &t.Wq);
    return t;
}

bool zero_bordered(const float *q, const TwinGeom &t) {
    auto it = g_zero_bordered.find(q);
    return it != g_zero_bordered.end() && it->second == t;
}

// `twin` as a kernel operand when it is a usable second copy of a [B,] C, H, W result: same sizes, rows contiguous,
// planes evenly spaced, memory behind it, and no overlap with the result itself.
bool twin_output(const THGPUTensor *twin, const THGPUTensor *like, TwinOutput &out) {
    PlaneLayout l;
    if (!twin || !like || twin->nDimension != like->nDimension || !plane_layout(twin, l)) return false;
    for (int d = 0; d < like->nDimension; ++d)
        if (twin->size[d] != like->size[d]) return false;
    if (twin->storage == like->storage) return false;
    out.base = THGPUTensor_data(twin);
    out.plane = l.plane;
    out.pitch = (int)l.pitch;
    return true;
}

// Whether `twin` is the view thgpu_SpatialConvolutionMM_gradOutputTwin hands out into a buffer that is on record as
// zero-bordered: then the floats between its rows are zeros that a producer may store again along with the rows.
bool twin_rows_in_zero_border(const THGPUTensor *twin, const TwinOutput &out) {
    const int o = twin->nDimension == 4 ? 1 : 0;
    for (const auto &kv : g_zero_bordered) {
        const TwinGeom &t = kv.second;
        if (kv.first + (long)t.top * t.Wq + t.left == out.base && t.Wq == out.pitch && (long)t.Hq * t.Wq == out.plane &&
            twin->size[o] == t.M && twin->size[o + 1] == t.Ho && twin->size[o + 2] == t.Wo &&
            (o ? twin->size[0] : 1) == t.B)
            return true;
    }
    return false;
}

int conv_update_output(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias, THGPUTensor *finput,
                       THGPUTensor *fgradInput, THGPUTensor *output, int kW, int kH, int dW, int dH, int padW,
                       int padH, OutputThreshold act, bool input_in_padded_buffer) {
    (void)fgradInput;  // the reference uses it as a buffer of ones for the bias GEMM; the bias is fused here
    ConvShape s;
    if (conv_shape(s, input, weight, kW, kH, dW, dH, padW, padH)) return 1;
    if (!bias || !finput || !output) return fail("SpatialConvolutionMM: null tensor");
    if (THGPUTensor_nElement(bias) != s.M) return fail("SpatialConvolutionMM: bias must have nOutputPlane elements");
    if (require_contiguous(weight, "weight") || require_contiguous(bias, "bias")) return 1;
    PlaneLayout in_layout;
    if (input_in_padded_buffer && !interior_of_padded(input, s, padH, padW, in_layout))
        return fail("SpatialConvolutionMM: input is not the interior of a buffer padded by %d x %d", padH, padW);

    const bool gathered = conv_use_gathered(s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW);
    const bool direct = gathered && input_in_padded_buffer;  // the input's own buffer is the padded image
    THGPUTensor *in = direct ? nullptr : THGPUTensor_newContiguous(input);
    if (!direct && !in) return 1;
    struct Release {
        THGPUTensor *t;
        ~Release() {
            if (t) THGPUTensor_free(t);
        }
    } release{in};

    if (direct) {
        // finput is not needed: nothing is copied
    } else if (gathered) {
        // finput holds the padded input instead of the columns
        if (size_padded(finput, s, padH, padW)) return 1;
    } else if (s.batched) {
        THGPUTensor_resize3d(finput, s.B, s.K, s.N);
    } else {
        THGPUTensor_resize2d(finput, s.K, s.N);
    }
    // The output keeps the layout it comes with when it already has the right sizes: densely packed, or rows inside
    // a larger buffer (the next layer's padded input).
    if (s.batched)
        THGPUTensor_resize4d(output, s.B, s.M, s.Ho, s.Wo);
    else
        THGPUTensor_resize3d(output, s.M, s.Ho, s.Wo);
    PlaneLayout out_layout;
    if (!plane_layout(output, out_layout) || THGPUTensor_nElement(output) != s.B * s.M * s.N)
        return fail("SpatialConvolutionMM: could not size output");
    if (!direct && !tensor_ready(finput, gathered ? s.B * s.C * (s.H + 2L * padH) * (s.W + 2L * padW) : s.B * s.K * s.N))
        return fail("SpatialConvolutionMM: could not size finput");
    if (!((direct || tensor_backed(in)) && tensor_backed(weight) && tensor_backed(bias)))
        return fail("SpatialConvolutionMM: a tensor's shape exceeds its storage");

    if (gathered) {
        const float *padded = direct ? dptr(input) - ((long)padH * in_layout.pitch + padW) : dptr(finput);
        if (!direct && pad_planes_launch(dptr(in), s.B * s.C, s.H, s.W, padH, padW, dptr(finput))) return 1;
        OutputLayout ol;
        ol.plane = out_layout.plane;
        ol.pitch = out_layout.dense ? 0 : (int)out_layout.pitch;
        return conv_implicit_forward(padded, dptr(weight), dptr(bias), dptr(output), s.B, s.C, s.H, s.W, s.M, kH, kW,
                                     padH, padW, dH, dW, act, ol);
    }
    if (im2col_launch(dptr(in), s.B, s.C, s.H, s.W, kH, kW, padH, padW, dH, dW, dptr(finput))) return 1;
    // output[b][m][n] = bias[m] + sum_k weight[m][k] * finput[b][k][n]
    GemmProblem p;
    p.A = dptr(weight);
    p.a_rc = true;
    p.sA = s.K;
    p.B = dptr(finput);
    p.b_rc = false;
    p.sB = s.N;
    p.bsB = (long)s.K * s.N;
    p.C = dptr(output);
    set_output_layout(p, out_layout, s.M, s.Wo);
    p.bias = dptr(bias);
    p.M = s.M;
    p.J = (int)(s.B * s.N);
    p.N = (int)s.N;
    p.R = s.K;
    p.tag = "gemm_conv_fwd";
    p.flops = 2.0 * s.M * (double)s.N * s.K * s.B;
    p.act = act.on;
    p.act_threshold = act.threshold;
    p.act_value = act.value;
    return gemm_launch(p);
}

// mask_on: gradInput is zeroed where `input` does not exceed mask_threshold.
// twin_ready: the caller says that gradOutput's producer also wrote it into fgradInput through the view
// thgpu_SpatialConvolutionMM_gradOutputTwin handed out (honoured only while the buffer is known to be zero-bordered
// for this geometry; otherwise the padded copy is made as usual).  twin: a second copy of gradInput to keep, or null;
// *wrote_twin says whether it was stored.
int conv_update_grad_input(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight, THGPUTensor *finput,
                           THGPUTensor *fgradInput, THGPUTensor *gradInput, int kW, int kH, int dW, int dH,
                           int padW, int padH, bool mask_on, float mask_threshold, bool twin_ready = false,
                           THGPUTensor *twin = nullptr, int *wrote_twin = nullptr) {
    if (wrote_twin) *wrote_twin = 0;
    (void)finput;
    ConvShape s;
    if (conv_shape(s, input, weight, kW, kH, dW, dH, padW, padH)) return 1;
    if (!gradOutput || !fgradInput || !gradInput) return fail("SpatialConvolutionMM: null tensor");
    if (check_grad_output(s, gradOutput)) return 1;
    if (require_contiguous(weight, "weight")) return 1;
    const bool gathered = conv_use_gathered_gradinput(s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW);
    THGPUTensor *go = THGPUTensor_newContiguous(gradOutput);
    if (!go) return 1;
    // The mask is `input`, read element for element beside gradInput.  The gathered product's store takes it in
    // any regular plane layout (dense, or the interior of a padded buffer); col2im wants it dense.
    PlaneLayout mask_layout;
    THGPUTensor *in = nullptr;
    InputMask mask;
    if (mask_on) {
        // (the strided layers' scattered store reads a dense mask only)
        if (gathered && plane_layout(input, mask_layout) && ((dH == 1 && dW == 1) || mask_layout.dense)) {
            mask.in = dptr(input);
        } else {
            in = THGPUTensor_newContiguous(input);
            if (!in || !plane_layout(in, mask_layout)) {
                if (in) THGPUTensor_free(in);
                THGPUTensor_free(go);
                return fail("SpatialConvolutionMM: input is not usable as a mask");
            }
            mask.in = dptr(in);
        }
        mask.threshold = mask_threshold;
        mask.plane = mask_layout.plane;
        mask.pitch = mask_layout.dense ? 0 : (int)mask_layout.pitch;
    }
    struct Release {  // frees the contiguous copies on every return path
        THGPUTensor *a, *b;
        ~Release() {
            if (a) THGPUTensor_free(a);
            if (b) THGPUTensor_free(b);
        }
    } release{go, in};

    if (gathered) {
        // fgradInput holds the padded gradOutput and the flipped kernels instead of the gradient columns
        const long need = conv_implicit_gradinput_scratch(s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW);
        if (s.batched)
            THGPUTensor_resize4d(gradInput, s.B, s.C, s.H, s.W);
        else
            THGPUTensor_resize3d(gradInput, s.C, s.H, s.W);
        // a delivered gradOutput is only trusted in the buffer it was handed out in: same memory, same geometry
        const TwinGeom tg = twin_geom(s, kH, kW, padH, padW, dH, dW);
        const bool q_ready = twin_ready && tensor_ready(fgradInput, need) && zero_bordered(dptr(fgradInput), tg);
        THGPUTensor_resize1d(fgradInput, need);
        if (!tensor_ready(fgradInput, need) || !tensor_ready(gradInput, s.B * (long)s.C * s.H * s.W))
            return fail("SpatialConvolutionMM: could not size gradInput/fgradInput");
        if (!(tensor_backed(go) && tensor_backed(weight)))
            return fail("SpatialConvolutionMM: a tensor's shape exceeds its storage");
        TwinOutput second;
        if (twin && !twin_output(twin, gradInput, second)) second = TwinOutput();
        bool wrote = false;
        const int rc = conv_implicit_gradinput(dptr(go), dptr(weight), dptr(fgradInput), dptr(gradInput), s.B, s.C, s.H,
                                               s.W, s.M, kH, kW, padH, padW, dH, dW, mask, q_ready, second, &wrote);
        // either way the padded region now holds this gradOutput between zero borders
        if (!rc) g_zero_bordered[dptr(fgradInput)] = tg;
        if (wrote_twin) *wrote_twin = !rc && wrote ? 1 : 0;
        return rc;
    }
    g_zero_bordered.erase(dptr(fgradInput));  // the gradient columns go there instead
    if (s.batched) {
        THGPUTensor_resize4d(gradInput, s.B, s.C, s.H, s.W);
        THGPUTensor_resize3d(fgradInput, s.B, s.K, s.N);
    } else {
        THGPUTensor_resize3d(gradInput, s.C, s.H, s.W);
        THGPUTensor_resize2d(fgradInput, s.K, s.N);
    }
    if (!tensor_ready(fgradInput, s.B * s.K * s.N) || !tensor_ready(gradInput, s.B * (long)s.C * s.H * s.W))
        return fail("SpatialConvolutionMM: could not size gradInput/fgradInput");
    if (!(tensor_backed(go) && tensor_backed(weight)))
        return fail("SpatialConvolutionMM: a tensor's shape exceeds its storage");
    g_zero_bordered.erase(dptr(fgradInput));
    {
        // fgradInput[b][k][n] = sum_m weight[m][k] * gradOutput[b][m][n]
        GemmProblem p;
        p.A = dptr(weight);
        p.a_rc = false;  // A(i = k, r = m) = weight[m][k]: contiguous along i
        p.sA = s.K;
        p.B = dptr(go);
        p.b_rc = false;
        p.sB = s.N;
        p.bsB = (long)s.M * s.N;
        p.C = dptr(fgradInput);
        p.sC = s.N;
        p.bsC = (long)s.K * s.N;
        p.M = s.K;
        p.J = (int)(s.B * s.N);
        p.N = (int)s.N;
        p.R = s.M;
        p.tag = "gemm_conv_gradinput";
        p.flops = 2.0 * s.M * (double)s.N * s.K * s.B;
        if (gemm_launch(p)) return 1;
    }
    return col2im_launch(dptr(fgradInput), s.B, s.C, s.H, s.W, kH, kW, padH, padW, dH, dW, dptr(gradInput), mask);
}

int conv_acc_grad_parameters(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradWeight,
                             THGPUTensor *gradBias, THGPUTensor *finput, THGPUTensor *fgradInput, int kW, int kH, int dW,
                             int dH, int padW, int padH, float scale, bool input_in_padded_buffer) {
    (void)fgradInput;
    ConvShape s;
    if (!gradWeight || !gradBias || !finput || !gradOutput) return fail("SpatialConvolutionMM: null tensor");
    if (conv_shape(s, input, gradWeight, kW, kH, dW, dH, padW, padH)) return 1;
    if (check_grad_output(s, gradOutput)) return 1;
    if (THGPUTensor_nElement(gradBias) != s.M) return fail("SpatialConvolutionMM: gradBias must have nOutputPlane elements");
    if (require_contiguous(gradWeight, "gradWeight") || require_contiguous(gradBias, "gradBias")) return 1;
    PlaneLayout in_layout;
    if (input_in_padded_buffer && !interior_of_padded(input, s, padH, padW, in_layout))
        return fail("SpatialConvolutionMM: input is not the interior of a buffer padded by %d x %d", padH, padW);
    const bool gathered = conv_use_gathered(s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW);
    const bool direct = gathered && input_in_padded_buffer;
    THGPUTensor *go = THGPUTensor_newContiguous(gradOutput);
    if (!go) return 1;
    THGPUTensor *in = direct ? nullptr : THGPUTensor_newContiguous(input);
    if (!direct && !in) {
        THGPUTensor_free(go);
        return 1;
    }
    struct Release {
        THGPUTensor *a, *b;
        ~Release() {
            if (a) THGPUTensor_free(a);
            if (b) THGPUTensor_free(b);
        }
    } release{go, in};
    if (!((direct || tensor_backed(in)) && tensor_backed(go) && tensor_backed(gradWeight) && tensor_backed(gradBias)))
        return fail("SpatialConvolutionMM: a tensor's shape exceeds its storage");
    // finput is rebuilt from `input` on every call, as the reference GPU code does
    // (gpunn-impl/SpatialConvolutionMM.cpp:388-396): the result then depends on the arguments alone,
    // whatever input the last forward pass saw and whoever else shares the buffer.  With
    // thgpu_conv_set_finput_reuse(1) a finput of the right shape is taken to be the forward's, as the CPU
    // module takes it (mcw_nn/generic/SpatialConvolutionMM.c:318,336).  An input that lies in its own padded
    // buffer needs neither: the gathered product reads it there.
    const bool reuse = g_finput_reuse;
    if (gathered) {
        const float *padded;
        if (direct) {
            padded = dptr(input) - ((long)padH * in_layout.pitch + padW);
        } else {
            if (!(reuse && is_padded(finput, s, padH, padW) && tensor_backed(finput))) {
                if (size_padded(finput, s, padH, padW)) return 1;
                if (pad_planes_launch(dptr(in), s.B * s.C, s.H, s.W, padH, padW, dptr(finput))) return 1;
            }
            padded = dptr(finput);
        }
        // The bias gradient is the row sums of the product's first operand: the GEMM computes them on the side
        // when it runs a tiled reduction-batched kernel; otherwise the two-stage sum does.
        bool bias_done = false;
        if (conv_implicit_gradweight(padded, dptr(go), dptr(gradWeight), s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH,
                                     dW, scale, tuning().gradbias_separate ? nullptr : dptr(gradBias), &bias_done))
            return 1;
        return bias_done ? 0 : gradbias_launch(dptr(go), dptr(gradBias), s.B, s.M, s.N, scale);
    }
    if (!(reuse && is_columns(finput, s) && tensor_backed(finput))) {
        if (s.batched)
            THGPUTensor_resize3d(finput, s.B, s.K, s.N);
        else
            THGPUTensor_resize2d(finput, s.K, s.N);
        if (!tensor_ready(finput, s.B * s.K * s.N)) return fail("SpatialConvolutionMM: could not size finput");
        if (im2col_launch(dptr(in), s.B, s.C, s.H, s.W, kH, kW, padH, padW, dH, dW, dptr(finput))) return 1;
    }
    bool bias_done = false;
    {
        // gradWeight[m][k] += scale * sum_b sum_n gradOutput[b][m][n] * finput[b][k][n]
        GemmProblem p;
        p.A = dptr(go);
        p.a_rc = true;
        p.sA = s.N;
        p.rbA = (long)s.M * s.N;
        p.B = dptr(finput);
        p.b_rc = true;
        p.sB = s.N;
        p.rbB = (long)s.K * s.N;
        p.C = dptr(gradWeight);
        p.sC = s.K;
        p.M = s.M;
        p.J = s.K;
        p.N = s.K;
        p.R = (int)s.N;
        p.nb = (int)s.B;
        p.alpha = scale;
        p.beta = 1.0f;
        p.tag = "gemm_conv_gradweight";
        p.flops = 2.0 * s.M * (double)s.N * s.K * s.B;
        p.rowsum = tuning().gradbias_separate ? nullptr : dptr(gradBias);
        p.rowsum_done = &bias_done;
        if (gemm_launch(p)) return 1;
    }
    return bias_done ? 0 : gradbias_launch(dptr(go), dptr(gradBias), s.B, s.M, s.N, scale);
}

}  // namespace

namespace thgpu {
void conv_forget_buffer(const float *p) {
    if (!g_zero_bordered.empty()) g_zero_bordered.erase(p);
}
}  // namespace thgpu

extern "C" {

int thgpu_SpatialConvolutionMM_updateOutput(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
                                            THGPUTensor *finput, THGPUTensor *fgradInput, THGPUTensor *output,
                                            int kW, int kH, int dW, int dH, int padW, int padH) {
    return conv_update_output(input, weight, bias, finput, fgradInput, output, kW, kH, dW, dH, padW, padH,
                              OutputThreshold(), false);
}

int thgpu_SpatialConvolutionMM_updateOutputFused(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
                                                 THGPUTensor *finput, THGPUTensor *fgradInput, THGPUTensor *output,
                                                 int kW, int kH, int dW, int dH, int padW, int padH, int flags,
                                                 float threshold, float val) {
    if (flags & ~(THGPU_FUSE_THRESHOLD | THGPU_INPUT_IN_PADDED_BUFFER)) return fail("SpatialConvolutionMM: unknown flags");
    OutputThreshold act;
    act.on = (flags & THGPU_FUSE_THRESHOLD) != 0;
    act.threshold = threshold;
    act.value = val;
    return conv_update_output(input, weight, bias, finput, fgradInput, output, kW, kH, dW, dH, padW, padH, act,
                              (flags & THGPU_INPUT_IN_PADDED_BUFFER) != 0);
}

int thgpu_SpatialConvolutionMM_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                               THGPUTensor *finput, THGPUTensor *fgradInput,
                                               THGPUTensor *gradInput, int kW, int kH, int dW, int dH, int padW,
                                               int padH) {
    return conv_update_grad_input(input, gradOutput, weight, finput, fgradInput, gradInput, kW, kH, dW, dH, padW,
                                  padH, false, 0.0f);
}

int thgpu_SpatialConvolutionMM_updateGradInputFused(THGPUTensor *input, THGPUTensor *gradOutput,
                                                    THGPUTensor *weight, THGPUTensor *finput,
                                                    THGPUTensor *fgradInput, THGPUTensor *gradInput, int kW, int kH,
                                                    int dW, int dH, int padW, int padH, int flags, float threshold) {
    if (flags & ~THGPU_FUSE_INPUT_MASK) return fail("SpatialConvolutionMM: unknown flags");
    return conv_update_grad_input(input, gradOutput, weight, finput, fgradInput, gradInput, kW, kH, dW, dH, padW,
                                  padH, (flags & THGPU_FUSE_INPUT_MASK) != 0, threshold);
}

int thgpu_SpatialConvolutionMM_gradOutputTwin(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *fgradInput,
                                              THGPUTensor *twin, int kW, int kH, int dW, int dH, int padW, int padH,
                                              int *available) {
    if (available) *available = 0;
    ConvShape s;
    if (conv_shape(s, input, weight, kW, kH, dW, dH, padW, padH)) return 1;
    if (!fgradInput || !twin || !available) return fail("SpatialConvolutionMM: null argument");
    if (!conv_use_gathered_gradinput(s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW)) return 0;
    const long need = conv_implicit_gradinput_scratch(s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW);
    const TwinGeom tg = twin_geom(s, kH, kW, padH, padW, dH, dW);
    const long q_floats = s.B * s.M * (long)tg.Hq * tg.Wq;
    THGPUTensor_resize1d(fgradInput, need);
    if (!tensor_ready(fgradInput, need)) return fail("SpatialConvolutionMM: could not size fgradInput");
    float *q = dptr(fgradInput);
    if (!zero_bordered(q, tg)) {
        if (fill_device(q, q_floats, 0.0f)) return 1;
        g_zero_bordered[q] = tg;
    }
    // the view of gradOutput's place inside the padded planes
    const long off = fgradInput->storageOffset + (long)tg.top * tg.Wq + tg.left;
    const long plane = (long)tg.Hq * tg.Wq;
    if (s.batched)
        THGPUTensor_setStorage4d(twin, fgradInput->storage, off, s.B, s.M * plane, s.M, plane, tg.Ho, tg.Wq, tg.Wo, 1);
    else
        THGPUTensor_setStorage3d(twin, fgradInput->storage, off, s.M, plane, tg.Ho, tg.Wq, tg.Wo, 1);
    if (!tensor_backed(twin)) return fail("SpatialConvolutionMM: could not place the gradOutput view");
    // the producer's launch may as well re-order this layer's kernel bank for the product that follows
    if (require_contiguous(weight, "weight") || !tensor_backed(weight)) return 1;
    conv_implicit_offer_bank(dptr(weight), q, s.B, s.C, s.H, s.W, s.M, kH, kW, padH, padW, dH, dW);
    *available = 1;
    return 0;
}

int thgpu_SpatialConvolutionMM_updateGradInputTwin(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                                   THGPUTensor *finput, THGPUTensor *fgradInput,
                                                   THGPUTensor *gradInput, int kW, int kH, int dW, int dH, int padW,
                                                   int padH, int flags, float threshold, THGPUTensor *twin,
                                                   int *wrote_twin) {
    if (flags & ~(THGPU_FUSE_INPUT_MASK | THGPU_GRADOUTPUT_IN_TWIN)) return fail("SpatialConvolutionMM: unknown flags");
    return conv_update_grad_input(input, gradOutput, weight, finput, fgradInput, gradInput, kW, kH, dW, dH, padW, padH,
                                  (flags & THGPU_FUSE_INPUT_MASK) != 0, threshold,
                                  (flags & THGPU_GRADOUTPUT_IN_TWIN) != 0, twin, wrote_twin);
}

int thgpu_SpatialConvolutionMM_accGradParameters(THGPUTensor *input, THGPUTensor *gradOutput,
                                                 THGPUTensor *gradWeight, THGPUTensor *gradBias,
                                                 THGPUTensor *finput, THGPUTensor *fgradInput, int kW, int kH,
                                                 int dW, int dH, int padW, int padH, float scale) {
    return conv_acc_grad_parameters(input, gradOutput, gradWeight, gradBias, finput, fgradInput, kW, kH, dW, dH, padW,
                                    padH, scale, false);
}

int thgpu_SpatialConvolutionMM_accGradParametersFused(THGPUTensor *input, THGPUTensor *gradOutput,
                                                      THGPUTensor *gradWeight, THGPUTensor *gradBias,
                                                      THGPUTensor *finput, THGPUTensor *fgradInput, int kW, int kH,
                                                      int dW, int dH, int padW, int padH, float scale, int flags) {
    if (flags & ~THGPU_INPUT_IN_PADDED_BUFFER) return fail("SpatialConvolutionMM: unknown flags");
    return conv_acc_grad_parameters(input, gradOutput, gradWeight, gradBias, finput, fgradInput, kW, kH, dW, dH, padW,
                                    padH, scale, (flags & THGPU_INPUT_IN_PADDED_BUFFER) != 0);
}

int thgpu_conv_gathers(long B, int C, int H, int W, int M, int kW, int kH, int dW, int dH, int padW, int padH) {
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || M <= 0 || kW <= 0 || kH <= 0 || dW <= 0 || dH <= 0 || padW < 0 ||
        padH < 0 || H + 2 * padH < kH || W + 2 * padW < kW)
        return 0;
    return conv_use_gathered(B, C, H, W, M, kH, kW, padH, padW, dH, dW) ? 1 : 0;
}

int thgpu_SpatialMaxPooling_updateOutput(THGPUTensor *input, THGPUTensor *output, THGPUTensor *indices, int kW,
                                         int kH, int dW, int dH) {
    if (!input || !output || !indices) return fail("SpatialMaxPooling: null tensor");
    if (!(input->nDimension == 3 || input->nDimension == 4)) return fail("3D or 4D (batch) tensor expected");
    if (kW <= 0 || kH <= 0 || dW <= 0 || dH <= 0) return fail("SpatialMaxPooling: invalid kernel/stride");
    const bool batched = input->nDimension == 4;
    const int o = batched ? 1 : 0;
    const long B = batched ? input->size[0] : 1;
    const long C = input->size[o];
    const int H = (int)input->size[o + 1], W = (int)input->size[o + 2];
    if (!(W >= kW && H >= kH)) return fail("input image smaller than kernel size");
    const int Ho = (H - kH) / dH + 1, Wo = (W - kW) / dW + 1;
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    if (!in) return 1;
    if (batched) {
        THGPUTensor_resize4d(output, B, C, Ho, Wo);
        THGPUTensor_resize5d(indices, 2, B, C, Ho, Wo);
    } else {
        THGPUTensor_resize3d(output, C, Ho, Wo);
        THGPUTensor_resize4d(indices, 2, C, Ho, Wo);
    }
    // The output keeps the layout it comes with when it already has the right sizes: densely packed, or rows inside
    // a larger buffer (the next layer's padded input).
    int rc = 0;
    PlaneLayout ol;
    if (!plane_layout(output, ol) || THGPUTensor_nElement(output) != B * C * Ho * Wo ||
        !tensor_ready(indices, 2 * B * C * Ho * Wo) || !tensor_backed(in))
        rc = fail("SpatialMaxPooling: could not size output/indices");
    if (!rc)
        rc = maxpool_fwd_launch(dptr(in), B * C, H, W, kH, kW, dH, dW, dptr(output), dptr(indices), ol.plane,
                                (int)ol.pitch);
    THGPUTensor_free(in);
    return rc;
}

static int pool_update_grad_input(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                  THGPUTensor *indices, int kW, int kH, int dW, int dH, bool mask_on,
                                  float mask_threshold, THGPUTensor *twin = nullptr, int *wrote_twin = nullptr) {
    if (wrote_twin) *wrote_twin = 0;
    if (!input || !gradOutput || !gradInput || !indices) return fail("SpatialMaxPooling: null tensor");
    if (!(input->nDimension == 3 || input->nDimension == 4)) return fail("3D or 4D (batch) tensor expected");
    if (kW <= 0 || kH <= 0 || dW <= 0 || dH <= 0) return fail("SpatialMaxPooling: invalid kernel/stride");
    const bool batched = input->nDimension == 4;
    const int o = batched ? 1 : 0;
    const long B = batched ? input->size[0] : 1;
    const long C = input->size[o];
    const int H = (int)input->size[o + 1], W = (int)input->size[o + 2];
    if (!(W >= kW && H >= kH)) return fail("input image smaller than kernel size");
    const int Ho = (H - kH) / dH + 1, Wo = (W - kW) / dW + 1;
    if (gradOutput->nDimension != input->nDimension || gradOutput->size[o] != C || gradOutput->size[o + 1] != Ho ||
        gradOutput->size[o + 2] != Wo || (batched && gradOutput->size[0] != B))
        return fail("SpatialMaxPooling: gradOutput size does not match the output size");
    if (!tensor_ready(indices, 2 * B * C * Ho * Wo))
        return fail("SpatialMaxPooling: indices do not match (run updateOutput first)");
    THGPUTensor *go = THGPUTensor_newContiguous(gradOutput);
    if (!go) return 1;
    THGPUTensor_resizeAs(gradInput, input);
    int rc = 0;
    if (!tensor_ready(gradInput, B * C * H * W) || !tensor_backed(go))
        rc = fail("SpatialMaxPooling: could not size gradInput");
    THGPUTensor *in = (!rc && mask_on) ? THGPUTensor_newContiguous(input) : nullptr;
    InputMask mask;
    if (!rc && mask_on) {
        if (!in || !tensor_backed(in)) rc = fail("SpatialMaxPooling: input is not usable as a mask");
        else {
            mask.in = dptr(in);
            mask.threshold = mask_threshold;
        }
    }
    if (!rc) {
        TwinOutput second;
        if (twin && !twin_output(twin, gradInput, second)) second = TwinOutput();
        bool wrote = false;
        rc = maxpool_bwd_launch(dptr(go), dptr(indices), B * C, H, W, Ho, Wo, kH, kW, dH, dW, dptr(gradInput), mask,
                                second, &wrote, second.base && twin_rows_in_zero_border(twin, second));
        if (wrote_twin) *wrote_twin = !rc && wrote ? 1 : 0;
    }
    if (in) THGPUTensor_free(in);
    THGPUTensor_free(go);
    return rc;
}

int thgpu_SpatialMaxPooling_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                            THGPUTensor *indices, int kW, int kH, int dW, int dH) {
    return pool_update_grad_input(input, gradOutput, gradInput, indices, kW, kH, dW, dH, false, 0.0f);
}

int thgpu_SpatialMaxPooling_updateGradInputMasked(THGPUTensor *input, THGPUTensor *gradOutput,
                                                  THGPUTensor *gradInput, THGPUTensor *indices, int kW, int kH,
                                                  int dW, int dH, float threshold) {
    return pool_update_grad_input(input, gradOutput, gradInput, indices, kW, kH, dW, dH, true, threshold);
}

int thgpu_SpatialMaxPooling_updateGradInputTwin(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                                THGPUTensor *indices, int kW, int kH, int dW, int dH, int flags,
                                                float threshold, THGPUTensor *twin, int *wrote_twin) {
    if (flags & ~THGPU_FUSE_INPUT_MASK) return fail("SpatialMaxPooling: unknown flags");
    return pool_update_grad_input(input, gradOutput, gradInput, indices, kW, kH, dW, dH,
                                  (flags & THGPU_FUSE_INPUT_MASK) != 0, threshold, twin, wrote_twin);
}

int thgpu_Threshold_updateOutput(THGPUTensor *input, THGPUTensor *output, float threshold, float val) {
    if (!input || !output) return fail("Threshold: null tensor");
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    if (!in) return 1;
    THGPUTensor_resizeAs(output, in);
    long n = THGPUTensor_nElement(in);
    int rc = 0;
    if (!tensor_ready(output, n) || !tensor_backed(in)) rc = fail("Threshold: could not size output");
    if (!rc) rc = threshold_fwd_launch(dptr(in), dptr(output), n, threshold, val);
    THGPUTensor_free(in);
    return rc;
}

int thgpu_Threshold_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                    float threshold) {
    if (!input || !gradOutput || !gradInput) return fail("Threshold: null tensor");
    if (THGPUTensor_nElement(input) != THGPUTensor_nElement(gradOutput))
        return fail("Threshold: input and gradOutput sizes do not match");
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    THGPUTensor *go = in ? THGPUTensor_newContiguous(gradOutput) : nullptr;
    if (!in || !go) {
        if (in) THGPUTensor_free(in);
        return 1;
    }
    THGPUTensor_resizeAs(gradInput, in);
    long n = THGPUTensor_nElement(in);
    int rc = 0;
    if (!tensor_ready(gradInput, n) || !tensor_backed(in) || !tensor_backed(go))
        rc = fail("Threshold: could not size gradInput");
    if (!rc) rc = threshold_bwd_launch(dptr(in), dptr(go), dptr(gradInput), n, threshold);
    THGPUTensor_free(in);
    THGPUTensor_free(go);
    return rc;
}

int thgpu_conv_set_mode(int mode) {
    if (mode < 0 || mode > 2)
        return fail("conv mode must be 0 (columns), 1 (gathered where it pays) or 2 (gathered where it fits)");
    conv_set_mode(mode);
    return 0;
}

int thgpu_conv_get_mode(void) { return conv_mode(); }

int thgpu_conv_set_finput_reuse(int on) {
    g_finput_reuse = on != 0;
    return 0;
}

int thgpu_conv_get_finput_reuse(void) { return g_finput_reuse ? 1 : 0; }

}  // extern "C"
