// Launchers of the hot-path kernels (all enqueue on the library stream and
// return 0 or a recorded error).
#pragma once

#include "common.h"

namespace thgpu {

// nn.Threshold's backward fused into the kernel that produces the gradient: an element of the result is kept
// where `in` (same shape and layout as the result) exceeds `threshold` and zeroed elsewhere.  in == nullptr: off.
struct InputMask {
    const float *in = nullptr;
    float threshold = 0.0f;
    // Layout of `in` where a kernel accepts another than the result's dense one (the gathered convolution's
    // gradInput store): floats between its planes (0: dense) and between its rows (0: dense).
    long plane = 0;
    int pitch = 0;
};

// Where a convolution's output planes go when not densely packed: floats between planes (images are
// nOutputPlane planes apart) and between the rows of a plane (0: dense rows).
struct OutputLayout {
    long plane = 0;  // 0: dense
    int pitch = 0;
};

// A second copy of a [B, C, H, W] result kept inside another buffer: element (plane, y, x) at
// base[plane*plane_stride + y*pitch + x] (planes of all images evenly spaced).  base == nullptr: none.  This is how
// the producer of a gradient writes it straight into the zero-bordered buffer that the convolution in front gathers
// its gradInput product from, so that no padded copy is made afterwards.
struct TwinOutput {
    float *base = nullptr;
    long plane = 0;
    int pitch = 0;
};

int im2col_launch(const float *im, long B, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW,
                  float *col);
int col2im_launch(const float *col, long B, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW,
                  float *im, InputMask mask = InputMask());
// out_plane / out_pitch: floats between the output's planes and rows when it is not densely packed (0: dense).
int maxpool_fwd_launch(const float *in, long planes, int H, int W, int kH, int kW, int dH, int dW, float *out,
                       float *indices, long out_plane = 0, int out_pitch = 0);
// *wrote_twin (when twin.base is set) says whether the kernel that ran also stored the second copy.  twin_gaps: the
// floats between the rows of the second copy are known to hold zeros and may be stored (as zeros) along with the rows.
int maxpool_bwd_launch(const float *gout, const float *indices, long planes, int H, int W, int Ho, int Wo, int kH,
                       int kW, int dH, int dW, float *gin, InputMask mask = InputMask(), TwinOutput twin = TwinOutput(),
                       bool *wrote_twin = nullptr, bool twin_gaps = false);
int threshold_fwd_launch(const float *in, float *out, long n, float th, float val);
int threshold_bwd_launch(const float *in, const float *gout, float *gin, long n, float th);
int gradbias_launch(const float *gout, float *gbias, long B, int M, long N, float scale);

// Convolution without the column buffer (conv_implicit.hip).  conv_mode: 0 = im2col / GEMM / col2im,
// 1 = gathered GEMMs where the shape fits and the route pays, 2 = wherever the shape fits.  The two
// predicates answer for the current mode: forward and gradWeight go together (they share finput),
// gradInput on its own.  `padded` is the input padded by (pH, pW), B*C planes of (H+2pH) x (W+2pW);
// `scratch` takes conv_implicit_gradinput_scratch floats.
int conv_mode();
void conv_set_mode(int mode);
bool conv_use_gathered(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW);
bool conv_use_gathered_gradinput(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW);
long conv_implicit_gradinput_scratch(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH,
                                     int sW);
int pad_planes_launch(const float *in, long planes, int H, int W, int pH, int pW, float *out);
// `act` applies nn.Threshold (threshold, value) to the output as it is stored; `mask` zeroes gradInput where the
// convolution's input does not exceed a threshold (the backward of a Threshold in front of the convolution).
struct OutputThreshold {
    bool on = false;
    float threshold = 0.0f, value = 0.0f;
};
int conv_implicit_forward(const float *padded, const float *weight, const float *bias, float *output, long B, int C,
                          int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW,
                          OutputThreshold act = OutputThreshold(), OutputLayout out = OutputLayout());
// Forward of a layer with at most 32 taps and 64 output planes without the tiled GEMM (conv_narrow.hip): whether the
// shape is taken, and the launch (padded images image_stride floats apart; output position (y, x) reads from
// y * row_step + x on; the gathered route's tap table).
bool conv_narrow_forward_fits(long B, int M, long K, int Wo, long N, int col_step, OutputLayout out);
int conv_narrow_forward(const float *padded, long image_stride, const float *weight, const float *bias, float *output,
                        long B, int M, int K, int Ho, int Wo, int row_step, const int *rowtab, OutputThreshold act);
// ... and its gradWeight (+= scale * sums over the batch) with gradBias (+= scale * row sums of gradOutput; may be
// null), gradOutput dense [B][64][Ho*Wo].
bool conv_narrow_gradweight_fits(long B, int M, long K, int Wo, long N, int col_step);
int conv_narrow_gradweight(const float *padded, long image_stride, const float *gradOutput, float *gradWeight,
                           float *gradBias, long B, int M, int K, int Ho, int Wo, int row_step, const int *rowtab,
                           float scale);
// gradBias (may be null) receives scale * the sums of gradOutput over images and positions when the product can
// compute them on the side; *bias_done says whether it did.
int conv_implicit_gradweight(const float *padded, const float *gradOutput, float *gradWeight, long B, int C, int H,
                             int W, int M, int kH, int kW, int pH, int pW, int sH, int sW, float scale, float *gradBias,
                             bool *bias_done);
// q_ready: the head of `scratch` already holds gradOutput in the padded layout conv_implicit_q_layout describes
// (its producer wrote it there through a TwinOutput, borders zero), so no padded copy is made.  twin: a second copy of
// gradInput (unit-stride layers only; *wrote_twin says whether it was stored).
int conv_implicit_gradinput(const float *gradOutput, const float *weight, float *scratch, float *gradInput, long B,
                            int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW,
                            InputMask mask = InputMask(), bool q_ready = false, TwinOutput twin = TwinOutput(),
                            bool *wrote_twin = nullptr);
// Where gradOutput [B, M, Ho, Wo] lies inside the padded buffer the gathered gradInput product reads (the head of its
// scratch): planes of Hq x Wq, the dense plane at row `top`, column `left`, zeros around it.
void conv_implicit_q_layout(int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW, int *top, int *left,
                            int *Hq, int *Wq);
// Offers the re-ordering of the layer's kernel bank (into the tail of `scratch`, where the gradInput product expects
// it) to the launches that come before that product (side_jobs.h).
void conv_implicit_offer_bank(const float *weight, float *scratch, long B, int C, int H, int W, int M, int kH, int kW,
                              int pH, int pW, int sH, int sW);
// Forgets what is known about a device buffer that is being released (nn_ops.hip keeps track of buffers whose borders
// it has zeroed).
void conv_forget_buffer(const float *p);

// Host-only checks of the launch planners (no GPU needed); each returns the number of violations.
long im2col_plan_selftest();
long pool_plan_selftest();

}  // namespace thgpu
