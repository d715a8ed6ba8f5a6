// Small independent jobs that ride along in another kernel's launch as extra workgroups behind its own (a launch of
// their own would cost several microseconds for one microsecond of work).
#pragma once

#include "common.h"

namespace thgpu {

// The kernel bank as the first operand of a gradInput product, one element per lane:
//   unit stride:  wt[c][m][kh][kw] = w[m][c][kH-1-kh][kW-1-kw]
//   strided:      wt[(c, ph, pw)][(m, a', b')] = w[m][c][ph + sH*(A-1-a')][pw + sW*(Bk-1-b')], zero where that tap lies
//                 outside the kernel and in the rows beyond C*sH*sW (the product's rows are padded to a whole tile).
struct WeightJob {
    const float *w;
    float *wt;
    int M, C, kH, kW;
    int sH, sW, A, Bk, rows, rows_pad;  // strided form only (sH = 0: unit stride)
    unsigned count;                     // elements of wt; 0: no job
};

__device__ __forceinline__ void reorder_weight(const WeightJob &j, unsigned idx) {
    if (idx >= j.count) return;
    if (j.sH == 0) {
        const unsigned kk = (unsigned)(j.kH * j.kW);
        const unsigned tap = idx % kk, cm = idx / kk;
        const unsigned m = cm % j.M, c = cm / j.M;
        const unsigned kh = tap / j.kW, kw = tap % j.kW;
        j.wt[idx] = j.w[((long)m * j.C + c) * kk + (j.kH - 1 - kh) * j.kW + (j.kW - 1 - kw)];
        return;
    }
    const unsigned R = (unsigned)(j.M * j.A * j.Bk);
    const unsigned row = idx / R, r = idx % R;
    float v = 0.0f;
    if (row < (unsigned)j.rows) {
        const unsigned pw = row % j.sW, ph = (row / j.sW) % j.sH, c = row / (j.sW * j.sH);
        const unsigned bb = r % j.Bk, aa = (r / j.Bk) % j.A, m = r / (j.Bk * j.A);
        const unsigned kh = ph + j.sH * (j.A - 1 - aa), kw = pw + j.sW * (j.Bk - 1 - bb);
        if (kh < (unsigned)j.kH && kw < (unsigned)j.kW) v = j.w[(((long)m * j.C + c) * j.kH + kh) * j.kW + kw];
    }
    j.wt[idx] = v;
}

// The re-ordering of a convolution's kernel bank that its gradInput product needs, offered to whoever launches a
// kernel before that product does (conv_implicit.hip keeps the one pending job):
//   offer_bank_job    by the code that prepares the product's gradOutput buffer;
//   take_bank_job     by a launcher that can carry extra workgroups: returns the job and marks it done;
//   bank_job_done     by the product: whether the bank at `wt` has been re-ordered since it was offered (clears it).
void offer_bank_job(const WeightJob &job);
bool take_bank_job(WeightJob &job);
bool bank_job_done(const float *wt);

}  // namespace thgpu
