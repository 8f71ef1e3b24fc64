// Shared between the conv2d entry point (gemm_api.hip) and the repacking
// implicit-GEMM path (conv2d.hip).
#pragma once

#include "nt_common.h"

namespace nt {

struct Conv2dRequest {
    int dtype;
    const void *x;
    const void *w;
    void *y;
    int N, C, H, W, K, R, S, P, Q, pad_h, pad_w;
    int64_t xs[4], ws[4], ys[4];  // element strides of input, filter, output
    // output position (p, q) and filter tap (r, s) read input (p * stride_h + r * dil_h - pad_h, q * stride_w + s * dil_w - pad_w)
    int stride_h = 1, stride_w = 1, dil_h = 1, dil_w = 1;
    bool unit_steps() const { return stride_h == 1 && stride_w == 1 && dil_h == 1 && dil_w == 1; }
};

// Runs the direct-to-LDS implicit GEMM when the request qualifies; returns
// NINETOOTHED_NO_KERNEL when it does not (the caller then uses the gather kernel).
int conv2d_fast(const Conv2dRequest &request, hipStream_t stream);

// Runs the convolution in one launch on the tensors as they lie (no repacking, no scratch memory) when the
// request qualifies -- pixels of an input row contiguous, output width a multiple of 8, padding_w <= 1,
// C*R*S a multiple of 32, contiguous filter and output, output channels filling 256-wide tiles --; returns
// NINETOOTHED_NO_KERNEL when it does not.
int conv2d_direct(const Conv2dRequest &request, hipStream_t stream);

}  // namespace nt
