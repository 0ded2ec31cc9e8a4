// Argument block shared by the int8 convolution kernels and their launchers.
#pragma once
#include "common.h"

namespace sofie {

struct QConvArgs {
   const int8_t *x, *w;
   const float *xf;          // if not null: the input is this float tensor, quantized with xscale / zpx on the fly
   float xscale;
   const int32_t *bias;
   const float *scale;
   void *y;
   int N, C, H, W, OC, KH, KW, ph, pw, sh, sw, groups;   // ph, pw: begin pads (top, left)
   int pbh, pbw;                                         // end pads (bottom, right)
   int OH, OW, icg, ocg;
   int zpx, zpy, lo, relu;
   int x_nhwc, y_nhwc, w_ohwi;
   int pool_kh, pool_kw, pool_sh, pool_sw;   // fused max pooling after the activation; pool_kh == 0: none
   int PH, PW;                               // pooled output size (OH, OW without pooling)
};

// One input channel, 3x3 kernel, stride 1, padding 1, channels-last int8 output, optionally fused
// with a 2x2 stride-2 max pooling: *done tells whether the kernel took the problem.
int qconv_first_layer(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done);

// 3x3 kernel, stride 1, 32 or 64 input channels, channels-last int8 in and out: the kernel that fetches the
// input rows straight into LDS. *done tells whether the kernel took the problem.
int qconv_ring(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done);

// Two such layers, the second reading the first one's (pooled) output, in one launch where every workgroup owns the
// same whole images in both. *done tells whether the launch was made (if not, nothing was launched).
int qconv_ring_pair(sofie_hip_ctx *ctx, const QConvArgs &g1, const QConvArgs &g2, bool *done);

}  // namespace sofie
