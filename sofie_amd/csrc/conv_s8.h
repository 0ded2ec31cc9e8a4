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
   int N, C, H, W, OC, KH, KW, ph, pw, sh, sw, groups;
   int OH, OW, icg, ocg;
   int zpx, zpy, lo, relu;
   int x_nhwc, y_nhwc, w_ohwi;
   int pool_kh, pool_kw, pool_sh, pool_sw;   // fused max pooling after the activation; pool_kh == 0: none
   int PH, PW;                               // pooled output size (OH, OW without pooling)
};

// floor(x / d) for 0 <= x < 2^31 as a multiply-high and a shift (shift < 0: d == 1).
struct FastDiv {
   unsigned magic;
   int shift;
};

inline FastDiv make_fastdiv(unsigned d)
{
   if (d <= 1) return {0u, -1};
   int s = 0;
   while ((1u << s) < d) ++s;
   const unsigned long long num = 1ull << (31 + s);
   return {(unsigned)((num + d - 1) / d), s - 1};
}

__device__ __forceinline__ int fdiv(int x, FastDiv f)
{
   return f.shift < 0 ? x : (int)(__umulhi((unsigned)x, f.magic) >> f.shift);
}

// One input channel, 3x3 kernel, stride 1, padding 1, channels-last int8 output, optionally fused
// with a 2x2 stride-2 max pooling: *done tells whether the kernel took the problem.
int qconv_first_layer(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done);

}  // namespace sofie
