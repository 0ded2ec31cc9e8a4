// int8 convolution with int32 accumulation and fused requantisation (QLinearConv semantics).
//
// k_qconv_simple: one thread per output element, any layout / group count / channel count.
#include "common.h"

using namespace sofie;

namespace {

struct QConvArgs {
   const int8_t *x, *w;
   const int32_t *bias;
   const float *scale;
   void *y;
   int N, C, H, W, OC, KH, KW, ph, pw, sh, sw, groups;
   int OH, OW, icg, ocg;
   int zpx, zpy, lo, relu;
   int x_nhwc, y_nhwc;
};

template <int OUT>
__global__ void k_qconv_simple(QConvArgs g)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   const size_t total = (size_t)g.N * g.OC * g.OH * g.OW;
   if (idx >= total) return;
   size_t r = idx;
   int n, oc, oh, ow;
   if (g.y_nhwc) {
      oc = (int)(r % g.OC); r /= g.OC;
      ow = (int)(r % g.OW); r /= g.OW;
      oh = (int)(r % g.OH); n = (int)(r / g.OH);
   } else {
      ow = (int)(r % g.OW); r /= g.OW;
      oh = (int)(r % g.OH); r /= g.OH;
      oc = (int)(r % g.OC); n = (int)(r / g.OC);
   }
   const int grp = oc / g.ocg;
   int acc = 0;
   for (int kh = 0; kh < g.KH; ++kh) {
      const int ih = oh * g.sh - g.ph + kh;
      for (int kw = 0; kw < g.KW; ++kw) {
         const int iw = ow * g.sw - g.pw + kw;
         const bool inside = ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
         for (int ic = 0; ic < g.icg; ++ic) {
            const int c = grp * g.icg + ic;
            int xv = g.zpx;   // padding cells hold the input zero-point
            if (inside)
               xv = g.x_nhwc ? g.x[(((size_t)n * g.H + ih) * g.W + iw) * g.C + c]
                             : g.x[(((size_t)n * g.C + c) * g.H + ih) * g.W + iw];
            acc += xv * (int)g.w[(((size_t)oc * g.icg + ic) * g.KH + kh) * g.KW + kw];
         }
      }
   }
   if (g.bias) acc += g.bias[oc];
   if constexpr (OUT == SOFIE_OUT_S32) static_cast<int *>(g.y)[idx] = acc;
   else static_cast<int8_t *>(g.y)[idx] = (int8_t)requant(acc, g.scale[oc], g.zpy, g.lo);
}

}  // namespace

extern "C" int sofie_hip_qconv2d_s8(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, const int8_t *w,
                                    const int32_t *bias, const float *scale, void *y, int y_layout, int N, int C,
                                    int H, int W, int OC, int KH, int KW, int pad_h, int pad_w, int stride_h,
                                    int stride_w, int groups, int zp_x, int zp_y, int act, int out_kind)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C > 0 && H > 0 && W > 0 && OC > 0 && KH > 0 && KW > 0, "non-positive dimension");
   SOFIE_REQUIRE(ctx, pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0, "bad pads/strides");
   SOFIE_REQUIRE(ctx, groups > 0 && C % groups == 0 && OC % groups == 0, "channels not divisible by groups");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   SOFIE_REQUIRE(ctx, (x_layout == SOFIE_LAYOUT_NCHW || x_layout == SOFIE_LAYOUT_NHWC) &&
                         (y_layout == SOFIE_LAYOUT_NCHW || y_layout == SOFIE_LAYOUT_NHWC), "unknown layout");
   SOFIE_REQUIRE(ctx, out_kind == SOFIE_OUT_S8 || out_kind == SOFIE_OUT_S32, "output kind must be S8 or S32");
   SOFIE_REQUIRE(ctx, zp_x >= -128 && zp_x <= 127 && zp_y >= -128 && zp_y <= 127, "zero-point out of int8 range");
   SOFIE_REQUIRE(ctx, H + 2 * pad_h >= KH && W + 2 * pad_w >= KW, "kernel larger than padded input");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && w && y, "null operand");
   SOFIE_REQUIRE(ctx, scale || out_kind == SOFIE_OUT_S32, "scale is required for S8 output");
   QConvArgs g{};
   g.x = x; g.w = w; g.bias = bias; g.scale = scale; g.y = y;
   g.N = N; g.C = C; g.H = H; g.W = W; g.OC = OC; g.KH = KH; g.KW = KW;
   g.ph = pad_h; g.pw = pad_w; g.sh = stride_h; g.sw = stride_w; g.groups = groups;
   g.OH = (H + 2 * pad_h - KH) / stride_h + 1;
   g.OW = (W + 2 * pad_w - KW) / stride_w + 1;
   g.icg = C / groups;
   g.ocg = OC / groups;
   g.zpx = zp_x; g.zpy = zp_y;
   g.relu = act == SOFIE_ACT_RELU;
   g.lo = (g.relu && zp_y > -128) ? zp_y : -128;
   g.x_nhwc = x_layout == SOFIE_LAYOUT_NHWC;
   g.y_nhwc = y_layout == SOFIE_LAYOUT_NHWC;
   const size_t total = (size_t)N * OC * g.OH * g.OW;
   const dim3 grid((unsigned)((total + 255) / 256)), block(256);
   if (out_kind == SOFIE_OUT_S32) hipLaunchKernelGGL(k_qconv_simple<SOFIE_OUT_S32>, grid, block, 0, ctx->stream, g);
   else hipLaunchKernelGGL(k_qconv_simple<SOFIE_OUT_S8>, grid, block, 0, ctx->stream, g);
   return check_launch(ctx, "k_qconv_simple");
}
