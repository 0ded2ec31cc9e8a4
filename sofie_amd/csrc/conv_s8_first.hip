// First layer of an int8 CNN: one input channel, 3x3 kernel, stride 1, padding 1, with the
// requantisation, the ReLU clamp and (optionally) a 2x2 stride-2 max pooling fused.
//
// With K = 9 the layer is bound by its output bytes, not by arithmetic, so it runs on the vector
// ALUs: one workgroup per image keeps the zero-point-padded image in LDS; a work item is one output
// pixel (or one pooled pixel = 2x2 output pixels) times all output channels. A kernel row of three
// taps plus a zero is one packed dword, so an output pixel costs three v_dot4_i32_i8 per channel on
// the packed rows of its window (unaligned 4-byte windows are cut out of two aligned dwords with
// v_alignbyte). Pooling is taken on the int32 accumulators: requantisation is monotonic in the
// accumulator (non-decreasing for scale >= 0, non-increasing for scale < 0), so the maximum of the
// requantised values is the requantised maximum (minimum for a negative scale), which equals
// pooling after requantisation bit for bit and needs a quarter of the conversions.
#include "conv_s8.h"

using namespace sofie;

namespace {

struct FirstArgs {
   const int8_t *x;
   const int8_t *w;       // [OC][9]
   const int32_t *bias;   // [OC] or null
   const float *scale;    // [OC]
   int8_t *y;             // [N][PH][PW][OC]
   int H, W, OC, PH, PW;
   int zpx, zpy, lo;
   int stride;            // LDS row stride of the padded image, a multiple of 4
};

__device__ __forceinline__ int window4(const unsigned char *row, int col)
{
   // bytes col .. col+3 of an LDS row whose base is 4-byte aligned
   const int *p = reinterpret_cast<const int *>(row + (col & ~3));
   return (int)__builtin_amdgcn_alignbyte((unsigned)p[1], (unsigned)p[0], (unsigned)(col & 3));
}

template <bool POOL>
__global__ void __launch_bounds__(256) k_qconv_first(FirstArgs a)
{
   extern __shared__ __align__(16) unsigned char smem[];
   v4i *const s_w = reinterpret_cast<v4i *>(smem);                         // [OC] {row0, row1, row2, bias}
   float *const s_scale = reinterpret_cast<float *>(smem + a.OC * 16);     // [OC]
   unsigned char *const s_img = smem + a.OC * 20;                          // [(H+2)][stride] (+8 bytes slack)
   const int tid = threadIdx.x;
   const int n = blockIdx.x;

   for (int oc = tid; oc < a.OC; oc += 256) {
      const int8_t *w = a.w + oc * 9;
      v4i t;
#pragma unroll
      for (int r = 0; r < 3; ++r)
         t[r] = (int)((unsigned)(unsigned char)w[r * 3] | ((unsigned)(unsigned char)w[r * 3 + 1] << 8) |
                      ((unsigned)(unsigned char)w[r * 3 + 2] << 16));
      t[3] = a.bias ? a.bias[oc] : 0;
      s_w[oc] = t;
      s_scale[oc] = a.scale[oc];
   }
   // padded image: border cells hold the input zero-point
   {
      const int8_t *img = a.x + (size_t)n * a.H * a.W;
      const int cells = (a.H + 2) * a.stride + 8;
      for (int i = tid; i < cells; i += 256) {
         const int r = i / a.stride, c = i - r * a.stride;
         const int ih = r - 1, iw = c - 1;
         const bool inside = ih >= 0 && ih < a.H && iw >= 0 && iw < a.W;
         s_img[i] = inside ? (unsigned char)img[ih * a.W + iw] : (unsigned char)a.zpx;
      }
   }
   __syncthreads();

   const float zpo = (float)(a.zpy + 128), lof = (float)(a.lo + 128);
   const int items = a.PH * a.PW;
   for (int it = tid; it < items; it += 256) {
      const int py = it / a.PW, px = it - py * a.PW;
      constexpr int NR = POOL ? 4 : 3, ND = POOL ? 2 : 1;
      const int oy = POOL ? 2 * py : py, ox = POOL ? 2 * px : px;
      int rows[NR][ND];
#pragma unroll
      for (int r = 0; r < NR; ++r) {
         const unsigned char *row = s_img + (oy + r) * a.stride;
#pragma unroll
         for (int d = 0; d < ND; ++d) rows[r][d] = window4(row, ox + d);
      }
      int8_t *out = a.y + ((size_t)(n * a.PH + py) * a.PW + px) * a.OC;
      for (int oc0 = 0; oc0 < a.OC; oc0 += 4) {
         unsigned pk = 0;
#pragma unroll
         for (int e = 0; e < 4; ++e) {
            const v4i wt = s_w[oc0 + e];
            const float sc = s_scale[oc0 + e];
            int hi = 0, lo = 0;
#pragma unroll
            for (int dy = 0; dy < ND; ++dy)
#pragma unroll
               for (int dx = 0; dx < ND; ++dx) {
                  int acc = wt[3];
                  acc = __builtin_amdgcn_sdot4(rows[dy][dx], wt[0], acc, false);
                  acc = __builtin_amdgcn_sdot4(rows[dy + 1][dx], wt[1], acc, false);
                  acc = __builtin_amdgcn_sdot4(rows[dy + 2][dx], wt[2], acc, false);
                  if (dy == 0 && dx == 0) { hi = acc; lo = acc; }
                  else { hi = max(hi, acc); lo = min(lo, acc); }
               }
            const int sel = sc < 0.0f ? lo : hi;
            float r = rintf(__fmul_rn(__int2float_rn(sel), sc));
            r = fmaxf(__fadd_rn(r, zpo), lof);
            pk = __builtin_amdgcn_cvt_pk_u8_f32(r, e, pk);
         }
         *reinterpret_cast<unsigned *>(out + oc0) = pk ^ 0x80808080u;
      }
   }
}

}  // namespace

namespace sofie {

int qconv_first_layer(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done)
{
   *done = false;
   const bool pool = g.pool_kh != 0;
   if (g.C != 1 || g.groups != 1 || g.KH != 3 || g.KW != 3 || g.sh != 1 || g.sw != 1 || g.ph != 1 || g.pw != 1) return SOFIE_HIP_OK;
   if (g.OC % 4 != 0 || !(g.y_nhwc) || (reinterpret_cast<uintptr_t>(g.y) & 3u) != 0) return SOFIE_HIP_OK;
   if (pool && !(g.pool_kh == 2 && g.pool_kw == 2 && g.pool_sh == 2 && g.pool_sw == 2)) return SOFIE_HIP_OK;
   FirstArgs a{};
   a.x = g.x; a.w = g.w; a.bias = g.bias; a.scale = g.scale; a.y = static_cast<int8_t *>(g.y);
   a.H = g.H; a.W = g.W; a.OC = g.OC; a.PH = g.PH; a.PW = g.PW;
   a.zpx = g.zpx; a.zpy = g.zpy; a.lo = g.lo;
   a.stride = (g.W + 2 + 3) / 4 * 4 + 4;
   const size_t lds = (size_t)g.OC * 20 + (size_t)(g.H + 2) * a.stride + 8;
   if (lds > 64 * 1024) return SOFIE_HIP_OK;
   const dim3 grid((unsigned)g.N), block(256);
   if (pool) hipLaunchKernelGGL(k_qconv_first<true>, grid, block, lds, ctx->stream, a);
   else hipLaunchKernelGGL(k_qconv_first<false>, grid, block, lds, ctx->stream, a);
   *done = true;
   return check_launch(ctx, "k_qconv_first");
}

}  // namespace sofie
