// First layer of an int8 CNN: one input channel, 3x3 kernel, stride 1, padding 1, with the
// requantisation, the ReLU clamp and (optionally) a 2x2 stride-2 max pooling fused.
//
// With K = 9 the layer is bound by its output bytes, so the point is to spend few vector instructions
// per output. A workgroup keeps a few zero-point-padded images in LDS; a wavefront takes 32 (pooled)
// pixels at a time and computes them with v_mfma_i32_32x32x16_i8, K = 16 laid out as the three
// kernel rows of four bytes (a zero weight and three taps) plus four zero weights. With that order the
// pixel operand of a lane is simply two 4-byte windows of consecutive image rows (lanes 0-31: rows
// y, y+1; lanes 32-63: rows y+2, y+3), cut out of aligned dwords with v_alignbyte; no byte shuffling.
// An image row sits in LDS behind four bytes of padding, so image dword j is LDS dword j + 1 and the
// staging is one aligned store per four pixels; the window of output column x starts at padded byte x + 2.
// For the pooled variant the four window positions are four matrix instructions whose accumulators are
// pooled register-wise (on the int32 values: requantisation is monotonic in the accumulator; if any
// scale of the workgroup's channels is negative, the minimum is taken for those channels), so a quarter
// of the values is converted. Two v_permlane32_swap turn the lane's four 4-channel groups into 16
// consecutive channels and the result leaves as one 16-byte store per lane.
#include <math.h>
#include <type_traits>
#include "conv_s8.h"

using namespace sofie;

namespace {

struct FirstArgs {
   const int8_t *x;
   const float *xf;       // float input to quantize on the fly (then x is unused), or null
   float xscale;
   const int8_t *w;       // [OC][9]
   const int32_t *bias;   // [OC] or null
   const float *scale;    // [OC]
   int8_t *y;             // [N][PH][PW][OC]
   int N, H, W, OC, PH, PW;
   int zpx, zpy, lo;
   int stride;            // LDS row stride of a padded image, a multiple of 4
   int img_bytes;         // LDS bytes of one padded image
   int ocb;               // blocks of 32 output channels (the last may be half used)
   int rows;              // LDS rows of one padded image (H + 3)
   int images;            // images per workgroup
   int dword_fill;        // W % 4 == 0 and x aligned: the images are filled a dword at a time
   int fast_div;          // x / xscale as a reciprocal multiply and two fused corrections (see quantize4)
   float xinv;            // 1 / xscale, correctly rounded
   FastDiv dper_image, dPW, dHW4, dW4;
   // how the coordinates of a work item move from one loop iteration to the next (the loops advance by a fixed
   // number of items, so no iteration divides): a staging thread moves on by 256 groups of four pixels, a
   // wavefront by 128 (pooled) output pixels
   int st_im, st_row, st_col;   // 256 = st_im * (H*W/4) + st_row * (W/4) + st_col
   int px_im, px_row, px_col;   // 128 = px_im * (PH*PW) + px_row * PW + px_col
};


// p: the aligned dword of an LDS row that holds byte `col` of it, sh = col & 3
__device__ __forceinline__ void windows(const unsigned char *p8, unsigned sh, int &w0, int &w1)
{
   // bytes col..col+3 and col+1..col+4 (col even)
   const int *p = reinterpret_cast<const int *>(p8);
   const unsigned lo = (unsigned)p[0], hi = (unsigned)p[1];
   w0 = (int)__builtin_amdgcn_alignbyte(hi, lo, sh);
   w1 = (int)__builtin_amdgcn_alignbyte(hi, lo, sh + 1u);
}

__device__ __forceinline__ int window(const unsigned char *p8, unsigned sh)
{
   const int *p = reinterpret_cast<const int *>(p8);
   return (int)__builtin_amdgcn_alignbyte((unsigned)p[1], (unsigned)p[0], sh);
}

__device__ __forceinline__ long pack64(int lo, int hi)
{
   return (long)(((unsigned long long)(unsigned)hi << 32) | (unsigned long long)(unsigned)lo);
}

// QuantizeLinear of one value: sat_s8(rint_half_even(x / scale) + zp), returned as a byte.
__device__ __forceinline__ unsigned quantize_byte(float v, float scale, int zp)
{
   float r = rintf(__fdiv_rn(v, scale));
   r = fminf(fmaxf(r, -1024.0f), 1024.0f);
   return (unsigned)min(127, max(-128, (int)r + zp)) & 0xffu;
}

// Four values to four bytes, the same result as quantize_byte. With FAST the quotient is q0 = x * inv
// corrected once, q = fma(fma(-q0, scale, x), inv, q0): for inv = RN(1 / scale) that is the correctly rounded
// x / scale (the remainder is exact in the fused operation); the host takes this path only for
// 2^-30 <= |scale| <= 2^30, and x is clamped to +-2^45 first (beyond it the result saturates either way), so
// nothing overflows. zpo = zp + 128: the byte conversion saturates to [0, 255] and rounds an integer to itself.
template <bool FAST>
__device__ __forceinline__ unsigned quantize4(v4f v, float scale, float inv, int zp, float zpo)
{
   if constexpr (!FAST) {
      return quantize_byte(v[0], scale, zp) | (quantize_byte(v[1], scale, zp) << 8) |
             (quantize_byte(v[2], scale, zp) << 16) | (quantize_byte(v[3], scale, zp) << 24);
   } else {
      unsigned pk = 0;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
         const float x = __builtin_amdgcn_fmed3f(v[t], -0x1p45f, 0x1p45f);
         const float q0 = __fmul_rn(x, inv);
         const float q = __fmaf_rn(__fmaf_rn(-q0, scale, x), inv, q0);
         pk = __builtin_amdgcn_cvt_pk_u8_f32(__fadd_rn(rintf(q), zpo), t, pk);
      }
      return pk ^ 0x80808080u;
   }
}

template <bool POOL>
// Four workgroups per CU (at most 128 registers): the loop is a chain of dependent vector instructions per group of
// pixels, and a fourth wavefront per SIMD fills the gaps the other three leave (25.4 us instead of 30.8 us for 4096
// images of 40x40 with 32 channels and pooling; five workgroups need 102 registers and lose more than they gain).
__global__ void __launch_bounds__(256, 4) k_qconv_first(FirstArgs a)
{
   extern __shared__ __align__(16) unsigned char smem[];
   const int OCP = a.ocb * 32;                                              // channels padded to blocks of 32
   float *const s_scale = reinterpret_cast<float *>(smem);                  // [OCP]
   int *const s_bias = reinterpret_cast<int *>(s_scale + OCP);              // [OCP]
   long *const s_wfrag = reinterpret_cast<long *>(s_bias + OCP);            // [OCP][2] matrix operand of the weights
   int *const s_flag = reinterpret_cast<int *>(s_wfrag + OCP * 2);          // [4] any negative scale
   unsigned char *const s_img = reinterpret_cast<unsigned char *>(s_flag + 4);
   const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
   const int half = lane >> 5, l32 = lane & 31;
   const int n0 = blockIdx.x * a.images;
   const int nimg = (a.N - n0) < a.images ? (a.N - n0) : a.images;

   // Staging of the images, in two halves: the loads of a thread's first groups of four pixels are requested here, before
   // anything else, and used below, behind the set-up of the channels' parameters (whose own loads would otherwise
   // be waited for first). A thread takes every 256th group of the workgroup's images, which lie back to back in
   // memory, so the loads are contiguous over the workgroup; the coordinates (image, row, dword) of a thread's next
   // group follow from the present ones by additions.
   constexpr int UN = 8;   // groups per thread whose loads are in flight together
   const int HW4 = (a.H * a.W) >> 2, W4 = a.W >> 2;
   const int total4 = a.dword_fill ? nimg * HW4 : 0;
   const v4f *const srcf = reinterpret_cast<const v4f *>(a.xf + (size_t)n0 * a.H * a.W);
   const unsigned *const srcq = reinterpret_cast<const unsigned *>(a.x + (size_t)n0 * a.H * a.W);
   const int wave_first = __builtin_amdgcn_readfirstlane(tid & ~63);
   int st_im = 0, st_row = 0, st_col = 0;
   auto request = [&](int base, unsigned (&q)[UN], v4f (&f)[UN], int (&dst)[UN]) {
      // a wavefront skips the groups that lie past the end for all of its lanes (the last round of a workgroup)
#pragma unroll
      for (int u = 0; u < UN; ++u) {
         const int idx = base + u * 256 + tid;
         if (base + u * 256 + wave_first < total4) {
            const int safe = idx < total4 ? idx : total4 - 1;   // the loads are unconditional within the wavefront
            if (a.xf) f[u] = srcf[safe];
            else q[u] = srcq[safe];
         }
         // image dword j of a row is LDS dword j + 1
         dst[u] = idx < total4 ? (int)__umul24(st_im, a.img_bytes) + (int)__umul24(st_row + 1, a.stride) + 4 * st_col + 4 : -1;
         st_col += a.st_col; st_row += a.st_row; st_im += a.st_im;
         if (st_col >= W4) { st_col -= W4; st_row += 1; }
         if (st_row >= a.H) { st_row -= a.H; st_im += 1; }
      }
   };
   unsigned q_first[UN];
   v4f f_first[UN];
   int dst_first[UN];
   if (a.dword_fill) {
      st_im = fdiv(tid, a.dHW4);
      const int r = tid - st_im * HW4;
      st_row = fdiv(r, a.dW4);
      st_col = r - st_row * W4;
      request(0, q_first, f_first, dst_first);
   }

   if (tid == 0) s_flag[0] = 0;
   __syncthreads();
   for (int oc = tid; oc < OCP; oc += 256) {
      const bool real = oc < a.OC;
      const int8_t *w = a.w + oc * 9;
      unsigned r[3] = {0u, 0u, 0u};
      if (real) {
#pragma unroll
         for (int k = 0; k < 3; ++k)
            r[k] = ((unsigned)(unsigned char)w[k * 3] << 8) | ((unsigned)(unsigned char)w[k * 3 + 1] << 16) |
                   ((unsigned)(unsigned char)w[k * 3 + 2] << 24);
      }
      s_wfrag[oc * 2] = pack64((int)r[0], (int)r[1]);      // lanes 0-31: kernel rows 0 and 1
      s_wfrag[oc * 2 + 1] = pack64((int)r[2], 0);          // lanes 32-63: kernel row 2 and four zero weights
      const float sc = real ? a.scale[oc] : 0.0f;
      s_scale[oc] = sc;
      s_bias[oc] = (real && a.bias) ? a.bias[oc] : 0;
      if (sc < 0.0f) s_flag[0] = 1;
   }
   // padded images: cells outside the image hold the input zero-point; one spare row below each image is
   // read (with zero weights) by the upper half of the wavefront
   if (a.dword_fill) {
      // Every cell first gets the zero-point (16 bytes per store), then the images' own cells are written over.
      const unsigned zp4 = 0x01010101u * (unsigned)(a.zpx & 0xff);
      const float zpo = (float)(a.zpx + 128);
      const int bytes = nimg * a.img_bytes;                 // a multiple of 4
      const v4i zfill = {(int)zp4, (int)zp4, (int)zp4, (int)zp4};
      for (int i = tid; i < (bytes >> 4); i += 256) reinterpret_cast<v4i *>(s_img)[i] = zfill;
      if (tid < ((bytes & 15) >> 2)) reinterpret_cast<unsigned *>(s_img + (bytes & ~15))[tid] = zp4;
      __syncthreads();
      auto deliver = [&](int base, unsigned (&q)[UN], v4f (&f)[UN], int (&dst)[UN]) {
#pragma unroll
         for (int u = 0; u < UN; ++u) {
            if (base + u * 256 + wave_first < total4) {
               if (a.xf) q[u] = a.fast_div ? quantize4<true>(f[u], a.xscale, a.xinv, a.zpx, zpo)
                                           : quantize4<false>(f[u], a.xscale, a.xinv, a.zpx, zpo);
               if (dst[u] >= 0) *reinterpret_cast<unsigned *>(s_img + dst[u]) = q[u];
            }
         }
      };
      deliver(0, q_first, f_first, dst_first);
      for (int base = 256 * UN; base < total4; base += 256 * UN) {
         unsigned q[UN];
         v4f f[UN];
         int dst[UN];
         request(base, q, f, dst);
         deliver(base, q, f, dst);
      }
   } else {
      for (int i = tid; i < nimg * a.img_bytes; i += 256) {
         const int im = i / a.img_bytes, o = i - im * a.img_bytes;
         const int r = o / a.stride, c = o - r * a.stride;
         const int ih = r - 1, iw = c - 4;
         const bool inside = ih >= 0 && ih < a.H && iw >= 0 && iw < a.W;
         const size_t src = ((size_t)(n0 + im) * a.H + (inside ? ih : 0)) * a.W + (inside ? iw : 0);
         const unsigned char v = a.xf ? (unsigned char)quantize_byte(a.xf[src], a.xscale, a.zpx) : (unsigned char)a.x[src];
         s_img[i] = inside ? v : (unsigned char)a.zpx;
      }
   }
   __syncthreads();
   const bool any_negative = s_flag[0] != 0;

   const float zpo = (float)(a.zpy + 128), lof = (float)(a.lo + 128);
   const bool plain = a.zpy == -128 && a.lo == -128;
   const int per_image = a.PH * a.PW;
   const int total = nimg * per_image;
   const int groups = (total + 31) / 32;
   constexpr int NP = POOL ? 4 : 1;               // matrix instructions (window positions) per group
   // weight operand, bias and scales of a block of 32 channels: register e of a tile belongs to channel
   // (e/4)*8 + half*4 + e%4. With one block they are loaded once.
   // The scales stay in LDS and are read where a group needs them (four 16-byte reads per group): held in
   // registers next to the bias tile and two or three accumulator tiles they pushed the loop over the 128
   // registers of four workgroups per CU, and a reload from scratch memory at the head of the loop waits for
   // every earlier memory instruction of the wavefront, the stores of its previous group included.
   long wfrag = 0;
   v16i binit;
   auto load_params = [&](int ob) {
      wfrag = s_wfrag[(ob * 32 + l32) * 2 + half];
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
         const v4i b = *reinterpret_cast<const v4i *>(s_bias + ob * 32 + gq * 8 + half * 4);
#pragma unroll
         for (int t = 0; t < 4; ++t) binit[gq * 4 + t] = b[t];
      }
   };
   const bool single = a.ocb == 1;
   load_params(0);
   // The loop is instantiated for the four combinations of (plain requantisation, scales of both signs): both
   // are uniform over the launch, and a run-time select inside the loop would cost more than the arithmetic.
   auto process = [&](auto plain_c, auto negative_c) {
      constexpr bool PLAIN = decltype(plain_c)::value;
      constexpr bool NEGATIVE = decltype(negative_c)::value;
      // The wavefront's pixels move on by 128 per iteration; image, row and column of a lane's pixel follow by
      // additions, and the output offset is linear in the pixel's number (the images of a workgroup are stored
      // back to back).
      int q = wave * 32 + l32;
      int im = fdiv(q, a.dper_image);
      int py, px;
      {
         const int rem = q - im * per_image;
         py = fdiv(rem, a.dPW);
         px = rem - py * a.PW;
      }
      unsigned yoff = (unsigned)q * (unsigned)a.OC + (unsigned)half * 16u;
      const unsigned ystep = 128u * (unsigned)a.OC;
      int8_t *const ybase = a.y + (size_t)n0 * per_image * a.OC;
      const int half_rows = (int)__umul24(2 * half, a.stride);
      for (int g = wave; g < groups; g += 4) {
         const bool valid = q < total;
         const int col = (POOL ? 2 * px : px) + 2;
         const int cell = (int)__umul24(im, a.img_bytes) + (int)__umul24(POOL ? 2 * py : py, a.stride) + (col & ~3);
         const unsigned char *base = s_img + half_rows + (valid ? cell : 0);   // a lane past the end reads the first pixel
         const unsigned sh = (unsigned)(col & 3);
         long pix[NP];
         if constexpr (POOL) {
            int r[3][2];
#pragma unroll
            for (int k = 0; k < 3; ++k) windows(base + k * a.stride, sh, r[k][0], r[k][1]);
#pragma unroll
            for (int j = 0; j < 4; ++j) pix[j] = pack64(r[j >> 1][j & 1], r[(j >> 1) + 1][j & 1]);
         } else {
            pix[0] = pack64(window(base, sh), window(base + a.stride, sh));
         }
         int8_t *out = ybase + yoff;
         q += 128;
         yoff += ystep;
         px += a.px_col; py += a.px_row; im += a.px_im;
         if (px >= a.PW) { px -= a.PW; py += 1; }
         if (py >= a.PH) { py -= a.PH; im += 1; }
         for (int ob = 0; ob < a.ocb; ++ob) {
            if (!single) load_params(ob);
            v4f sc[4];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) sc[gq] = *reinterpret_cast<const v4f *>(s_scale + ob * 32 + gq * 8 + half * 4);
            // one window position at a time keeps two accumulator tiles live (more wavefronts per SIMD); the
            // bias tile is the C operand of every matrix instruction (max(a + b) = max(a) + b), which costs nothing
            v16i acc = __builtin_amdgcn_mfma_i32_32x32x16_i8(wfrag, pix[0], binit, 0, 0, 0);
            if constexpr (POOL) {
               v16i lo;
               if constexpr (NEGATIVE) lo = acc;
#pragma unroll
               for (int j = 1; j < 4; ++j) {
                  const v16i c = __builtin_amdgcn_mfma_i32_32x32x16_i8(wfrag, pix[j], binit, 0, 0, 0);
#pragma unroll
                  for (int e = 0; e < 16; ++e) acc[e] = max(acc[e], c[e]);
                  if constexpr (NEGATIVE) {
#pragma unroll
                     for (int e = 0; e < 16; ++e) lo[e] = min(lo[e], c[e]);
                  }
               }
               if constexpr (NEGATIVE) {
#pragma unroll
                  for (int e = 0; e < 16; ++e) acc[e] = sc[e >> 2][e & 3] < 0.0f ? lo[e] : acc[e];
               }
            }
            unsigned d[4];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
               unsigned pk = 0;
#pragma unroll
               for (int t = 0; t < 4; ++t) {
                  float r = __fmul_rn(__int2float_rn(acc[gq * 4 + t]), sc[gq][t]);
                  if constexpr (!PLAIN) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);   // the byte conversion rounds half to even itself
                  pk = __builtin_amdgcn_cvt_pk_u8_f32(r, t, pk);
               }
               d[gq] = pk ^ 0x80808080u;
            }
            // lanes 0-31 hold channels {0-3, 8-11, 16-19, 24-27} of their pixel, lanes 32-63 {4-7, 12-15, 20-23, 28-31}:
            // after the swaps the lower half has channels 0-15 and the upper half 16-31, in order
            const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
            const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
            const v4i v = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
            if (valid && ob * 32 + half * 16 < a.OC) store16_wt(out + ob * 32, v);   // the two halves of the wavefront write whole lines between them
         }
      }
   };
   using yes = std::integral_constant<bool, true>;
   using no = std::integral_constant<bool, false>;
   if (plain) {
      if (POOL && any_negative) process(yes{}, yes{});
      else process(yes{}, no{});
   } else {
      if (POOL && any_negative) process(no{}, yes{});
      else process(no{}, no{});
   }
}

}  // namespace

namespace sofie {

int qconv_first_layer(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done)
{
   *done = false;
   const bool pool = g.pool_kh != 0;
   if (g.C != 1 || g.groups != 1 || g.KH != 3 || g.KW != 3 || g.sh != 1 || g.sw != 1 || g.ph != 1 || g.pw != 1 ||
       g.pbh != 1 || g.pbw != 1) return SOFIE_HIP_OK;
   if (g.OC % 16 != 0 || !g.y_nhwc || !aligned16(g.y)) return SOFIE_HIP_OK;
   if (pool && !(g.pool_kh == 2 && g.pool_kw == 2 && g.pool_sh == 2 && g.pool_sw == 2)) return SOFIE_HIP_OK;
   if (g.PH <= 0 || g.PW <= 0) return SOFIE_HIP_OK;
   FirstArgs a{};
   a.x = g.x; a.xf = g.xf; a.xscale = g.xscale; a.w = g.w; a.bias = g.bias; a.scale = g.scale; a.y = static_cast<int8_t *>(g.y);
   a.N = g.N; a.H = g.H; a.W = g.W; a.OC = g.OC; a.PH = g.PH; a.PW = g.PW;
   a.zpx = g.zpx; a.zpy = g.zpy; a.lo = g.lo;
   a.stride = (((g.W + 2) >> 2) + 2) * 4;         // four bytes of left padding; a window spans two aligned dwords
   a.img_bytes = (g.H + 3) * a.stride;
   a.ocb = (g.OC + 31) / 32;
   a.rows = g.H + 3;
   a.dword_fill = g.W % 4 == 0 && (g.xf ? aligned16(g.xf) : (reinterpret_cast<uintptr_t>(g.x) & 3u) == 0);
   {
      const float as = fabsf(g.xscale);
      a.fast_div = g.xf && as >= 0x1p-30f && as <= 0x1p30f;
      a.xinv = a.fast_div ? 1.0f / g.xscale : 0.0f;
   }
   if (a.dword_fill) {
      const int HW4 = g.H * g.W / 4, W4 = g.W / 4;
      a.dHW4 = make_fastdiv((unsigned)HW4);
      a.dW4 = make_fastdiv((unsigned)W4);
      a.st_im = 256 / HW4;
      a.st_row = (256 % HW4) / W4;
      a.st_col = (256 % HW4) % W4;
   }
   {
      const int per_image = g.PH * g.PW;
      a.px_im = 128 / per_image;
      a.px_row = (128 % per_image) / g.PW;
      a.px_col = (128 % per_image) % g.PW;
   }
   a.dper_image = make_fastdiv((unsigned)(g.PH * g.PW));
   a.dPW = make_fastdiv((unsigned)g.PW);
   // Images per workgroup: four workgroups share a CU, and the kernel is as slow as the busiest CU, so the
   // count is the one that leaves the fewest image-times on a workgroup slot (rounds of workgroups x images each);
   // of equal ones the larger (fewer parameter loads). At most 16 images and 36 KB of them.
   const size_t fixed = (size_t)a.ocb * 32 * 24 + 16 + 16;
   const int slots = 4 * (ctx->num_cus > 0 ? ctx->num_cus : 256);
   int best = 0;
   long best_cost = 0;
   for (int k = 1; k <= 16; ++k) {
      if (fixed + (size_t)k * a.img_bytes > 36 * 1024) break;
      const long wgs = (g.N + k - 1) / k;
      const long cost = ((wgs + slots - 1) / slots) * k;
      if (best == 0 || cost <= best_cost) { best = k; best_cost = cost; }
   }
   if (best == 0) return SOFIE_HIP_OK;
   a.images = best;
   const size_t lds = fixed + (size_t)a.images * a.img_bytes;
   const dim3 grid((unsigned)((g.N + a.images - 1) / a.images)), block(256);
   if (pool) hipLaunchKernelGGL(k_qconv_first<true>, grid, block, lds, ctx->stream, a);
   else hipLaunchKernelGGL(k_qconv_first<false>, grid, block, lds, ctx->stream, a);
   *done = true;
   return check_launch(ctx, "k_qconv_first");
}

}  // namespace sofie
