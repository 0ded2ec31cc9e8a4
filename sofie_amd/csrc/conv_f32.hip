// fp32 NCHW convolution as an implicit GEMM on the matrix cores (v_mfma_f32_32x32x2_f32).
//
// Per image and group:  Y[oc, pixel] = sum_k Wmat[oc, k] * xcol[k, pixel],  k = (ic, kh, kw),
// which is the product the reference forms with Im2col + sgemm_, except that xcol is never
// written anywhere: a workgroup stages the raw input patch (rows and columns its pixel tile
// touches, halo included, zero filled outside the image) for a block of input channels in LDS
// and every MFMA column operand is gathered from that patch at  base(pixel) + offset(k).
// base() depends only on the lane's pixel and is computed once; offset() depends only on k and
// lives in a small LDS table. The weight block of the K-chunk is staged k-major next to it.
// Output rows of the MFMA tile are output channels, columns are pixels, so 32 lanes write 32
// consecutive pixels of one channel plane: coalesced NCHW stores, bias and ReLU fused.
// Roofline: MFMA fp32; per K-step of 2 each wavefront issues TI*TJ MFMAs (64 cycles each)
// against TI+TJ+1 ds_read_b32.
#include <type_traits>

#include "common.h"
#include "gemm_tile.h"

using namespace sofie;

namespace {

// Most patch cells of a channel block in k_conv2d_f32_dma (a thread keeps an offset per 256 cells).
#define SOFIE_CONV_DMA_PATCH 3584

// Geometry of one output phase of a strided transposed convolution when all phases run in one launch.
struct PhaseArgs {
   int KH, KW, th0, tw0, ph, pw, oy0, ox0, OH, OW, rows_out, PH, PW, ICB, KC;
   int woff;           // k_conv2d_f32_dma: first float of the phase's sub-kernel in the gathered weights
   FastDiv dPW, dPH, dKC, dOW, dK4;
};
#define SOFIE_CONV_MAX_PHASES 4

struct ConvArgs {
   const float *x, *w, *bias;
   float *y;
   int N, C, H, W, OC, KH, KW, ph, pw, sh, sw, dh, dw, groups;
   int OH, OW, icg, ocg;
   int ICB, KC;        // input channels per K-chunk, K-chunk length (even)
   int PH, PW;         // staged patch extent
   int rows_out;       // output rows a pixel tile can span
   int relu;
   // Transposed convolution (uh, uw > 0): the same implicit GEMM over the input seen with uh-1 / uw-1 zeros
   // between its rows / columns, unit output stride, and the weights w [C, OC/groups, KH, KW] read with both
   // kernel axes reversed. ph / pw are then dil*(K-1) - pad of the transposed convolution (may be negative).
   int transposed, uh, uw;
   // Tap (a, b) of this launch is element (th0 + a * ths, tw0 + b * tws) of the KH0 x KW0 kernel in memory, and output
   // pixel (q, r) of this launch is pixel (oy0 + q * oys, ox0 + r * oxs) of the OH0 x OW0 output plane. A plain
   // convolution has the identity for both; a transposed convolution with a stride runs one launch per output
   // phase (oy mod stride, ox mod stride), each with the taps that reach that phase and no zeros in between.
   int KH0, KW0, th0, ths, tw0, tws;
   int OH0, OW0, oy0, oys, ox0, oxs;
   int wvec;           // weights are staged with 16-byte loads (see launch)
   FastDiv dPW, dPH, dKC, dK4;   // divisions by the patch extents and the K-chunk length (/4) in the staging loops
   FastDiv dUH, dUW, dOW;
   // csplit > 1 (k_conv2d_f32_dma): blockIdx.z = (image [* phases + phase]) * csplit + slice; a slice sums its share of
   // the channel blocks into partial [slice][N][OC][output plane] without bias and ReLU, k_conv_f32_split_finish adds the slices
   int csplit;
   float *partial;
   // nphases > 1: blockIdx.z = image * nphases + phase, and the phase's geometry replaces the fields above
   int nphases;
   PhaseArgs phase[SOFIE_CONV_MAX_PHASES];
};

// Input row / column behind position `up` of the zero-interleaved input, or -1 where a zero sits.
__device__ __forceinline__ int source_index(int up, int u, FastDiv d)
{
   if (up < 0) return -1;
   if (u == 1) return up;
   const int q = fdiv(up, d);
   return q * u == up ? q : -1;
}

// TR: the launch is (a phase of) a transposed convolution; the plain convolution is compiled without the tap and
// output maps.
template <int TI, int TJ, bool TR>
__global__ void __launch_bounds__(256) k_conv2d_f32(ConvArgs g)
{
   constexpr int BOC = 2 * TI * 32, BP = 2 * TJ * 32, LDW = BOC + 1;
   // geometry of this workgroup's launch: the kernel's own, or that of its output phase when all phases of a strided
   // transposed convolution run in one launch (picked with static indices so that it stays in scalar registers)
   PhaseArgs q;
   q.KH = g.KH; q.KW = g.KW; q.th0 = g.th0; q.tw0 = g.tw0; q.ph = g.ph; q.pw = g.pw; q.oy0 = g.oy0; q.ox0 = g.ox0;
   q.OH = g.OH; q.OW = g.OW; q.rows_out = g.rows_out; q.PH = g.PH; q.PW = g.PW; q.ICB = g.ICB; q.KC = g.KC;
   q.dPW = g.dPW; q.dPH = g.dPH; q.dKC = g.dKC; q.dOW = g.dOW;
   int n = blockIdx.z;
   if constexpr (TR) {
      if (g.nphases > 1) {
         const int pi = blockIdx.z % g.nphases;
         n = blockIdx.z / g.nphases;
         q = g.phase[0];
#pragma unroll
         for (int i = 1; i < SOFIE_CONV_MAX_PHASES; ++i)
            if (pi == i) q = g.phase[i];
         if ((int)blockIdx.x * BP >= q.OH * q.OW) return;   // the grid is as wide as the phase with most pixel tiles
      }
   }
   extern __shared__ __align__(16) unsigned char smem_raw[];
   float *sW = reinterpret_cast<float *>(smem_raw);                  // [KC][LDW]
   float *patch = sW + q.KC * LDW;                                   // [ICB][PH][PW]
   int *koff = reinterpret_cast<int *>(patch + q.ICB * q.PH * q.PW); // [KC]

   const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
   const int wm = wave >> 1, wn = wave & 1;
   const int fr = lane & 31, fk = lane >> 5;

   const int octiles = (g.ocg + BOC - 1) / BOC;
   const int grp = blockIdx.y / octiles;
   const int oc0 = (blockIdx.y % octiles) * BOC;    // within the group
   const int OHW = q.OH * q.OW;
   const int p0 = blockIdx.x * BP;
   const int oh0 = p0 / q.OW;
   const int ih0 = oh0 * g.sh - q.ph, iw0 = -q.pw;
   const int KHW = q.KH * q.KW;
   const int Kfull = g.icg * KHW;

   for (int k = tid; k < q.KC; k += 256) {
      const int icl = k / KHW, t = k % KHW;
      const int kh = t / q.KW, kw = t % q.KW;
      koff[k] = (icl < q.ICB) ? (icl * q.PH + kh * g.dh) * q.PW + kw * g.dw : 0;
   }

   int base[TJ];
#pragma unroll
   for (int j = 0; j < TJ; ++j) {
      const int p = p0 + wn * TJ * 32 + j * 32 + fr;
      base[j] = (p < OHW) ? ((p / q.OW - oh0) * g.sh) * q.PW + (p % q.OW) * g.sw : 0;
   }

   v16f acc[TI][TJ];
#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
         for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

   const float *xg = g.x + ((size_t)n * g.C + (size_t)grp * g.icg) * g.H * g.W;
   const float *wg = g.w + (size_t)grp * g.ocg * Kfull;
   const int patch_len = q.ICB * q.PH * q.PW;

   for (int ic0 = 0; ic0 < g.icg; ic0 += q.ICB) {
      const int icn = (g.icg - ic0) < q.ICB ? (g.icg - ic0) : q.ICB;
      const int kc = icn * KHW;
      __syncthreads();   // previous chunk fully consumed (also orders the koff table on entry)
      // Staging: every load of a batch is issued before the first value is used (the addresses of cells outside the
      // image, channels past the block and columns past the group are clamped to element 0 and the value replaced
      // by zero afterwards), so a batch costs one memory latency instead of one per element.
      auto stage_patch = [&](auto batch) {
         constexpr int UP = decltype(batch)::value;
         for (int e0 = 0; e0 < patch_len; e0 += 256 * UP) {
            float v[UP];
            bool inside[UP];
#pragma unroll
            for (int u = 0; u < UP; ++u) {
               const int e = e0 + u * 256 + tid;
               const int t = fdiv(e, q.dPW), c = e - t * q.PW;
               const int icl = fdiv(t, q.dPH), r = t - icl * q.PH;
               int ih = ih0 + r, iw = iw0 + c;
               if constexpr (TR) {
                  ih = source_index(ih, g.uh, g.dUH);
                  iw = source_index(iw, g.uw, g.dUW);
               }
               inside[u] = e < patch_len && icl < icn && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
               v[u] = xg[inside[u] ? ((size_t)(ic0 + icl) * g.H + ih) * g.W + iw : 0];
            }
#pragma unroll
            for (int u = 0; u < UP; ++u) {
               const int e = e0 + u * 256 + tid;
               if (e < patch_len) patch[e] = inside[u] ? v[u] : 0.0f;
            }
         }
      };
      // six loads per thread and batch: twelve (one batch for a 3x3 block of eight channels) costs a workgroup per CU
      // in registers and measured 14 % slower
      stage_patch(std::integral_constant<int, 6>{});
      if (!TR && g.wvec) {
         // four consecutive k of one output channel per 16-byte load (every block is full and 16-byte aligned)
         const int K4 = q.KC >> 2, total4 = K4 * BOC;
         auto stage_weights4 = [&](auto batch) {
            constexpr int UW = decltype(batch)::value;
            for (int e0 = 0; e0 < total4; e0 += 256 * UW) {
               v4f v[UW];
               int dst[UW];
#pragma unroll
               for (int u = 0; u < UW; ++u) {
                  const int e = e0 + u * 256 + tid;
                  const int ocl = fdiv(e, g.dK4), k4 = e - ocl * K4;
                  const bool ok = e < total4 && oc0 + ocl < g.ocg;
                  v[u] = *reinterpret_cast<const v4f *>(wg + (ok ? (size_t)(oc0 + ocl) * Kfull + (size_t)ic0 * KHW + 4 * k4 : 0));
                  if (!ok) v[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
                  dst[u] = e < total4 ? 4 * k4 * LDW + ocl : -1;
               }
#pragma unroll
               for (int u = 0; u < UW; ++u) {
                  if (dst[u] >= 0) {
#pragma unroll
                     for (int q = 0; q < 4; ++q) sW[dst[u] + q * LDW] = v[u][q];
                  }
               }
            }
         };
         stage_weights4(std::integral_constant<int, 3>{});
      } else {
         constexpr int UW = 8;
         const int total = q.KC * BOC;
         for (int e0 = 0; e0 < total; e0 += 256 * UW) {
            float v[UW];
            bool ok[UW];
#pragma unroll
            for (int u = 0; u < UW; ++u) {
               const int e = e0 + u * 256 + tid;
               const int ocl = fdiv(e, q.dKC), k = e - ocl * q.KC;
               ok[u] = e < total && k < kc && oc0 + ocl < g.ocg;
               size_t off = 0;
               if (ok[u]) {
                  if constexpr (TR) {
                     const int icl = k / KHW, t = k - icl * KHW;
                     const int ta = t / q.KW, tb = t - ta * q.KW;
                     off = ((((size_t)grp * g.icg + ic0 + icl) * g.ocg + oc0 + ocl) * g.KH0 + q.th0 + ta * g.ths) * g.KW0 + q.tw0 +
                           tb * g.tws;
                  } else {
                     off = (size_t)grp * g.ocg * Kfull + (size_t)(oc0 + ocl) * Kfull + (size_t)ic0 * KHW + k;
                  }
               }
               v[u] = g.w[off];
            }
#pragma unroll
            for (int u = 0; u < UW; ++u) {
               const int e = e0 + u * 256 + tid;
               const int ocl = fdiv(e, q.dKC), k = e - ocl * q.KC;
               if (e < total) sW[k * LDW + ocl] = ok[u] ? v[u] : 0.0f;
            }
         }
      }
      __syncthreads();
      const float *wrow = sW + wm * TI * 32 + fr;
      for (int s = 0; s < q.KC / 2; ++s) {
         const int kk = 2 * s + fk;
         const int ko = koff[kk];
         float fa[TI], fb[TJ];
#pragma unroll
         for (int i = 0; i < TI; ++i) fa[i] = wrow[kk * LDW + i * 32];
#pragma unroll
         for (int j = 0; j < TJ; ++j) fb[j] = patch[base[j] + ko];
#pragma unroll
         for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j)
               acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
   }

   const size_t plane = TR ? (size_t)g.OH0 * g.OW0 : (size_t)OHW;
   float *yn = g.y + ((size_t)n * g.OC + (size_t)grp * g.ocg) * plane;
#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
         const int p = p0 + wn * TJ * 32 + j * 32 + fr;
         if (p >= OHW) continue;
         size_t po = (size_t)p;
         if constexpr (TR) {
            const int row = fdiv(p, q.dOW);
            po = (size_t)(q.oy0 + row * g.oys) * g.OW0 + q.ox0 + (p - row * q.OW) * g.oxs;
         }
#pragma unroll
         for (int r = 0; r < 16; ++r) {
            const int oc = oc0 + wm * TI * 32 + i * 32 + (r >> 2) * 8 + fk * 4 + (r & 3);
            if (oc >= g.ocg) continue;
            float v = acc[i][j][r];
            if (g.bias) v = __fadd_rn(v, g.bias[grp * g.ocg + oc]);
            if (g.relu) v = v > 0.0f ? v : 0.0f;
            yn[(size_t)oc * plane + po] = v;
         }
      }
}

// The same implicit GEMM with both operands of channel block c+1 travelling global memory -> LDS without registers
// (buffer_load ... lds) under the matrix loop of block c. The weights come from a copy laid out for it, wt [group]
// [K = input channel, tap][wstride >= OC/groups, a multiple of 4] (k_transpose_weights / k_gather_phase_weights write it
// into the scratch buffer in front of the launch), so that a row of the LDS tile [KC][BOC] is a contiguous piece of a
// row of wt and goes 16 bytes per lane. A patch cell is 4 bytes per lane from wherever it sits in the image;
// padding cells ask for an offset outside the descriptor's range and receive 0. Nothing of a block depends on the
// block but a uniform offset, so a thread keeps NP patch offsets and one weight offset for the whole kernel.
// PHASES: the launch holds the output phases of a strided transposed convolution (blockIdx.z = image * nphases +
// phase). A phase is a plain unit-stride convolution of the input with its sub-kernel (g.w then holds the sub-kernels
// in the order above, one after the other) whose outputs go to every stride-th pixel of the output plane.
template <int TI, int TJ, bool PHASES = false, int KWT = 0>
__global__ void __launch_bounds__(256, TI == 1 ? 7 : 3) k_conv2d_f32_dma(ConvArgs gg)
{
   constexpr int BOC = 2 * TI * 32, BP = 2 * TJ * 32;
   constexpr int NP = SOFIE_CONV_DMA_PATCH / 256;
   constexpr int ROWS_PER_REQUEST = 1024 / BOC;       // weight rows one request of 256 lanes x 16 bytes covers
   constexpr unsigned OUTSIDE = 0x40000000u;          // an offset no descriptor of this kernel reaches
   struct Geometry {
      const float *x, *w, *bias;
      float *y;
      int C, H, W, OC, KH, KW, ph, pw, sh, sw, dh, dw, OH, OW, icg, ocg, ICB, KC, PH, PW, relu;
      FastDiv dPW, dPH;
   } g;
   g.x = gg.x; g.w = gg.w; g.bias = gg.bias; g.y = gg.y;
   g.C = gg.C; g.H = gg.H; g.W = gg.W; g.OC = gg.OC; g.KH = gg.KH; g.KW = gg.KW; g.ph = gg.ph; g.pw = gg.pw;
   g.sh = gg.sh; g.sw = gg.sw; g.dh = gg.dh; g.dw = gg.dw; g.OH = gg.OH; g.OW = gg.OW; g.icg = gg.icg; g.ocg = gg.ocg;
   g.ICB = gg.ICB; g.KC = gg.KC; g.PH = gg.PH; g.PW = gg.PW; g.relu = gg.relu;
   g.dPW = gg.dPW; g.dPH = gg.dPH;
   const int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
   int n = bz;
   int oy0 = 0, ox0 = 0;
   int c_begin = 0, c_end = g.icg / g.ICB;
   FastDiv dOW = gg.dOW;
   int slice = 0;
   if (gg.csplit > 1) {
      // blockIdx.z = (image [* phases + phase]) * slices + slice
      slice = bz % gg.csplit;
      n = bz / gg.csplit;
   }
   if constexpr (PHASES) {
      const int pi = n % gg.nphases;
      n = n / gg.nphases;
      PhaseArgs q = gg.phase[0];
#pragma unroll
      for (int i = 1; i < SOFIE_CONV_MAX_PHASES; ++i)
         if (pi == i) q = gg.phase[i];
      if (bx * BP >= q.OH * q.OW) return;   // the grid is as wide as the phase with most pixel tiles
      g.KH = q.KH; g.KW = q.KW; g.ph = q.ph; g.pw = q.pw; g.OH = q.OH; g.OW = q.OW; g.ICB = q.ICB; g.KC = q.KC;
      g.PH = q.PH; g.PW = q.PW; g.dPW = q.dPW; g.dPH = q.dPH;
      g.w = gg.w + q.woff;
      oy0 = q.oy0; ox0 = q.ox0; dOW = q.dOW;
      c_end = g.icg / g.ICB;
   }
   if (gg.csplit > 1) {
      // a slice of the channel blocks (possibly none of them): raw sums into its copy of the output in the scratch buffer
      const int per = (c_end + gg.csplit - 1) / gg.csplit;
      c_begin = slice * per;
      c_end = c_end < c_begin + per ? c_end : c_begin + per;
      g.y = gg.partial + (size_t)slice * gg.N * g.OC * (PHASES ? gg.OH0 * gg.OW0 : g.OH * g.OW);
      g.bias = nullptr;
      g.relu = 0;
   }
   extern __shared__ __align__(16) unsigned char smem_raw[];
   const int patch_len = g.ICB * g.PH * g.PW;
   const int patch_room = (patch_len + 255) & ~255;                  // requests write whole groups of 256 cells
   const int buf_len = g.KC * BOC + patch_room;                      // floats of one buffer: [KC][BOC] weights, patch
   float *const bufs = reinterpret_cast<float *>(smem_raw);
   int *const koff = reinterpret_cast<int *>(bufs + 2 * buf_len);    // [KC]

   const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int wm = wave >> 1, wn = wave & 1;
   const int fr = lane & 31, fk = lane >> 5;
   const int octiles = (g.ocg + BOC - 1) / BOC;
   const int grp = by / octiles;
   const int oc0 = (by % octiles) * BOC;    // within the group
   const int OHW = g.OH * g.OW;
   const int p0 = bx * BP;
   const int oh0 = fdiv(p0, dOW);
   const int ih0 = oh0 * g.sh - g.ph, iw0 = -g.pw;
   const int KHW = g.KH * g.KW;
   const int Kfull = g.icg * KHW;
   const int wstride = (g.ocg + 3) & ~3;
   const size_t HW = (size_t)g.H * g.W;

   if constexpr (KWT == 0)
      for (int k = tid; k < g.KC; k += 256) {
         const int icl = k / KHW, t = k % KHW;
         const int kh = t / g.KW, kw = t % g.KW;
         koff[k] = (icl * g.PH + kh * g.dh) * g.PW + kw * g.dw;
      }
   int base[TJ];
#pragma unroll
   for (int j = 0; j < TJ; ++j) {
      const int p = p0 + wn * TJ * 32 + j * 32 + fr;
      const int row = fdiv(p, dOW);
      base[j] = (p < OHW) ? ((row - oh0) * g.sh) * g.PW + (p - row * g.OW) * g.sw : 0;
      if constexpr (KWT > 0) base[j] += fk * g.PH * g.PW;
   }
   v16f acc[TI][TJ];
#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
         for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

   // descriptors: this image's channels of the group, this group's weights (the launcher keeps both under 1 GiB)
   const rsrc_t xrs = make_rsrc(g.x + ((size_t)n * g.C + (size_t)grp * g.icg) * HW, (unsigned)((size_t)g.icg * HW * 4));
   const rsrc_t wrs = make_rsrc(g.w + (size_t)grp * Kfull * wstride, (unsigned)((size_t)Kfull * wstride * 4));
   // byte offsets of this thread's patch cells inside a block's channels, and of its 16 bytes of weight row tid /
   // (BOC/4) (the rows of its later requests are ROWS_PER_REQUEST further each: same parity, same rotation)
   const int npatch = (patch_len + 255) >> 8;        // patch requests per thread (of NP)
   unsigned pofs[NP];
#pragma unroll
   for (int u = 0; u < NP; ++u) {
      pofs[u] = OUTSIDE;
      if (u >= npatch) continue;
      const int e = u * 256 + tid;
      const int t = fdiv(e, g.dPW), c = e - t * g.PW;
      const int icl = fdiv(t, g.dPH), r = t - icl * g.PH;
      const int ih = ih0 + r, iw = iw0 + c;
      const bool inside = e < patch_len && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
      pofs[u] = inside ? (unsigned)(((icl * g.H + ih) * g.W + iw) * 4) : OUTSIDE;
   }
   const int wrow0 = tid / (BOC / 4);
   const int wcol = (tid % (BOC / 4)) * 4;
   const unsigned wofs = oc0 + wcol < wstride ? (unsigned)((wrow0 * wstride + oc0 + wcol) * 4) : OUTSIDE;
   const unsigned xblock = (unsigned)(g.ICB * HW * 4), wblock = (unsigned)(g.KC * wstride * 4);
   const unsigned wstep = (unsigned)(ROWS_PER_REQUEST * wstride * 4);
   const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem_raw;   // LDS byte address of the buffers

   auto request = [&](int c, int buf) {
      const unsigned sw = lds0 + (unsigned)buf * buf_len * 4, sp = sw + (unsigned)g.KC * BOC * 4;
#pragma unroll
      for (int u = 0; u < NP; ++u)
         if (u < npatch) dma4(xrs, sp + (u * 256 + wave * 64) * 4, (int)pofs[u], (int)(c * xblock));
      for (int r0 = 0; r0 < g.KC; r0 += ROWS_PER_REQUEST)
         if (r0 + wrow0 < g.KC)
            dma16(wrs, sw + (r0 * BOC + wave * 256) * 4, (int)wofs, (int)(c * wblock + (r0 / ROWS_PER_REQUEST) * wstep));
   };

   const int nsteps = p0 + wn * TJ * 32 < OHW ? g.KC / 2 : 0;   // a wavefront with no pixel of the plane multiplies nothing
   if (c_begin < c_end) request(c_begin, 0);
   wait_vmcnt<0>();
   __syncthreads();   // the first block and the koff table are in LDS
   for (int c = c_begin; c < c_end; ++c) {
      if (c + 1 < c_end) request(c + 1, (c + 1 - c_begin) & 1);
      const float *const sW = bufs + ((c - c_begin) & 1) * buf_len, *const patch = sW + g.KC * BOC;
      if constexpr (KWT > 0) {
         // K runs (channel pair, kernel row, kernel column, channel of the pair): the two K values of a matrix
         // instruction are the same tap of two neighbouring channels, so a lane's patch address is its own constant
         // (pixel, channel of the pair) plus a uniform offset per kernel row, and the kernel's columns are immediate
         // offsets: no table of offsets, three vector additions per kernel row
         const float *wl = sW + fk * BOC + wm * TI * 32 + fr;
         if (nsteps > 0)
            for (int m = 0; m < g.ICB / 2; ++m)
               for (int kh = 0; kh < g.KH; ++kh) {
                  const int row = __builtin_amdgcn_readfirstlane((2 * m * g.PH + kh * g.dh) * g.PW);
                  const float *pb[TJ];
#pragma unroll
                  for (int j = 0; j < TJ; ++j) pb[j] = patch + base[j] + row;
#pragma unroll
                  for (int kw = 0; kw < KWT; ++kw) {
                     float fa[TI], fb[TJ];
#pragma unroll
                     for (int i = 0; i < TI; ++i) fa[i] = wl[kw * 2 * BOC + i * 32];
#pragma unroll
                     for (int j = 0; j < TJ; ++j) fb[j] = pb[j][kw];
#pragma unroll
                     for (int i = 0; i < TI; ++i)
#pragma unroll
                        for (int j = 0; j < TJ; ++j)
                           acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
                  }
                  wl += KWT * 2 * BOC;
               }
      } else {
         const float *wl = sW + wm * TI * 32 + fr;
         for (int s = 0; s < nsteps; ++s) {
            const int kk = 2 * s + fk;
            const int ko = koff[kk];
            float fa[TI], fb[TJ];
#pragma unroll
            for (int i = 0; i < TI; ++i) fa[i] = wl[kk * BOC + i * 32];
#pragma unroll
            for (int j = 0; j < TJ; ++j) fb[j] = patch[base[j] + ko];
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
               for (int j = 0; j < TJ; ++j)
                  acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
         }
      }
      // the next block has landed (this wavefront's requests; the barrier makes it every wavefront's), and the
      // buffer it replaces next was last read in this block
      wait_vmcnt<0>();
      __syncthreads();
   }

   // Stores through a descriptor of this image's output channels of the group (the launcher keeps it under 1 GiB): a
   // lane's offset is its pixel (and its K half's four channels), the channel of a store is a uniform offset, and what
   // lies behind the plane's pixels or the group's channels falls outside the descriptor's range and is dropped.
   const size_t plane = PHASES ? (size_t)gg.OH0 * gg.OW0 : (size_t)OHW;
   const rsrc_t yrs = make_rsrc(g.y + ((size_t)n * g.OC + (size_t)grp * g.ocg) * plane, (unsigned)((size_t)g.ocg * plane * 4));
   const unsigned plane4 = (unsigned)(plane * 4);
   // biases the same way (no bias: an empty range, every load returns 0)
   const __amdgpu_buffer_rsrc_t brs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(g.bias) + (g.bias ? grp * g.ocg : 0), 0, g.bias ? g.ocg * 4 : 0, 0x00020000);
   float bv[TI][16];
#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r)
         bv[i][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                 brs, fk * 16, (oc0 + wm * TI * 32 + i * 32 + (r >> 2) * 8 + (r & 3)) * 4, 0));
#pragma unroll
   for (int j = 0; j < TJ; ++j) {
      const int p = p0 + wn * TJ * 32 + j * 32 + fr;
      unsigned po = (unsigned)p;
      if constexpr (PHASES) {
         const int row = fdiv(p, dOW);
         po = (unsigned)((oy0 + row * gg.oys) * gg.OW0 + ox0 + (p - row * g.OW) * gg.oxs);
      }
      const unsigned voff = p < OHW ? po * 4 + (unsigned)fk * 4 * plane4 : OUTSIDE;
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
         for (int r = 0; r < 16; ++r) {
            const int oc_uniform = oc0 + wm * TI * 32 + i * 32 + (r >> 2) * 8 + (r & 3);   // + 4 * fk in the lane's offset
            float v = __fadd_rn(acc[i][j][r], bv[i][r]);
            if (g.relu) v = v > 0.0f ? v : 0.0f;
            store4_buf(yrs, v, voff, (unsigned)oc_uniform * plane4);
         }
   }
}

// Sum of the channel slices' partial outputs in slice order, then bias and ReLU: one thread per output value.
__global__ void __launch_bounds__(256) k_conv_f32_split_finish(const float *__restrict__ partial, float *__restrict__ y,
                                                               const float *__restrict__ bias, int slices, size_t total,
                                                               int plane, int OC, int relu)
{
   const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
   if (idx >= total) return;
   float p[8];
#pragma unroll
   for (int i = 0; i < 8; ++i) p[i] = i < slices ? partial[(size_t)i * total + idx] : 0.0f;
   float v = p[0];
#pragma unroll
   for (int i = 1; i < 8; ++i)
      if (i < slices) v = __fadd_rn(v, p[i]);
   if (bias) v = __fadd_rn(v, bias[(idx / plane) % OC]);
   if (relu) v = v > 0.0f ? v : 0.0f;
   y[idx] = v;
}

// Weights of a plain convolution w [OC][C/groups][KH][KW] as k_conv2d_f32_dma reads them: wt [group][K][wstride],
// K = (input channel, tap), or (channel pair, tap, channel of the pair) with `pairs`; wstride = OC/groups rounded up
// to 4 (the cells behind the last channel are 0).
__global__ void k_transpose_weights(const float *w, float *wt, int groups, int ocg, int Kfull, int wstride, int pairs, int KHW)
{
   const int e = blockIdx.x * blockDim.x + threadIdx.x;
   if (e >= groups * Kfull * wstride) return;
   const int oc = e % wstride, grp = e / (wstride * Kfull);
   int k = (e / wstride) % Kfull;
   if (pairs) k = (2 * (k / (2 * KHW)) + (k & 1)) * KHW + (k >> 1) % KHW;
   wt[e] = oc < ocg ? w[((size_t)grp * ocg + oc) * Kfull + k] : 0.0f;
}

// Sub-kernels of the output phases of a strided transposed convolution, gathered from its weights w [C, OC/groups, KH0,
// KW0] into the order k_conv2d_f32_dma reads: phase after phase, each [groups][K = input channel, tap][wstride] (K =
// (channel pair, tap, channel of the pair) with `pairs`) with tap (a, b) = element (th0 + a*ths, tw0 + b*tws) of the
// kernel and zeros behind the last channel. One thread per value.
__global__ void k_gather_phase_weights(ConvArgs g, float *dst, int total, int wstride, int pairs)
{
   const int e = blockIdx.x * blockDim.x + threadIdx.x;
   if (e >= total) return;
   int pi = 0;
#pragma unroll
   for (int i = 1; i < SOFIE_CONV_MAX_PHASES; ++i)
      if (i < g.nphases && e >= g.phase[i].woff) pi = i;
   PhaseArgs q = g.phase[0];
#pragma unroll
   for (int i = 1; i < SOFIE_CONV_MAX_PHASES; ++i)
      if (pi == i) q = g.phase[i];
   int r = e - q.woff;
   const int oc = r % wstride; r /= wstride;
   int a, b, ic;
   if (pairs) {      // K = (channel pair, tap, channel of the pair)
      const int parity = r & 1; r >>= 1;
      b = r % q.KW; r /= q.KW;
      a = r % q.KH; r /= q.KH;
      ic = 2 * (r % (g.icg / 2)) + parity;
      r /= g.icg / 2;
   } else {
      b = r % q.KW; r /= q.KW;
      a = r % q.KH; r /= q.KH;
      ic = r % g.icg;
      r /= g.icg;
   }
   const int grp = r;
   dst[e] = oc < g.ocg ? g.w[((((size_t)grp * g.icg + ic) * g.ocg + oc) * g.KH0 + q.th0 + a * g.ths) * g.KW0 + q.tw0 + b * g.tws]
                       : 0.0f;
}

// One thread per output element: any kernel size, used when the staged patch of the tiled
// kernel would not fit LDS.
__global__ void k_conv2d_f32_simple(ConvArgs g)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   const size_t total = (size_t)g.N * g.OC * g.OH * g.OW;
   if (idx >= total) return;
   size_t r = idx;
   const int ow = (int)(r % g.OW); r /= g.OW;
   const int oh = (int)(r % g.OH); r /= g.OH;
   const int oc = (int)(r % g.OC);
   const int n = (int)(r / g.OC);
   const int grp = oc / g.ocg;
   float acc = 0.0f;
   for (int ic = 0; ic < g.icg; ++ic)
      for (int kh = 0; kh < g.KH; ++kh) {
         int ih = oh * g.sh - g.ph + kh * g.dh;
         if (g.transposed) ih = source_index(ih, g.uh, g.dUH);
         if (ih < 0 || ih >= g.H) continue;
         for (int kw = 0; kw < g.KW; ++kw) {
            int iw = ow * g.sw - g.pw + kw * g.dw;
            if (g.transposed) iw = source_index(iw, g.uw, g.dUW);
            if (iw < 0 || iw >= g.W) continue;
            const float wv = g.transposed
                                ? g.w[((((size_t)grp * g.icg + ic) * g.ocg + (oc - grp * g.ocg)) * g.KH0 + g.th0 + kh * g.ths) * g.KW0 +
                                      g.tw0 + kw * g.tws]
                                : g.w[(((size_t)oc * g.icg + ic) * g.KH + kh) * g.KW + kw];
            acc = __fadd_rn(acc, __fmul_rn(g.x[(((size_t)n * g.C + grp * g.icg + ic) * g.H + ih) * g.W + iw], wv));
         }
      }
   if (g.bias) acc = __fadd_rn(acc, g.bias[oc]);
   if (g.relu) acc = acc > 0.0f ? acc : 0.0f;
   g.y[(((size_t)n * g.OC + oc) * g.OH0 + g.oy0 + oh * g.oys) * g.OW0 + g.ox0 + ow * g.oxs] = acc;
}

// LDS of k_conv2d_f32_dma: two buffers (weight tile [kc][BOC], patch rounded up to whole requests of 256 cells) and the
// patch offsets of the kc taps.
inline size_t dma_lds_bytes(int kc, size_t plen, int BOC)
{
   return (2 * ((size_t)kc * BOC + ((plen + 255) & ~(size_t)255)) + kc) * 4;
}

// LDS a workgroup of k_conv2d_f32_dma may use: the CU's 160 KB over the number of workgroups it should hold. Three by
// default (while one waits for its next channel block two keep the matrix cores busy: 2.66 ms at 64 KB, 1.99 ms at
// 52 KB on 256x64x56x56 -> 128); more, with smaller channel blocks, when that lets a grid of few workgroups run in
// whole rounds (the 1792 workgroups of a 64-image 28x28 -> 56x56 transposed layer: 7 per CU in one round instead of
// 3 + 3 + 1, 145 against 162 us). max_resident: what the kernel's registers allow (7 with 32 accumulators, 3 with 128).
inline size_t dma_lds_budget(const sofie_hip_ctx *ctx, size_t workgroups, int max_resident)
{
   const size_t cus = ctx->num_cus > 0 ? (size_t)ctx->num_cus : 256;
   int best = 3;
   double best_fill = 0.0;
   for (int r = 3; r <= max_resident; ++r) {
      const size_t slots = cus * r, rounds = (workgroups + slots - 1) / slots;
      const double fill = (double)workgroups / (double)(rounds * slots);
      if (fill > best_fill + 0.02) {
         best = r;
         best_fill = fill;
      }
   }
   return best == 3 ? (size_t)52 * 1024 : (size_t)(160 * 1024) / best - 512;
}

template <int TI, int TJ>
int launch(sofie_hip_ctx *ctx, ConvArgs &g, bool *done)
{
   constexpr int BOC = 2 * TI * 32, BP = 2 * TJ * 32, LDW = BOC + 1;
   const int KHW = g.KH * g.KW;
   const int OHW = g.OH * g.OW;
   g.rows_out = (BP + g.OW - 2) / g.OW + 1;
   if (g.rows_out > g.OH) g.rows_out = g.OH;
   g.PH = (g.rows_out - 1) * g.sh + (g.KH - 1) * g.dh + 1;
   g.PW = (g.OW - 1) * g.sw + (g.KW - 1) * g.dw + 1;
   // Three workgroups per CU (160 KB of LDS): while one stages its next channel block the other two
   // keep the matrix cores busy. Measured on 256x64x56x56 -> 128, 3x3: 2.66 ms at 64 KB, 1.99 ms at 52 KB.
   const size_t budget = 52 * 1024;
   *done = false;
   const int octiles = cdiv(g.ocg, BOC);
   if ((size_t)g.groups * octiles > 65535 || g.N > 65535) return SOFIE_HIP_OK;
   if (!g.transposed) {
      // First choice: operands by LDS-DMA under the matrix loop (k_conv2d_f32_dma), on a copy of the weights laid out
      // for it (a small kernel in front). The largest full channel block with an even K whose two LDS buffers fit the
      // budget; at least nine K-steps of matrix work per block.
      const size_t HW = (size_t)g.H * g.W;
      const int wstride = (g.ocg + 3) & ~3;
      const size_t wt_floats = (size_t)g.groups * g.icg * KHW * wstride;
      const size_t budget = dma_lds_budget(ctx, (size_t)cdiv(OHW, BP) * g.groups * octiles * g.N, TI == 1 ? 7 : 3);
      if ((size_t)g.icg * HW * 4 < (1u << 30) && (size_t)g.icg * KHW * wstride * 4 < (1u << 30) &&
          (size_t)g.ocg * OHW * 4 < (1u << 30)) {
         auto pick = [&](bool even) {
            for (int icb = g.icg < 96 / KHW ? g.icg : 96 / KHW; icb >= 1; --icb) {
               const int kc = icb * KHW;
               if (kc < 16) break;
               if (g.icg % icb != 0 || kc % 2 != 0 || (even && icb % 2 != 0) ||
                   dma_lds_bytes(kc, (size_t)icb * g.PH * g.PW, BOC) > budget || (size_t)icb * g.PH * g.PW > SOFIE_CONV_DMA_PATCH)
                  continue;
               return icb;
            }
            return 0;
         };
         // kernels 1 to 3 columns wide without dilation along them run without the table of patch offsets, on even
         // channel blocks with K ordered by channel pairs
         const int kwt = g.KW == 1 || ((g.KW == 2 || g.KW == 3) && g.dw == 1) ? g.KW : 0;
         int icb = kwt ? pick(true) : 0;
         const bool pairs = icb > 0;
         if (!icb) icb = pick(false);
         if (icb) {
            g.ICB = icb;
            g.KC = icb * KHW;
            g.dPW = make_fastdiv((unsigned)g.PW);
            g.dPH = make_fastdiv((unsigned)g.PH);
            // Tiles for at most two thirds of the compute units (a layer on one image or a few): the channel blocks are dealt to up to 8
            // slices, each a workgroup of its own that writes raw sums, and a second pass adds them (a fixed order)
            const size_t tiles = (size_t)cdiv(OHW, BP) * g.groups * octiles * g.N;
            const int nblocks = g.icg / icb;
            int csplit = 1;
            if (tiles * 3 <= (size_t)ctx->num_cus * 2 && nblocks >= 2) {   // nearer to one tile per compute unit the second pass costs what the slices gain
               int want = (int)cdiv(2 * ctx->num_cus, (int)tiles);   // more slices measured slower (one 56x56 image: 22.8 against 19.3 us)
               if (want > 8) want = 8;
               if (want > nblocks) want = nblocks;
               while (want > 1 && (size_t)want * g.N * g.OC * OHW * 4 > ((size_t)32 << 20)) --want;   // partial sums of at most 32 MB
               csplit = cdiv(nblocks, cdiv(nblocks, want));
            }
            const size_t out_floats = (size_t)g.N * g.OC * OHW;
            const size_t wbytes = (wt_floats * sizeof(float) + 255) & ~(size_t)255;
            const size_t pbytes = csplit > 1 ? (size_t)csplit * out_floats * sizeof(float) : 0;
            void *ws = nullptr, *ps = nullptr;
            bool fresh = true;
            const int layout[] = {1, g.groups, g.ocg, g.icg, g.KH, g.KW, wstride, pairs ? 1 : 0};
            if (int rc = packed_weights(ctx, g.w, layout_key(layout, 8), wt_floats * sizeof(float), &ws, &fresh)) return rc;
            if (pbytes) {
               if (fresh && ws == ctx->workspace) {
                  // the copy of the weights sits in the context's scratch buffer: the partial sums go behind it
                  if (int rc = workspace(ctx, wbytes + pbytes, &ws)) return rc;
                  ps = static_cast<unsigned char *>(ws) + wbytes;
               } else if (int rc = workspace(ctx, pbytes, &ps)) return rc;
            }
            if (fresh) {
               hipLaunchKernelGGL(k_transpose_weights, dim3((unsigned)((wt_floats + 255) / 256)), dim3(256), 0, ctx->stream, g.w,
                                  static_cast<float *>(ws), g.groups, g.ocg, g.icg * KHW, wstride, pairs ? 1 : 0, KHW);
               if (int rc = check_launch(ctx, "k_transpose_weights")) return rc;
            }
            ConvArgs h = g;
            h.w = static_cast<const float *>(ws);
            h.csplit = csplit;
            h.partial = static_cast<float *>(ps);
            constexpr auto kern0 = k_conv2d_f32_dma<TI, TJ, false, 0>, kern1 = k_conv2d_f32_dma<TI, TJ, false, 1>,
                           kern2 = k_conv2d_f32_dma<TI, TJ, false, 2>, kern3 = k_conv2d_f32_dma<TI, TJ, false, 3>;
            SOFIE_LARGE_LDS(kern0);
            SOFIE_LARGE_LDS(kern1);
            SOFIE_LARGE_LDS(kern2);
            SOFIE_LARGE_LDS(kern3);
            const auto kern = !pairs ? kern0 : kwt == 1 ? kern1 : kwt == 2 ? kern2 : kern3;
            hipLaunchKernelGGL(kern, dim3(cdiv(OHW, BP), g.groups * octiles, g.N * csplit), dim3(256),
                               dma_lds_bytes(g.KC, (size_t)icb * g.PH * g.PW, BOC), ctx->stream, h);
            *done = true;
            if (int rc = check_launch(ctx, pairs ? "k_conv2d_f32_dma_pairs" : "k_conv2d_f32_dma")) return rc;
            if (csplit == 1) return SOFIE_HIP_OK;
            hipLaunchKernelGGL(k_conv_f32_split_finish, dim3((unsigned)((out_floats + 255) / 256)), dim3(256), 0, ctx->stream,
                               h.partial, g.y, g.bias, csplit, out_floats, OHW, g.OC, g.relu);
            return check_launch(ctx, "k_conv_f32_split_finish");
         }
      }
   }
   int icb = 96 / KHW;
   if (icb < 1) icb = 1;
   if (icb > g.icg) icb = g.icg;
   size_t lds = 0;
   for (; icb >= 1; --icb) {
      const int kc = (icb * KHW + 1) & ~1;
      lds = ((size_t)kc * LDW + (size_t)icb * g.PH * g.PW + kc) * 4;
      if (lds <= budget) {
         g.ICB = icb;
         g.KC = kc;
         break;
      }
   }
   if (icb < 1) return SOFIE_HIP_OK;   // does not fit: caller uses the simple kernel
   g.dPW = make_fastdiv((unsigned)g.PW);
   g.dPH = make_fastdiv((unsigned)g.PH);
   g.dKC = make_fastdiv((unsigned)g.KC);
   g.dK4 = make_fastdiv((unsigned)(g.KC >= 4 ? g.KC / 4 : 1));
   // 16-byte weight loads: every channel block full (no k past the block inside a load), blocks and rows of the
   // [OC, K] matrix 16-byte aligned
   g.wvec = !g.transposed && g.icg % g.ICB == 0 && g.KC == g.ICB * KHW && g.KC % 4 == 0 && (g.icg * KHW) % 4 == 0 &&
            (reinterpret_cast<uintptr_t>(g.w) & 15u) == 0;
   constexpr auto kern_t = k_conv2d_f32<TI, TJ, true>, kern_p = k_conv2d_f32<TI, TJ, false>;
   SOFIE_LARGE_LDS(kern_t);
   SOFIE_LARGE_LDS(kern_p);
   auto kern = g.transposed ? kern_t : kern_p;
   hipLaunchKernelGGL(kern, dim3(cdiv(OHW, BP), g.groups * octiles, g.N), dim3(256), lds, ctx->stream, g);
   *done = true;
   return check_launch(ctx, "k_conv2d_f32");
}

// All output phases of a strided transposed convolution in one launch of k_conv2d_f32<.., true>: every phase gets
// the channel block and patch geometry a launch of its own would get; the grid is as wide as the phase with most
// pixel tiles. *done stays false if a phase does not fit (the caller then launches the phases one by one).
template <int TI, int TJ>
int launch_phases(sofie_hip_ctx *ctx, ConvArgs &g, bool *done)
{
   constexpr int BOC = 2 * TI * 32, BP = 2 * TJ * 32, LDW = BOC + 1;
   const size_t budget = 52 * 1024;
   *done = false;
   const int octiles = cdiv(g.ocg, BOC);
   if ((size_t)g.groups * octiles > 65535 || (size_t)g.N * g.nphases > 65535) return SOFIE_HIP_OK;
   size_t lds_max = 0;
   int tiles_max = 0;
   // First choice: operands by LDS-DMA under the matrix loop, on sub-kernels gathered into the [K][channel] order (a
   // small kernel in front, into the context's scratch buffer). Every phase needs a full channel block with an even K
   // of at least 16 that fits.
   {
      size_t workgroups = 0;
      for (int i = 0; i < g.nphases; ++i)
         workgroups += (size_t)cdiv(g.phase[i].OH * g.phase[i].OW, BP) * g.groups * octiles * g.N;
      const size_t budget = dma_lds_budget(ctx, workgroups, TI == 1 ? 7 : 3);
      const int wstride = (g.ocg + 3) & ~3;
      bool fits = (size_t)g.icg * g.H * g.W * 4 < (1u << 30) && (size_t)g.ocg * g.OH0 * g.OW0 * 4 < (1u << 30);
      // every phase as wide as the others, 1 to 3 columns: the table-free loop on even channel blocks, K by channel pairs
      int kwt = g.phase[0].KW >= 1 && g.phase[0].KW <= 3 ? g.phase[0].KW : 0;
      for (int i = 1; i < g.nphases; ++i)
         if (g.phase[i].KW != kwt) kwt = 0;
      int woff = 0;
      auto plan = [&](bool even) {
         bool ok = fits;
         woff = 0;
         lds_max = 0;
         tiles_max = 0;
         for (int i = 0; i < g.nphases && ok; ++i) {
            PhaseArgs &p = g.phase[i];
            const int KHW = p.KH * p.KW;
            p.rows_out = (BP + p.OW - 2) / p.OW + 1;
            if (p.rows_out > p.OH) p.rows_out = p.OH;
            p.PH = (p.rows_out - 1) + (p.KH - 1) + 1;      // unit stride and dilation inside a phase
            p.PW = (p.OW - 1) + (p.KW - 1) + 1;
            bool found = false;
            for (int icb = g.icg < 96 / KHW ? g.icg : 96 / KHW; icb >= 1 && !found; --icb) {
               const int kc = icb * KHW;
               const size_t plen = (size_t)icb * p.PH * p.PW;
               const size_t lds = dma_lds_bytes(kc, plen, BOC);
               if (kc < 16) break;
               if (g.icg % icb != 0 || kc % 2 != 0 || (even && icb % 2 != 0) || lds > budget || plen > SOFIE_CONV_DMA_PATCH) continue;
               p.ICB = icb;
               p.KC = kc;
               p.dPW = make_fastdiv((unsigned)p.PW);
               p.dPH = make_fastdiv((unsigned)p.PH);
               p.dOW = make_fastdiv((unsigned)p.OW);
               if (lds > lds_max) lds_max = lds;
               found = true;
            }
            ok = found && (size_t)g.icg * KHW * wstride * 4 < (1u << 30);
            p.woff = woff;
            woff += g.groups * g.icg * KHW * wstride;       // a multiple of 4 floats
            if (cdiv(p.OH * p.OW, BP) > tiles_max) tiles_max = cdiv(p.OH * p.OW, BP);
         }
         return ok;
      };
      const bool pairs = kwt && plan(true);
      if (pairs || plan(false)) {
         void *ws = nullptr;
         bool fresh = true;
         int layout[12 + 6 * SOFIE_CONV_MAX_PHASES] = {2, g.groups, g.ocg, g.icg, g.KH0, g.KW0, g.ths, g.tws, wstride, pairs ? 1 : 0, g.nphases, woff};
         for (int i = 0; i < g.nphases; ++i) {
            const PhaseArgs &q = g.phase[i];
            const int v[6] = {q.KH, q.KW, q.th0, q.tw0, q.woff, i};
            for (int e = 0; e < 6; ++e) layout[12 + 6 * i + e] = v[e];
         }
         if (int rc = packed_weights(ctx, g.w, layout_key(layout, 12 + 6 * g.nphases), (size_t)woff * sizeof(float), &ws, &fresh)) return rc;
         // fewer tiles than compute units: slices of the channel blocks as in the plain convolution
         int csplit = 1, min_blocks = g.icg;
         for (int i = 0; i < g.nphases; ++i)
            if (g.icg / g.phase[i].ICB < min_blocks) min_blocks = g.icg / g.phase[i].ICB;
         const size_t out_floats = (size_t)g.N * g.OC * g.OH0 * g.OW0;
         if (workgroups * 3 <= (size_t)ctx->num_cus * 2 && min_blocks >= 2 && (size_t)g.N * g.nphases * 8 <= 65535) {
            int want = (int)cdiv(2 * ctx->num_cus, (int)workgroups);
            if (want > 8) want = 8;
            if (want > min_blocks) want = min_blocks;
            while (want > 1 && (size_t)want * out_floats * 4 > ((size_t)32 << 20)) --want;
            csplit = want;
         }
         void *ps = nullptr;
         if (csplit > 1) {
            const size_t wbytes = ((size_t)woff * sizeof(float) + 255) & ~(size_t)255, pbytes = (size_t)csplit * out_floats * sizeof(float);
            if (fresh && ws == ctx->workspace) {
               if (int rc = workspace(ctx, wbytes + pbytes, &ws)) return rc;
               ps = static_cast<unsigned char *>(ws) + wbytes;
            } else if (int rc = workspace(ctx, pbytes, &ps)) return rc;
         }
         if (fresh) {
            hipLaunchKernelGGL(k_gather_phase_weights, dim3((unsigned)cdiv(woff, 256)), dim3(256), 0, ctx->stream, g,
                               static_cast<float *>(ws), woff, wstride, pairs ? 1 : 0);
            if (int rc = check_launch(ctx, "k_gather_phase_weights")) return rc;
         }
         ConvArgs h = g;
         h.w = static_cast<const float *>(ws);
         h.csplit = csplit;
         h.partial = static_cast<float *>(ps);
         constexpr auto kern0 = k_conv2d_f32_dma<TI, TJ, true, 0>, kern1 = k_conv2d_f32_dma<TI, TJ, true, 1>,
                        kern2 = k_conv2d_f32_dma<TI, TJ, true, 2>, kern3 = k_conv2d_f32_dma<TI, TJ, true, 3>;
         SOFIE_LARGE_LDS(kern0);
         SOFIE_LARGE_LDS(kern1);
         SOFIE_LARGE_LDS(kern2);
         SOFIE_LARGE_LDS(kern3);
         const auto kern = !pairs ? kern0 : kwt == 1 ? kern1 : kwt == 2 ? kern2 : kern3;
         hipLaunchKernelGGL(kern, dim3(tiles_max, g.groups * octiles, g.N * g.nphases * csplit), dim3(256), lds_max, ctx->stream, h);
         *done = true;
         if (int rc = check_launch(ctx, pairs ? "k_conv2d_f32_dma_pairs_phases" : "k_conv2d_f32_dma_phases")) return rc;
         if (csplit == 1) return SOFIE_HIP_OK;
         hipLaunchKernelGGL(k_conv_f32_split_finish, dim3((unsigned)((out_floats + 255) / 256)), dim3(256), 0, ctx->stream,
                            h.partial, g.y, g.bias, csplit, out_floats, g.OH0 * g.OW0, g.OC, g.relu);
         return check_launch(ctx, "k_conv_f32_split_finish");
      }
      lds_max = 0;
      tiles_max = 0;
   }
   for (int i = 0; i < g.nphases; ++i) {
      PhaseArgs &p = g.phase[i];
      const int KHW = p.KH * p.KW;
      p.rows_out = (BP + p.OW - 2) / p.OW + 1;
      if (p.rows_out > p.OH) p.rows_out = p.OH;
      p.PH = (p.rows_out - 1) + (p.KH - 1) + 1;      // unit stride and dilation inside a phase
      p.PW = (p.OW - 1) + (p.KW - 1) + 1;
      int icb = 96 / KHW;
      if (icb < 1) icb = 1;
      if (icb > g.icg) icb = g.icg;
      size_t lds = 0;
      for (; icb >= 1; --icb) {
         const int kc = (icb * KHW + 1) & ~1;
         lds = ((size_t)kc * LDW + (size_t)icb * p.PH * p.PW + kc) * 4;
         if (lds <= budget) {
            p.ICB = icb;
            p.KC = kc;
            break;
         }
      }
      if (icb < 1) return SOFIE_HIP_OK;
      p.dPW = make_fastdiv((unsigned)p.PW);
      p.dPH = make_fastdiv((unsigned)p.PH);
      p.dKC = make_fastdiv((unsigned)p.KC);
      p.dOW = make_fastdiv((unsigned)p.OW);
      if (lds > lds_max) lds_max = lds;
      if (cdiv(p.OH * p.OW, BP) > tiles_max) tiles_max = cdiv(p.OH * p.OW, BP);
   }
   g.wvec = 0;
   g.dK4 = make_fastdiv(1u);
   constexpr auto kern = k_conv2d_f32<TI, TJ, true>;
   SOFIE_LARGE_LDS(kern);
   hipLaunchKernelGGL(kern, dim3(tiles_max, g.groups * octiles, g.N * g.nphases), dim3(256), lds_max, ctx->stream, g);
   *done = true;
   return check_launch(ctx, "k_conv2d_f32_phases");
}

int run_conv(sofie_hip_ctx *ctx, ConvArgs &g)
{
   if (g.KH0 == 0) {   // identity tap and output maps
      g.KH0 = g.KH; g.KW0 = g.KW;
      g.th0 = g.transposed ? g.KH - 1 : 0; g.ths = g.transposed ? -1 : 1;
      g.tw0 = g.transposed ? g.KW - 1 : 0; g.tws = g.transposed ? -1 : 1;
      g.OH0 = g.OH; g.OW0 = g.OW; g.oy0 = 0; g.oys = 1; g.ox0 = 0; g.oxs = 1;
   }
   g.dUH = make_fastdiv((unsigned)(g.uh > 0 ? g.uh : 1));
   g.dUW = make_fastdiv((unsigned)(g.uw > 0 ? g.uw : 1));
   g.dOW = make_fastdiv((unsigned)g.OW);
   bool done = false;
   int rc;
   // 128 channels x 128 pixels per workgroup where that gives every compute unit a tile, else 64 x 128, else 64 x 64: a
   // layer on one image or a few has too few of the large tiles to fill the device (one 56x56 image, 64 -> 128
   // channels: 25 tiles of 128 x 128, 98 of 64 x 64)
   const size_t pixels = (size_t)g.OH * g.OW;
   auto tiles = [&](int boc, int bp) { return (size_t)cdiv((int)pixels, bp) * g.groups * cdiv(g.ocg, boc) * g.N; };
   if (g.ocg > 64 && tiles(128, 128) >= (size_t)ctx->num_cus) rc = launch<2, 2>(ctx, g, &done);
   else if (tiles(64, 128) >= (size_t)ctx->num_cus) rc = launch<1, 2>(ctx, g, &done);
   else rc = launch<1, 1>(ctx, g, &done);
   if (rc || done) return rc;
   const size_t total = (size_t)g.N * g.OC * g.OH * g.OW;
   hipLaunchKernelGGL(k_conv2d_f32_simple, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, g);
   return check_launch(ctx, "k_conv2d_f32_simple");
}

struct Conv3dArgs {
   const float *x, *w, *bias;
   float *y;
   int N, C, D, H, W, OC, KD, KH, KW, pd, ph, pw, sd, sh, sw, dd, dh, dw, OD, OH, OW, icg, ocg, relu;
};

// 3-D convolution, one thread per output element; the sum runs over (input channel, kd, kh, kw) in this order
// with separately rounded products and sums, the order of the column matrix the reference multiplies
// (Im2col_3d, SOFIE_common.hxx:522-580, then sgemm_). Consecutive threads take consecutive output columns, so the
// input reads of a wavefront are contiguous and its weight reads are one address.
__global__ void __launch_bounds__(256) k_conv3d_f32(Conv3dArgs g)
{
   const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
   const size_t total = (size_t)g.N * g.OC * g.OD * g.OH * g.OW;
   if (idx >= total) return;
   size_t r = idx;
   const int ow = (int)(r % g.OW); r /= g.OW;
   const int oh = (int)(r % g.OH); r /= g.OH;
   const int od = (int)(r % g.OD); r /= g.OD;
   const int oc = (int)(r % g.OC);
   const int n = (int)(r / g.OC);
   const int grp = oc / g.ocg;
   float acc = 0.0f;
   for (int ic = 0; ic < g.icg; ++ic) {
      const float *xc = g.x + ((size_t)n * g.C + grp * g.icg + ic) * g.D * g.H * g.W;
      const float *wc = g.w + ((size_t)oc * g.icg + ic) * g.KD * g.KH * g.KW;
      for (int kd = 0; kd < g.KD; ++kd) {
         const int id = od * g.sd - g.pd + kd * g.dd;
         if (id < 0 || id >= g.D) continue;
         for (int kh = 0; kh < g.KH; ++kh) {
            const int ih = oh * g.sh - g.ph + kh * g.dh;
            if (ih < 0 || ih >= g.H) continue;
            for (int kw = 0; kw < g.KW; ++kw) {
               const int iw = ow * g.sw - g.pw + kw * g.dw;
               if (iw < 0 || iw >= g.W) continue;
               acc = __fadd_rn(acc, __fmul_rn(xc[((size_t)id * g.H + ih) * g.W + iw], wc[(kd * g.KH + kh) * g.KW + kw]));
            }
         }
      }
   }
   if (g.bias) acc = __fadd_rn(acc, g.bias[oc]);
   if (g.relu) acc = acc > 0.0f ? acc : 0.0f;
   g.y[idx] = acc;
}

}  // namespace

extern "C" int sofie_hip_conv3d_f32(sofie_hip_ctx *ctx, const float *x, const float *w, const float *bias, float *y,
                                    int N, int C, int D, int H, int W, int OC, int KD, int KH, int KW, int pad_d,
                                    int pad_h, int pad_w, int stride_d, int stride_h, int stride_w, int dil_d, int dil_h,
                                    int dil_w, int groups, int act)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C > 0 && D > 0 && H > 0 && W > 0 && OC > 0 && KD > 0 && KH > 0 && KW > 0,
                 "non-positive dimension");
   SOFIE_REQUIRE(ctx, pad_d >= 0 && pad_h >= 0 && pad_w >= 0 && stride_d > 0 && stride_h > 0 && stride_w > 0 && dil_d > 0 &&
                         dil_h > 0 && dil_w > 0,
                 "bad pads/strides/dilations");
   SOFIE_REQUIRE(ctx, groups > 0 && C % groups == 0 && OC % groups == 0, "channels not divisible by groups");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   const int ed = dil_d * (KD - 1) + 1, eh = dil_h * (KH - 1) + 1, ew = dil_w * (KW - 1) + 1;
   SOFIE_REQUIRE(ctx, D + 2 * pad_d >= ed && H + 2 * pad_h >= eh && W + 2 * pad_w >= ew, "kernel larger than padded input");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && w && y, "null operand");
   Conv3dArgs g{};
   g.x = x; g.w = w; g.bias = bias; g.y = y;
   g.N = N; g.C = C; g.D = D; g.H = H; g.W = W; g.OC = OC; g.KD = KD; g.KH = KH; g.KW = KW;
   g.pd = pad_d; g.ph = pad_h; g.pw = pad_w; g.sd = stride_d; g.sh = stride_h; g.sw = stride_w;
   g.dd = dil_d; g.dh = dil_h; g.dw = dil_w;
   g.OD = (D + 2 * pad_d - ed) / stride_d + 1;
   g.OH = (H + 2 * pad_h - eh) / stride_h + 1;
   g.OW = (W + 2 * pad_w - ew) / stride_w + 1;
   g.icg = C / groups;
   g.ocg = OC / groups;
   g.relu = act == SOFIE_ACT_RELU;
   const size_t total = (size_t)N * OC * g.OD * g.OH * g.OW;
   SOFIE_REQUIRE(ctx, total < ((size_t)1 << 38), "output too large");
   hipLaunchKernelGGL(k_conv3d_f32, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, g);
   return check_launch(ctx, "k_conv3d_f32");
}

extern "C" int sofie_hip_conv2d_f32(sofie_hip_ctx *ctx, const float *x, const float *w, const float *bias, float *y,
                                    int N, int C, int H, int W, int OC, int KH, int KW, int pad_top, int pad_left,
                                    int pad_bottom, int pad_right, int stride_h, int stride_w, int dil_h, int dil_w,
                                    int groups, int act)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C > 0 && H > 0 && W > 0 && OC > 0 && KH > 0 && KW > 0, "non-positive dimension");
   SOFIE_REQUIRE(ctx, pad_top >= 0 && pad_left >= 0 && pad_bottom >= 0 && pad_right >= 0 && stride_h > 0 && stride_w > 0 &&
                         dil_h > 0 && dil_w > 0, "bad pads/strides/dilations");
   SOFIE_REQUIRE(ctx, groups > 0 && C % groups == 0 && OC % groups == 0, "channels not divisible by groups");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   const int eh = dil_h * (KH - 1) + 1, ew = dil_w * (KW - 1) + 1;
   SOFIE_REQUIRE(ctx, H + pad_top + pad_bottom >= eh && W + pad_left + pad_right >= ew, "kernel larger than padded input");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && w && y, "null operand");
   ConvArgs g{};
   g.x = x; g.w = w; g.bias = bias; g.y = y;
   g.N = N; g.C = C; g.H = H; g.W = W; g.OC = OC; g.KH = KH; g.KW = KW;
   // the kernels place the windows by the begin pads; the end pads only decide how many windows there are
   g.ph = pad_top; g.pw = pad_left; g.sh = stride_h; g.sw = stride_w; g.dh = dil_h; g.dw = dil_w; g.groups = groups;
   g.OH = (H + pad_top + pad_bottom - eh) / stride_h + 1;
   g.OW = (W + pad_left + pad_right - ew) / stride_w + 1;
   g.icg = C / groups;
   g.ocg = OC / groups;
   g.relu = act == SOFIE_ACT_RELU;
   return run_conv(ctx, g);
}

extern "C" int sofie_hip_conv_transpose2d_f32(sofie_hip_ctx *ctx, const float *x, const float *w, const float *bias,
                                              float *y, int N, int C, int H, int W, int OC, int KH, int KW, int pad_h,
                                              int pad_w, int stride_h, int stride_w, int dil_h, int dil_w, int groups,
                                              int OH, int OW, int act)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C > 0 && H > 0 && W > 0 && OC > 0 && KH > 0 && KW > 0, "non-positive dimension");
   SOFIE_REQUIRE(ctx, pad_h >= 0 && pad_w >= 0 && stride_h > 0 && stride_w > 0 && dil_h > 0 && dil_w > 0,
                 "bad pads/strides/dilations");
   SOFIE_REQUIRE(ctx, groups > 0 && C % groups == 0 && OC % groups == 0, "channels not divisible by groups");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   // the output may be shorter than the full extent (end padding) or longer by less than a stride (output padding)
   const long full_h = (long)stride_h * (H - 1) + (long)dil_h * (KH - 1) + 1 - pad_h;
   const long full_w = (long)stride_w * (W - 1) + (long)dil_w * (KW - 1) + 1 - pad_w;
   SOFIE_REQUIRE(ctx, OH > 0 && OW > 0 && OH < full_h + stride_h && OW < full_w + stride_w, "output size does not fit the geometry");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && w && y, "null operand");
   ConvArgs g{};
   g.x = x; g.w = w; g.bias = bias; g.y = y;
   g.N = N; g.C = C; g.H = H; g.W = W; g.OC = OC; g.KH = KH; g.KW = KW;
   g.ph = dil_h * (KH - 1) - pad_h;
   g.pw = dil_w * (KW - 1) - pad_w;
   g.sh = 1; g.sw = 1; g.dh = dil_h; g.dw = dil_w; g.groups = groups;
   g.OH = OH; g.OW = OW;
   g.icg = C / groups;
   g.ocg = OC / groups;
   g.relu = act == SOFIE_ACT_RELU;
   g.transposed = 1; g.uh = stride_h; g.uw = stride_w;
   if (dil_h != 1 || dil_w != 1 || (stride_h == 1 && stride_w == 1)) return run_conv(ctx, g);
   // One launch per output phase. Output row oy = ry + stride*q is reached by the reversed taps k0, k0 + stride, ...
   // with (ry - p + k0) divisible by the stride (p = K-1-pad), and tap a reads input row q + a + (ry - p + k0)/stride:
   // a unit-stride correlation over the input as it is, with a sub-kernel of about K/stride taps.
   const int py = KH - 1 - pad_h, px = KW - 1 - pad_w;
   // the launch geometry of one phase: tap (a, b) of the phase is element (th0 + a*ths, tw0 + b*tws) of the kernel
   auto phase_of = [&](int ry, int rx) {
      const int k0y = (((py - ry) % stride_h) + stride_h) % stride_h, k0x = (((px - rx) % stride_w) + stride_w) % stride_w;
      ConvArgs p = g;
      p.uh = 1; p.uw = 1;
      p.KH0 = KH; p.KW0 = KW;
      p.KH = k0y < KH ? (KH - 1 - k0y) / stride_h + 1 : 0;
      p.KW = k0x < KW ? (KW - 1 - k0x) / stride_w + 1 : 0;
      p.th0 = KH - 1 - k0y; p.ths = -stride_h;
      p.tw0 = KW - 1 - k0x; p.tws = -stride_w;
      p.ph = -((ry - py + k0y) / stride_h);
      p.pw = -((rx - px + k0x) / stride_w);
      p.OH0 = OH; p.OW0 = OW; p.oy0 = ry; p.oys = stride_h; p.ox0 = rx; p.oxs = stride_w;
      p.OH = (OH - 1 - ry) / stride_h + 1;
      p.OW = (OW - 1 - rx) / stride_w + 1;
      return p;
   };
   // All phases in one launch when there are at most SOFIE_CONV_MAX_PHASES of them and each has taps: a phase on its
   // own fills a fraction of the device (a quarter of the output pixels), and the launches would run one after another.
   {
      ConvArgs all = g;
      all.uh = 1; all.uw = 1;
      all.KH0 = KH; all.KW0 = KW; all.ths = -stride_h; all.tws = -stride_w;
      all.OH0 = OH; all.OW0 = OW; all.oys = stride_h; all.oxs = stride_w;
      all.nphases = 0;
      bool ok = stride_h * stride_w <= SOFIE_CONV_MAX_PHASES;
      for (int ry = 0; ry < stride_h && ok; ++ry)
         for (int rx = 0; rx < stride_w && ok; ++rx) {
            if (ry >= OH || rx >= OW) { ok = false; break; }
            const ConvArgs p = phase_of(ry, rx);
            if (p.KH == 0 || p.KW == 0) { ok = false; break; }
            PhaseArgs &q = all.phase[all.nphases++];
            q.KH = p.KH; q.KW = p.KW; q.th0 = p.th0; q.tw0 = p.tw0; q.ph = p.ph; q.pw = p.pw;
            q.oy0 = p.oy0; q.ox0 = p.ox0; q.OH = p.OH; q.OW = p.OW;
         }
      if (ok && all.nphases > 1) {
         all.dUH = make_fastdiv(1u); all.dUW = make_fastdiv(1u); all.dOW = make_fastdiv(1u);
         bool done = false;
         // tiles as for the plain convolution: the largest that still give every compute unit one
         auto tiles = [&](int boc, int bp) {
            size_t t = 0;
            for (int i = 0; i < all.nphases; ++i) t += (size_t)cdiv(all.phase[i].OH * all.phase[i].OW, bp);
            return t * all.groups * cdiv(all.ocg, boc) * all.N;
         };
         int rc;
         if (all.ocg > 64 && tiles(128, 128) >= (size_t)ctx->num_cus) rc = launch_phases<2, 2>(ctx, all, &done);
         else if (tiles(64, 128) >= (size_t)ctx->num_cus) rc = launch_phases<1, 2>(ctx, all, &done);
         else rc = launch_phases<1, 1>(ctx, all, &done);
         if (rc || done) return rc;
      }
   }
   for (int ry = 0; ry < stride_h; ++ry)
      for (int rx = 0; rx < stride_w; ++rx) {
         if (ry >= OH || rx >= OW) continue;
         ConvArgs p = phase_of(ry, rx);
         if (p.KH == 0 || p.KW == 0) {
            // no tap reaches this phase: the outputs are the bias; the plain kernel's loops run zero times
            p.KH = 0; p.KW = 0;
            p.dUH = make_fastdiv(1u); p.dUW = make_fastdiv(1u); p.dOW = make_fastdiv((unsigned)p.OW);
            const size_t total = (size_t)N * OC * p.OH * p.OW;
            hipLaunchKernelGGL(k_conv2d_f32_simple, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream, p);
            if (int rc = check_launch(ctx, "k_conv2d_f32_simple")) return rc;
            continue;
         }
         if (int rc = run_conv(ctx, p)) return rc;
      }
   return SOFIE_HIP_OK;
}
