// int8 convolution with int32 accumulation and fused requantisation (QLinearConv semantics).
//
// k_qconv_mfma: implicit GEMM on the matrix cores for NHWC activations, weights packed
// [OC][KH][KW][C], groups = 1, C a multiple of 32 and OC a multiple of 64. The GEMM view is
// Y[pixel, oc] = sum_k patch[pixel, k] * w[oc, k] with k = (kh, kw, c), so the NHWC output is
// the row-major GEMM result and shares the GEMM epilogue (requantise, pack four channels per
// lane, 16-byte row stores through an LDS staging block).
//   * 512 threads = 8 wavefronts; each wavefront owns MB x NB accumulator tiles of 32 x 32
//     (v_mfma_i32_32x32x32_i8); a workgroup covers TM = (8/WN)*MB*32 consecutive output pixels
//     of the linear (n, oh, ow) order times WN*NB*32 output channels.
//   * Workgroups are persistent: the workgroup's slice of the weights stays in LDS for its
//     whole life ([oc][K + pad]), and it walks over pixel tiles with a stride of the grid.
//   * The input of a pixel tile is a contiguous band of rows of the zero-point-padded images
//     stacked on top of each other ("virtual rows": image n, padded row r -> n*HP + r). The
//     band is copied once into LDS as [row][padded column][C + pad]; every (kh, kw) tap of
//     every pixel then reads it from there, so HBM/L2 sees each input byte about once per
//     tile instead of KH*KW times. Cells outside the image are written as zp_x.
//   * The band of the NEXT tile is fetched into registers before the MFMA loop of the current
//     one and written to LDS after its epilogue.
// The 16-byte pads make the pixel stride and the weight row stride odd multiples of 16 bytes,
// which keeps the 16-byte-per-lane operand reads of 32 consecutive pixels / channels off the
// same LDS banks.
//
// k_qconv_simple: one thread per output element, any layout / group count / channel count.
#include "common.h"
#include "conv_s8.h"
#include "gemm_tile.h"

using namespace sofie;

namespace {

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
            const int wv = g.w_ohwi ? g.w[(((size_t)oc * g.KH + kh) * g.KW + kw) * g.icg + ic]
                                    : g.w[(((size_t)oc * g.icg + ic) * g.KH + kh) * g.KW + kw];
            acc += xv * wv;
         }
      }
   }
   if (g.bias) acc += g.bias[oc];
   if constexpr (OUT == SOFIE_OUT_S32) static_cast<int *>(g.y)[idx] = acc;
   else static_cast<int8_t *>(g.y)[idx] = (int8_t)requant(acc, g.scale[oc], g.zpy, g.lo);
}

// ------------------------------------------------------------------------------ MFMA path
struct QConvTileArgs {
   const int8_t *x;      // NHWC
   const int8_t *w;      // [OC][KH][KW][C]
   GemmArgs ep;          // Y, scale, bias, M = N*OH*OW, N = OC, ldy = OC, zp, lo, relu
   int H, W, C, KH, KW, ph, pw, sh, sw, OH, OW, HP, WP;
   int K, KS, CS;        // bytes of one weight row, its LDS stride, LDS stride of one pixel
   int RB;               // LDS stride of one band row
   int C16, C32;
   int RL, RP;           // 16-byte chunks per band row; band rows fetched per pass
   int ntiles;
   unsigned fill;        // zp_x replicated into four bytes
   FastDiv dOW, dOH, dHP, dRL, dC16, dK16;
};

// POOL: a 2x2 stride-2 max pooling is fused. A wavefront then owns 32 POOLED pixels; its MB = 4
// accumulator tiles along m are the four positions of the pooling window, so the pooling is a
// register-wise maximum over the four tiles (on the int32 accumulators: the requantisation is monotonic;
// for a negative scale the minimum is taken) and only a quarter of the values is converted and stored.
// In that mode the "pixels" the tiles, the epilogue and a.OH / a.OW / a.ep.M count are pooled pixels.
//
// KFIX: 0 for any kernel size and channel count (the K loop walks taps and channel blocks with run-time
// counters); C/32 (1 or 2) for a 3x3 kernel on 32 or 64 channels. Then the K loop is unrolled over its
// 9*KFIX steps: a fragment address is a per-tile register (pixel, kernel row) plus a constant that goes
// into the offset field of the LDS read, and the loop holds matrix instructions and LDS reads only.
template <int MB, int NB, int WN, int PF, int OUT, bool POOL, int KFIX>
__global__ void __launch_bounds__(512) k_qconv_mfma(QConvTileArgs a)
{
   static_assert(!POOL || MB == 4, "the four window positions are the four m tiles");
   constexpr int WM = 8 / WN;
   constexpr int MBP = POOL ? 1 : MB;                 // m tiles of 32 (pooled) pixels per wavefront
   constexpr int TM = WM * MBP * 32;                  // (pooled) pixels per workgroup tile
   constexpr int RPP = POOL ? 2 : 1;                  // convolution rows per (pooled) row
   constexpr int OCT = WN * NB * 32;
   extern __shared__ __align__(16) unsigned char smem[];
   constexpr int WB = EpilogueStaging<NB, OUT>::WAVE_BYTES;
   unsigned char *const s_w = smem;                                        // [OCT][KS]
   float *const s_scale = reinterpret_cast<float *>(smem + OCT * a.KS);    // [OCT]
   int *const s_bias = reinterpret_cast<int *>(s_scale + OCT);             // [OCT]
   unsigned char *const s_stg = reinterpret_cast<unsigned char *>(s_bias + OCT);   // [8][WB] epilogue staging
   // the int8 epilogue needs no staging (it transposes with lane swaps)
   unsigned char *const s_p = s_stg + (OUT == SOFIE_OUT_S8 ? 0 : 8 * WB);   // band [rows][WP][CS]

   const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
   const int wn = wave % WN, wm = wave / WN;
   const int half = lane >> 5, l32 = lane & 31;
   const int nob = a.ep.N / OCT;
   const int ob = blockIdx.x % nob;
   const int wg = blockIdx.x / nob, nwg = gridDim.x / nob;
   const int mtot = a.ep.M;

   // ---- weights of this channel block: resident for the life of the workgroup
   // The slice is contiguous in global memory (OCT rows of K bytes), so 16-byte chunk q of it sits at wsrc + 16 q and
   // goes to row q / K16, column chunk q % K16 of the padded LDS rows. A thread has up to WCH loads in flight before
   // it writes the first one: one load per store would pay the full memory latency for every chunk, with every
   // workgroup of the launch asking for the same lines at the same time.
   {
      constexpr int WCH = 8;
      const int K16 = a.K >> 4;
      const int total = OCT * K16;
      const int8_t *wsrc = a.w + (size_t)ob * OCT * a.K;
      for (int base = tid; base < total; base += 512 * WCH) {
         v4i chunk[WCH];
#pragma unroll
         for (int u = 0; u < WCH; ++u) {
            const int q = base + u * 512;
            chunk[u] = *reinterpret_cast<const v4i *>(wsrc + (size_t)(q < total ? q : base) * 16);
         }
#pragma unroll
         for (int u = 0; u < WCH; ++u) {
            const int q = base + u * 512;
            const int r = fdiv(q, a.dK16);
            if (q < total) *reinterpret_cast<v4i *>(s_w + r * a.KS + (q - r * K16) * 16) = chunk[u];
         }
      }
   }

   stage_column_params(a.ep, s_scale, s_bias, tid, ob * OCT, OCT);
   const bool plain = OUT == SOFIE_OUT_S8 && a.ep.zp == -128 && a.ep.lo == -128;
   bool any_negative = false;   // pooled variant: some scale of the workgroup's channels is negative (set below)

   // ---- band loader: thread -> (row of the pass, 16-byte chunk of the row)
   const int rsub = fdiv(tid, a.dRL);
   const int col = tid - rsub * a.RL;
   const int wp = fdiv(col, a.dC16);
   const int c16 = col - wp * a.C16;
   const int iw = wp - a.pw;
   const bool col_active = rsub < a.RP;
   const bool col_inside = iw >= 0 && iw < a.W;
   const int src_col = iw * a.C + c16 * 16;
   const int lds_col = wp * a.CS + c16 * 16;
   const int row_bytes = a.RB;
   const v4i fillv = {(int)a.fill, (int)a.fill, (int)a.fill, (int)a.fill};

   struct Band { int vr_lo, rows; };
   auto band_of = [&](int t) {
      const int m0 = t * TM;
      const int mlast = (m0 + TM < mtot ? m0 + TM : mtot) - 1;
      const int R0 = fdiv(m0, a.dOW), R1 = fdiv(mlast, a.dOW);
      const int n0 = fdiv(R0, a.dOH), n1 = fdiv(R1, a.dOH);
      Band b;
      b.vr_lo = n0 * a.HP + (R0 - n0 * a.OH) * RPP * a.sh;
      b.rows = n1 * a.HP + ((R1 - n1 * a.OH) * RPP + RPP - 1) * a.sh + a.KH - b.vr_lo;
      return b;
   };
   v4i pre[PF];
   unsigned pre_inside = 0;    // bit i: pre[i] holds image data (otherwise the cell is padding)
   auto fetch = [&](Band b) {
      pre_inside = 0;
#pragma unroll
      for (int i = 0; i < PF; ++i) {
         const int r = i * a.RP + rsub;
         const int vr = b.vr_lo + r;
         const int n = fdiv(vr, a.dHP);
         const int ih = vr - n * a.HP - a.ph;
         const bool inside = col_active && col_inside && r < b.rows && ih >= 0 && ih < a.H;
         // the load is unconditional (of the first pixel when the cell is outside) and its value is
         // looked at only when it is written to LDS, so all loads of a band are in flight together
         const size_t off = inside ? ((size_t)(n * a.H + ih) * a.W) * a.C + src_col : 0;
         pre[i] = *reinterpret_cast<const v4i *>(a.x + off);
         pre_inside |= inside ? (1u << i) : 0u;
      }
   };
   auto stash = [&](Band b) {
#pragma unroll
      for (int i = 0; i < PF; ++i) {
         const int r = i * a.RP + rsub;
         if (col_active && r < b.rows)
            *reinterpret_cast<v4i *>(s_p + r * row_bytes + lds_col) = ((pre_inside >> i) & 1u) ? pre[i] : fillv;
      }
   };

   int b_off[NB];
#pragma unroll
   for (int i = 0; i < NB; ++i) b_off[i] = ((wn * NB + i) * 32 + l32) * a.KS + half * 16;
   const int tap_step = a.CS - a.C32 * 32;              // from the end of one tap's channels to the next tap
   const int row_step = a.RB - a.KW * a.CS;             // from the end of one kernel row to the next
   const int nsteps = a.KH * a.KW * a.C32;
   const int nq = half * 4;
   const float *const w_scale = s_scale + wn * NB * 32;
   const int *const w_bias = s_bias + wn * NB * 32;
   unsigned char *const w_stg = s_stg + wave * WB;

   // LDS offsets of the wavefront's pixels inside the band of tile tt
   int a_off[MB];
   auto pixel_offsets = [&](int tt, int vr_lo) {
      if constexpr (POOL) {
         int m = tt * TM + wm * 32 + l32;
         m = m < mtot ? m : mtot - 1;
         const int R = fdiv(m, a.dOW);
         const int pw_ = m - R * a.OW;
         const int n = fdiv(R, a.dOH);
         const int v = n * a.HP + (R - n * a.OH) * 2 * a.sh - vr_lo;
#pragma unroll
         for (int j = 0; j < 4; ++j)
            a_off[j] = (v + (j >> 1) * a.sh) * a.RB + (2 * pw_ + (j & 1)) * a.sw * a.CS + half * 16;
      } else {
#pragma unroll
         for (int j = 0; j < MB; ++j) {
            int m = tt * TM + (wm * MB + j) * 32 + l32;
            m = m < mtot ? m : mtot - 1;
            const int R = fdiv(m, a.dOW);
            const int ow = m - R * a.OW;
            const int n = fdiv(R, a.dOH);
            const int v = n * a.HP + (R - n * a.OH) * a.sh - vr_lo;
            a_off[j] = v * a.RB + ow * a.sw * a.CS + half * 16;
         }
      }
   };

   // K loop over (kh, kw, 32-channel block) of one tile into acc; the accumulators start at the
   // bias. Fragments of later steps are read while the matrix instructions of the current step issue.
   // r_bias (unpooled variant): the bias as accumulator tiles, loaded once; it is the C operand of the first
   // step's matrix instructions, which saves copying it into every accumulator of every tile.
   v16i r_bias[POOL ? 1 : NB];
   auto kloop = [&](v16i (&acc)[NB][MB]) {
      v4i fa[POOL ? 2 : 3][MB], fb[POOL ? 2 : 3][NB];
      if constexpr (KFIX > 0) {
         constexpr int NBUF = POOL ? 2 : 3;          // fragment buffers: the reads run NBUF - 1 steps ahead
         constexpr int CSF = KFIX * 32 + 16;         // pixel stride of the band (a.CS) for 32 / 64 channels
         constexpr int NS = 9 * KFIX;
         const unsigned char *pa[3][MB], *pb[NB];
#pragma unroll
         for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int j = 0; j < MB; ++j) pa[kh][j] = s_p + (a_off[j] + kh * a.RB);
#pragma unroll
         for (int i = 0; i < NB; ++i) pb[i] = s_w + b_off[i];
         v16i zero;
#pragma unroll
         for (int e = 0; e < 16; ++e) zero[e] = 0;
#pragma unroll
         for (int s = 0; s < NS + NBUF - 1; ++s) {
            if (s < NS) {
               const int kh = s / (3 * KFIX), kw = (s / KFIX) % 3, cb = s % KFIX;
               // in the order the matrix instructions of the step need them: weights 0, every pixel tile, weights 1...
               fb[s % NBUF][0] = *reinterpret_cast<const v4i *>(pb[0] + s * 32);
#pragma unroll
               for (int j = 0; j < MB; ++j)
                  fa[s % NBUF][j] = *reinterpret_cast<const v4i *>(pa[kh][j] + (kw * CSF + cb * 32));
#pragma unroll
               for (int i = 1; i < NB; ++i) fb[s % NBUF][i] = *reinterpret_cast<const v4i *>(pb[i] + s * 32);
            }
            if (s >= NBUF - 1) {
               const int d = s - (NBUF - 1), buf = d % NBUF;
#pragma unroll
               for (int i = 0; i < NB; ++i)
#pragma unroll
                  for (int j = 0; j < MB; ++j) {
                     if (d == 0) {
                        // the first step starts from the bias tiles (from zero with the fused pooling)
                        if constexpr (POOL) acc[i][j] = MmaI8::mma(fb[buf][i], fa[buf][j], zero);
                        else acc[i][j] = MmaI8::mma(fb[buf][i], fa[buf][j], r_bias[i]);
                     } else {
                        acc[i][j] = MmaI8::mma(fb[buf][i], fa[buf][j], acc[i][j]);
                     }
                  }
            }
            // Pin the order: left alone, the scheduler sinks the fragment reads of a step to just before their first use
            // (or, in the pooled instance, behind all but one of the step's matrix instructions). One read is issued
            // behind each of the first matrix instructions of the step, so every read has at least the rest of the step
            // to land and the reads do not queue up in front of the matrix instructions.
            if (s < NS && s >= NBUF - 1) {
#pragma unroll
               for (int gidx = 0; gidx < MB + NB; ++gidx) {
                  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one matrix instruction
                  __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
               }
               __builtin_amdgcn_sched_group_barrier(0x008, MB * NB - (MB + NB) > 0 ? MB * NB - (MB + NB) : 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
         }
         return;
      }
      int ka = 0, kb = 0, c32 = 0, kw = 0;
      auto advance = [&]() {
         ka += 32; kb += 32;
         if (++c32 == a.C32) {
            c32 = 0; ka += tap_step;
            if (++kw == a.KW) { kw = 0; ka += row_step; }
         }
      };
      auto load = [&](int buf, bool valid) {
         // every fragment load is unconditional (one past the last step re-reads step 0), so that the
         // waits in front of the matrix instructions count exactly
         const int oa = valid ? ka : 0, ob_ = valid ? kb : 0;
#pragma unroll
         for (int j = 0; j < MB; ++j) fa[buf][j] = *reinterpret_cast<const v4i *>(s_p + a_off[j] + oa);
#pragma unroll
         for (int i = 0; i < NB; ++i) fb[buf][i] = *reinterpret_cast<const v4i *>(s_w + b_off[i] + ob_);
      };
      auto mma = [&](int buf) {
#pragma unroll
         for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int j = 0; j < MB; ++j) acc[i][j] = MmaI8::mma(fb[buf][i], fa[buf][j], acc[i][j]);
      };
      if constexpr (!POOL) {
         // three fragment buffers: the reads of step s+2 are issued before the matrix instructions of step s
         load(0, true);
         advance();
         load(1, nsteps > 1);
         // step 0 starts the accumulators from the bias tiles
         advance();
         load(2, nsteps > 2);
         if constexpr (!POOL) {
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
               for (int j = 0; j < MB; ++j) acc[i][j] = MmaI8::mma(fb[0][i], fa[0][j], r_bias[i]);
         }
         int s = 1;   // steps s and s+1 sit in buffers 1 and 2
         for (; s + 2 < nsteps; s += 3) {
            advance();
            load(0, true);
            mma(1);
            advance();
            load(1, s + 3 < nsteps);
            mma(2);
            advance();
            load(2, s + 4 < nsteps);
            mma(0);
         }
         if (s < nsteps) mma(1);
         if (s + 1 < nsteps) mma(2);
      } else {
         // the pooled variant has twice the accumulators and keeps two fragment buffers. Step 0 starts from a
         // constant zero C operand (no accumulator is initialised); the bias is added to the pooled values, a
         // quarter as many (max(a + b) = max(a) + b)
         load(0, true);
         advance();
         load(1, nsteps > 1);
         {
            v16i zero;
#pragma unroll
            for (int e = 0; e < 16; ++e) zero[e] = 0;
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
               for (int j = 0; j < MB; ++j) acc[i][j] = MmaI8::mma(fb[0][i], fa[0][j], zero);
         }
         int s = 1;   // step s sits in buffer 1
         for (; s + 1 < nsteps; s += 2) {
            advance();
            load(0, true);
            mma(1);
            advance();
            load(1, s + 2 < nsteps);
            mma(0);
         }
         if (s < nsteps) mma(1);
      }
   };
   // the lane's scales, loaded once (after the first barrier); the pooled variant needs the registers for
   // its four accumulator tiles and reads the scales from LDS instead
   v4f r_scale[POOL ? 1 : NB * 4];
   auto epilogue = [&](v16i (&acc)[NB][MB], int tt) {
      const int m_wave = tt * TM + wm * MBP * 32, n_wave = ob * OCT + wn * NB * 32;
      if constexpr (POOL) {
         v16i pooled[NB][1];
         if (!any_negative) {
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
               for (int e = 0; e < 16; ++e)
                  pooled[i][0][e] = max(max(acc[i][0][e], acc[i][1][e]), max(acc[i][2][e], acc[i][3][e]));
         } else {
            // a negative scale turns the order around: those channels take the minimum
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
               for (int q = 0; q < 4; ++q) {
                  const v4f sc = *reinterpret_cast<const v4f *>(w_scale + i * 32 + q * 8 + nq);
#pragma unroll
                  for (int t = 0; t < 4; ++t) {
                     const int e = q * 4 + t;
                     const int hi = max(max(acc[i][0][e], acc[i][1][e]), max(acc[i][2][e], acc[i][3][e]));
                     const int lo = min(min(acc[i][0][e], acc[i][1][e]), min(acc[i][2][e], acc[i][3][e]));
                     pooled[i][0][e] = sc[t] < 0.0f ? lo : hi;
                  }
               }
         }
         if constexpr (OUT == SOFIE_OUT_S8) {
            if (plain) tile_epilogue_s8_direct<NB, 1, true, true>(a.ep, pooled, w_scale, w_bias, lane, m_wave, n_wave);
            else tile_epilogue_s8_direct<NB, 1, false, true>(a.ep, pooled, w_scale, w_bias, lane, m_wave, n_wave);
         }
      } else if constexpr (OUT == SOFIE_OUT_S8) {
         if (plain) tile_epilogue_s8_direct<NB, MB, true, false>(a.ep, acc, w_scale, w_bias, lane, m_wave, n_wave, &r_scale);
         else tile_epilogue_s8_direct<NB, MB, false, false>(a.ep, acc, w_scale, w_bias, lane, m_wave, n_wave, &r_scale);
      } else {
         tile_epilogue_wave<MmaI8, NB, MB, OUT, false, false, true>(a.ep, acc, w_stg, w_scale, w_bias, lane, m_wave, n_wave,
                                                                    &r_scale);
      }
   };

   // One tile per iteration. The two wavefronts that share a SIMD do their halves in opposite order
   // (wavefronts 0-3: matrix loop of tile t, then its epilogue; wavefronts 4-7: epilogue of their previous
   // tile, then the matrix loop of tile t), which staggers their LDS and global-memory phases and lets one
   // wavefront's requantisation run beside the other's matrix instructions. That overlap is partial: the counters of
   // the 56x56 layer show vector instructions executing in 40 % of the matrix pipe's busy cycles, and a tile takes
   // about 8000 cycles for 2 x 2304 cycles of matrix instructions per SIMD. A tile is one long chain of instructions
   // per wavefront (about 810, of which 72 are matrix instructions); variants with two band buffers and one barrier
   // per tile, with the band rows' address arithmetic on the scalar unit or in LDS tables, and with three wavefronts
   // per SIMD were all measured and none was faster.
   const bool mma_first = wave < 4;
   int t = wg, t_prev = -1;
   Band cur = {0, 0};
   if (t < a.ntiles) {
      cur = band_of(t);
      fetch(cur);
      pixel_offsets(t, cur.vr_lo);
   }
   // weights and column parameters are in LDS; the pooled variant also learns whether any scale of the
   // workgroup's channels is negative (uniform, so the common case pools with a maximum only)
   __syncthreads();
   if constexpr (POOL) {
      int neg = 0;
      for (int c = tid; c < OCT; c += 512) neg |= s_scale[c] < 0.0f;
      any_negative = __syncthreads_or(neg) != 0;
   }
   if constexpr (!POOL) {
#pragma unroll
      for (int gi = 0; gi < NB * 4; ++gi) {
         r_scale[gi] = *reinterpret_cast<const v4f *>(w_scale + (gi >> 2) * 32 + (gi & 3) * 8 + nq);
         const v4i bi = *reinterpret_cast<const v4i *>(w_bias + (gi >> 2) * 32 + (gi & 3) * 8 + nq);
#pragma unroll
         for (int e = 0; e < 4; ++e) r_bias[gi >> 2][(gi & 3) * 4 + e] = bi[e];
      }
   }
   v16i acc[NB][MB];
   while (t < a.ntiles) {
      stash(cur);
      __syncthreads();                       // the band of tile t is complete
      const int tn = t + nwg;
      const bool more = tn < a.ntiles;
      if (more) cur = band_of(tn);
      if (mma_first) {
         if (more) fetch(cur);
         kloop(acc);
         epilogue(acc, t);
      } else {
         if (t_prev >= 0) epilogue(acc, t_prev);
         if (more) fetch(cur);
         kloop(acc);
      }
      if (more) pixel_offsets(tn, cur.vr_lo);
      t_prev = t;
      t = tn;
      __syncthreads();                       // every wavefront is done reading the band
   }
   if (!mma_first && t_prev >= 0) epilogue(acc, t_prev);
}

// Launches the MFMA kernel if the problem fits it; *done tells whether it did. With g.pool_kh != 0 only the
// kernel with the fused 2x2 stride-2 pooling is considered.
template <int OUT>
int launch_mfma(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done)
{
   *done = false;
   const bool pool = g.pool_kh != 0;
   if constexpr (OUT == SOFIE_OUT_S8) {
      if (int rc = qconv_ring(ctx, g, done)) return rc;
      if (*done) return SOFIE_HIP_OK;
   }
   if (g.groups != 1 || g.C % 32 != 0 || g.OC % 64 != 0 || !g.x_nhwc || !g.y_nhwc || !g.w_ohwi) return SOFIE_HIP_OK;
   if (!aligned16(g.x) || !aligned16(g.w) || !aligned16(g.y)) return SOFIE_HIP_OK;
   if (pool && !(OUT == SOFIE_OUT_S8 && g.pool_kh == 2 && g.pool_kw == 2 && g.pool_sh == 2 && g.pool_sw == 2)) return SOFIE_HIP_OK;
   // rows and columns the tiles count: pooled pixels when the pooling is fused
   const int TH = pool ? g.PH : g.OH, TW = pool ? g.PW : g.OW;
   const int rpp = pool ? 2 : 1;                      // convolution rows per tile row
   const long long mtot = (long long)g.N * TH * TW;
   const int HP = g.H + g.ph + g.pbh, WP = g.W + g.pw + g.pbw;
   if (mtot <= 0) return SOFIE_HIP_OK;
   if (mtot >= (1ll << 31) - 1024 || (long long)g.N * HP >= (1ll << 31) - 4096) return SOFIE_HIP_OK;
   if ((size_t)g.N * g.H * g.W * g.C >= ((size_t)1 << 40)) return SOFIE_HIP_OK;
   const int WN = g.OC % 128 == 0 ? 2 : 1;
   const int OCT = WN * 64;
   const int TM = pool ? (8 / WN) * 32 : (8 / WN) * 64;
   QConvTileArgs a{};
   a.x = g.x; a.w = g.w;
   a.ep.Y = g.y; a.ep.scale = g.scale; a.ep.bias = g.bias;
   a.ep.M = (int)mtot; a.ep.N = g.OC; a.ep.ldy = g.OC;
   a.ep.zp = g.zpy; a.ep.lo = g.lo; a.ep.relu = g.relu; a.ep.s = 1.0f;
   a.ep.vec_store = 1;   // OC % 64 == 0 and y 16-byte aligned
   a.H = g.H; a.W = g.W; a.C = g.C; a.KH = g.KH; a.KW = g.KW; a.ph = g.ph; a.pw = g.pw; a.sh = g.sh; a.sw = g.sw;
   a.OH = TH; a.OW = TW; a.HP = HP; a.WP = WP;
   a.K = g.KH * g.KW * g.C;
   a.KS = ((a.K / 16) % 2 == 0) ? a.K + 16 : a.K;
   a.CS = ((g.C / 16) % 2 == 0) ? g.C + 16 : g.C;
   a.C16 = g.C / 16; a.C32 = g.C / 32;
   a.RL = WP * a.C16;
   if (a.RL > 512) return SOFIE_HIP_OK;
   a.RP = 512 / a.RL;
   a.ntiles = (int)((mtot + TM - 1) / TM);
   a.fill = 0x01010101u * (unsigned)(g.zpx & 0xff);
   a.dOW = make_fastdiv(TW); a.dOH = make_fastdiv(TH); a.dHP = make_fastdiv(HP);
   a.dRL = make_fastdiv(a.RL); a.dC16 = make_fastdiv(a.C16); a.dK16 = make_fastdiv(a.K / 16);
   // most rows a band can have: the convolution rows a tile touches, the image boundaries it can cross
   // (each adds the rows between the last window of one image and the first of the next) and KH - 1
   const int tile_rows = (TM - 1) / TW + 2;
   int gap = HP - TH * rpp * g.sh;
   if (gap < 0) gap = 0;
   int crossings = (tile_rows - 1) / TH + 1;
   if (crossings > g.N - 1) crossings = g.N - 1;
   const long long rows_max = (long long)(tile_rows * rpp - 1) * g.sh + (long long)crossings * gap + g.KH;
   const int passes = (int)((rows_max + a.RP - 1) / a.RP);
   if (passes > 12) return SOFIE_HIP_OK;
   // Band row pitch. Consecutive output pixels sit sw*CS bytes apart; the pitch is padded so that the
   // step from the last pixel of an output row to the first of the next is the same modulo the 256 bytes
   // the LDS banks span. The 16 lanes that read together then keep hitting distinct banks across row ends.
   a.RB = WP * a.CS;
   if (g.sh == 1 && !pool) {
      const int want = (int)(((long long)g.OW * g.sw * a.CS) % 256);
      a.RB += ((want - a.RB % 256) % 256 + 256) % 256;
   }
   const size_t band = (size_t)rows_max * a.RB;
   const size_t staging = OUT == SOFIE_OUT_S8 ? 0 : (size_t)8 * EpilogueStaging<2, OUT>::WAVE_BYTES;
   const size_t lds = (size_t)OCT * a.KS + (size_t)OCT * 8 + staging + band;
   if (lds > 160 * 1024) return SOFIE_HIP_OK;
   if ((size_t)g.OC * a.K >= ((size_t)1 << 31)) return SOFIE_HIP_OK;

   // 3x3 kernels on 32 or 64 channels take the kernels whose K loop is unrolled with constant offsets
   const int kfix = (g.KH == 3 && g.KW == 3 && (g.C == 32 || g.C == 64) && a.CS == g.C + 16) ? g.C / 32 : 0;
   const int nob = g.OC / OCT;
   int per = ctx->num_cus / nob;
   if (per < 1) per = 1;
   if (per > a.ntiles) per = a.ntiles;
   const dim3 grid((unsigned)(per * nob)), block(512);
#define SOFIE_QCONV_LAUNCH_K(MB_, WN_, PF_, POOL_, KFIX_)                                                     \
   do {                                                                                                       \
      constexpr auto kern = k_qconv_mfma<MB_, 2, WN_, PF_, OUT, POOL_, KFIX_>;                                \
      SOFIE_LARGE_LDS(kern);                                                                                  \
      hipLaunchKernelGGL(kern, grid, block, lds, ctx->stream, a);                                             \
   } while (0)
#define SOFIE_QCONV_LAUNCH(MB_, WN_, PF_, POOL_)                                                              \
   do {                                                                                                       \
      if constexpr (OUT != SOFIE_OUT_S8) SOFIE_QCONV_LAUNCH_K(MB_, WN_, PF_, POOL_, 0);                       \
      else if (kfix == 1) SOFIE_QCONV_LAUNCH_K(MB_, WN_, PF_, POOL_, 1);                                      \
      else if (kfix == 2) SOFIE_QCONV_LAUNCH_K(MB_, WN_, PF_, POOL_, 2);                                      \
      else SOFIE_QCONV_LAUNCH_K(MB_, WN_, PF_, POOL_, 0);                                                     \
   } while (0)
#define SOFIE_QCONV_BY_PASSES(MB_, WN_, POOL_)                                                                \
   do {                                                                                                       \
      if constexpr (OUT != SOFIE_OUT_S8) SOFIE_QCONV_LAUNCH(2, WN_, 12, false); /* raw accumulators: not tuned */ \
      else if (passes <= 3) SOFIE_QCONV_LAUNCH(MB_, WN_, 3, POOL_);                                           \
      else if (passes <= 4) SOFIE_QCONV_LAUNCH(MB_, WN_, 4, POOL_);                                           \
      else if (passes <= 5) SOFIE_QCONV_LAUNCH(MB_, WN_, 5, POOL_);                                           \
      else if (passes <= 6) SOFIE_QCONV_LAUNCH(MB_, WN_, 6, POOL_);                                           \
      else if (passes <= 8) SOFIE_QCONV_LAUNCH(MB_, WN_, 8, POOL_);                                           \
      else SOFIE_QCONV_LAUNCH(MB_, WN_, 12, POOL_);                                                           \
   } while (0)
   if (pool) {
      if (WN == 2) SOFIE_QCONV_BY_PASSES(4, 2, true);
      else SOFIE_QCONV_BY_PASSES(4, 1, true);
   } else {
      if (WN == 2) SOFIE_QCONV_BY_PASSES(2, 2, false);
      else SOFIE_QCONV_BY_PASSES(2, 1, false);
   }
#undef SOFIE_QCONV_BY_PASSES
#undef SOFIE_QCONV_LAUNCH
#undef SOFIE_QCONV_LAUNCH_K
   *done = true;
   return check_launch(ctx, "k_qconv_mfma");
}

size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

// The MFMA kernel takes channels-last activations and [OC][KH][KW][C] weights; other layouts of a shape
// it takes are converted through scratch memory of this many bytes.
bool mfma_shape(const QConvArgs &g) { return g.groups == 1 && g.C % 32 == 0 && g.OC % 64 == 0 && g.N <= 65535; }
size_t layout_scratch_bytes(const QConvArgs &g)
{
   if (!mfma_shape(g) || (g.x_nhwc && g.y_nhwc && g.w_ohwi)) return 0;
   return up256(g.x_nhwc ? 0 : (size_t)g.N * g.C * g.H * g.W) + up256(g.y_nhwc ? 0 : (size_t)g.N * g.OC * g.OH * g.OW) +
          up256(g.w_ohwi ? 0 : (size_t)g.OC * g.C * g.KH * g.KW);
}

// Convolution without pooling; scratch has layout_scratch_bytes(g) bytes.
template <int OUT>
int run_conv(sofie_hip_ctx *ctx, const QConvArgs &g, int8_t *scratch)
{
   constexpr int ESZ = OutSize<OUT>::value;
   bool done = false;
   if constexpr (OUT == SOFIE_OUT_S8) {
      if (int rc = qconv_first_layer(ctx, g, &done)) return rc;
      if (done) return SOFIE_HIP_OK;
   }
   if (ESZ == 1 && mfma_shape(g) && (!g.x_nhwc || !g.y_nhwc || !g.w_ohwi)) {
      const size_t xb = g.x_nhwc ? 0 : (size_t)g.N * g.C * g.H * g.W;
      const size_t yb = g.y_nhwc ? 0 : (size_t)g.N * g.OC * g.OH * g.OW;
      const size_t wb = g.w_ohwi ? 0 : (size_t)g.OC * g.C * g.KH * g.KW;
      int8_t *xs = scratch, *ys = xs + up256(xb), *wsb = ys + up256(yb);
      QConvArgs h = g;
      if (xb) {
         if (int rc = relayout_s8(ctx, g.x, xs, g.N, g.C, g.H, g.W, SOFIE_LAYOUT_NCHW, SOFIE_LAYOUT_NHWC)) return rc;
         h.x = xs; h.x_nhwc = 1;
      }
      if (wb) {
         if (int rc = relayout_s8(ctx, g.w, wsb, g.OC, g.C, g.KH, g.KW, SOFIE_LAYOUT_NCHW, SOFIE_LAYOUT_NHWC)) return rc;
         h.w = wsb; h.w_ohwi = 1;
      }
      if (yb) { h.y = ys; h.y_nhwc = 1; }
      if (int rc = launch_mfma<OUT>(ctx, h, &done)) return rc;
      if (done) {
         if (yb) return relayout_s8(ctx, ys, static_cast<int8_t *>(g.y), g.N, g.OC, g.OH, g.OW, SOFIE_LAYOUT_NHWC,
                                    SOFIE_LAYOUT_NCHW);
         return SOFIE_HIP_OK;
      }
   } else {
      if (int rc = launch_mfma<OUT>(ctx, g, &done)) return rc;
      if (done) return SOFIE_HIP_OK;
   }
   const size_t total = (size_t)g.N * g.OC * g.OH * g.OW;
   const dim3 grid((unsigned)((total + 255) / 256)), block(256);
   hipLaunchKernelGGL(k_qconv_simple<OUT>, grid, block, 0, ctx->stream, g);
   return check_launch(ctx, "k_qconv_simple");
}

// Scratch bytes run() needs for g (beyond what the caller may have reserved in front of them).
size_t run_scratch_bytes(const QConvArgs &g)
{
   if (g.pool_kh == 0) return layout_scratch_bytes(g);
   QConvArgs h = g;
   h.pool_kh = h.pool_kw = h.pool_sh = h.pool_sw = 0;
   return up256((size_t)g.N * g.OC * g.OH * g.OW) + layout_scratch_bytes(h);
}

// scratch: run_scratch_bytes(g) bytes of device memory.
template <int OUT>
int run(sofie_hip_ctx *ctx, const QConvArgs &g, int8_t *scratch)
{
   if (g.pool_kh == 0) return run_conv<OUT>(ctx, g, scratch);
   // fused kernels first; otherwise the convolution goes to scratch memory in the layout of y and the
   // pooling kernel reads it from there
   bool done = false;
   if (int rc = qconv_first_layer(ctx, g, &done)) return rc;
   if (done) return SOFIE_HIP_OK;
   if (int rc = launch_mfma<OUT>(ctx, g, &done)) return rc;
   if (done) return SOFIE_HIP_OK;
   QConvArgs h = g;
   h.pool_kh = h.pool_kw = h.pool_sh = h.pool_sw = 0;
   h.PH = g.OH; h.PW = g.OW;
   const size_t conv_bytes = up256((size_t)g.N * g.OC * g.OH * g.OW);
   h.y = scratch;
   if (int rc = run_conv<OUT>(ctx, h, scratch + conv_bytes)) return rc;
   return sofie_hip_maxpool2d_s8(ctx, scratch, static_cast<int8_t *>(g.y),
                                 g.y_nhwc ? SOFIE_LAYOUT_NHWC : SOFIE_LAYOUT_NCHW, g.N, g.OC, g.OH, g.OW, g.pool_kh,
                                 g.pool_kw, 0, 0, 0, 0, g.pool_sh, g.pool_sw);
}

template <int OUT>
int run(sofie_hip_ctx *ctx, const QConvArgs &g)
{
   void *ws = nullptr;
   const size_t need = run_scratch_bytes(g);
   if (need)
      if (int rc = workspace(ctx, need, &ws)) return rc;
   return run<OUT>(ctx, g, static_cast<int8_t *>(ws));
}

int fill_args(sofie_hip_ctx *ctx, QConvArgs &g, const int8_t *x, int x_layout, const int8_t *w, int w_layout,
              const int32_t *bias, const float *scale, void *y, int y_layout, int N, int C, int H, int W, int OC, int KH,
              int KW, int pad_top, int pad_left, int pad_bottom, int pad_right, int stride_h, int stride_w, int groups,
              int zp_x, int zp_y, int act, int out_kind)
{
   SOFIE_REQUIRE(ctx, N >= 0 && C > 0 && H > 0 && W > 0 && OC > 0 && KH > 0 && KW > 0, "non-positive dimension");
   SOFIE_REQUIRE(ctx, pad_top >= 0 && pad_left >= 0 && pad_bottom >= 0 && pad_right >= 0 && stride_h > 0 && stride_w > 0,
                 "bad pads/strides");
   SOFIE_REQUIRE(ctx, groups > 0 && C % groups == 0 && OC % groups == 0, "channels not divisible by groups");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   SOFIE_REQUIRE(ctx, (x_layout == SOFIE_LAYOUT_NCHW || x_layout == SOFIE_LAYOUT_NHWC) &&
                         (y_layout == SOFIE_LAYOUT_NCHW || y_layout == SOFIE_LAYOUT_NHWC) &&
                         (w_layout == SOFIE_LAYOUT_NCHW || w_layout == SOFIE_LAYOUT_NHWC), "unknown layout");
   SOFIE_REQUIRE(ctx, out_kind == SOFIE_OUT_S8 || out_kind == SOFIE_OUT_S32, "output kind must be S8 or S32");
   SOFIE_REQUIRE(ctx, zp_x >= -128 && zp_x <= 127 && zp_y >= -128 && zp_y <= 127, "zero-point out of int8 range");
   SOFIE_REQUIRE(ctx, H + pad_top + pad_bottom >= KH && W + pad_left + pad_right >= KW, "kernel larger than padded input");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, w && y, "null operand");
   SOFIE_REQUIRE(ctx, scale || out_kind == SOFIE_OUT_S32, "scale is required for S8 output");
   g.x = x; g.w = w; g.bias = bias; g.scale = scale; g.y = y;
   g.N = N; g.C = C; g.H = H; g.W = W; g.OC = OC; g.KH = KH; g.KW = KW;
   g.ph = pad_top; g.pw = pad_left; g.pbh = pad_bottom; g.pbw = pad_right;
   g.sh = stride_h; g.sw = stride_w; g.groups = groups;
   g.OH = (H + pad_top + pad_bottom - KH) / stride_h + 1;
   g.OW = (W + pad_left + pad_right - KW) / stride_w + 1;
   g.PH = g.OH; g.PW = g.OW;
   g.icg = C / groups;
   g.ocg = OC / groups;
   g.zpx = zp_x; g.zpy = zp_y;
   g.relu = act == SOFIE_ACT_RELU;
   g.lo = (g.relu && zp_y > -128) ? zp_y : -128;
   // with one channel (one output channel) both activation layouts are the same bytes
   g.x_nhwc = x_layout == SOFIE_LAYOUT_NHWC || C == 1;
   g.y_nhwc = y_layout == SOFIE_LAYOUT_NHWC || OC == 1;
   g.w_ohwi = w_layout == SOFIE_LAYOUT_NHWC || g.icg == 1 || KH * KW == 1;
   return SOFIE_HIP_OK;
}

}  // namespace

extern "C" int sofie_hip_qconv2d_s8(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, const int8_t *w, int w_layout,
                                    const int32_t *bias, const float *scale, void *y, int y_layout, int N, int C,
                                    int H, int W, int OC, int KH, int KW, int pad_top, int pad_left, int pad_bottom,
                                    int pad_right, int stride_h, int stride_w, int groups, int zp_x, int zp_y, int act,
                                    int out_kind)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   QConvArgs g{};
   if (int rc = fill_args(ctx, g, x, x_layout, w, w_layout, bias, scale, y, y_layout, N, C, H, W, OC, KH, KW, pad_top, pad_left,
                          pad_bottom, pad_right, stride_h, stride_w, groups, zp_x, zp_y, act, out_kind))
      return rc;
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x, "null operand");
   if (out_kind == SOFIE_OUT_S32) return run<SOFIE_OUT_S32>(ctx, g);
   return run<SOFIE_OUT_S8>(ctx, g);
}

extern "C" int sofie_hip_qconv2d_pool_s8(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, const int8_t *w,
                                         int w_layout, const int32_t *bias, const float *scale, int8_t *y, int y_layout,
                                         int N, int C, int H, int W, int OC, int KH, int KW, int pad_top, int pad_left,
                                         int pad_bottom, int pad_right, int stride_h, int stride_w, int groups, int zp_x,
                                         int zp_y, int act,
                                         int pool_kh, int pool_kw, int pool_stride_h, int pool_stride_w)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   QConvArgs g{};
   if (int rc = fill_args(ctx, g, x, x_layout, w, w_layout, bias, scale, y, y_layout, N, C, H, W, OC, KH, KW, pad_top, pad_left,
                          pad_bottom, pad_right, stride_h, stride_w, groups, zp_x, zp_y, act, SOFIE_OUT_S8))
      return rc;
   SOFIE_REQUIRE(ctx, pool_kh > 0 && pool_kw > 0 && pool_stride_h > 0 && pool_stride_w > 0, "bad pooling window");
   SOFIE_REQUIRE(ctx, pool_kh <= g.OH && pool_kw <= g.OW, "pooling window larger than the convolution output");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x, "null operand");
   g.pool_kh = pool_kh; g.pool_kw = pool_kw; g.pool_sh = pool_stride_h; g.pool_sw = pool_stride_w;
   g.PH = (g.OH - pool_kh) / pool_stride_h + 1;
   g.PW = (g.OW - pool_kw) / pool_stride_w + 1;
   return run<SOFIE_OUT_S8>(ctx, g);
}

extern "C" int sofie_hip_qconv2d_s8_chain(sofie_hip_ctx *ctx, const int8_t *x, int x_layout, int N, int n_layers,
                                          const sofie_hip_qconv_layer *layers)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, n_layers >= 1 && n_layers <= SOFIE_QCONV_CHAIN_MAX && layers, "bad layer list");
   QConvArgs g[SOFIE_QCONV_CHAIN_MAX];
   const int8_t *in = x;
   int in_layout = x_layout;
   for (int l = 0; l < n_layers; ++l) {
      const sofie_hip_qconv_layer &q = layers[l];
      g[l] = QConvArgs{};
      if (int rc = fill_args(ctx, g[l], in, in_layout, q.w, q.w_layout, q.bias, q.scale, q.y, q.y_layout, N, q.C, q.H, q.W, q.OC,
                             q.KH, q.KW, q.pad_top, q.pad_left, q.pad_bottom, q.pad_right, q.stride_h, q.stride_w, q.groups,
                             q.zp_x, q.zp_y, q.act, SOFIE_OUT_S8))
         return rc;
      if (q.pool_kh != 0 || q.pool_kw != 0) {
         SOFIE_REQUIRE(ctx, q.pool_kh > 0 && q.pool_kw > 0 && q.pool_stride_h > 0 && q.pool_stride_w > 0, "bad pooling window");
         SOFIE_REQUIRE(ctx, q.pool_kh <= g[l].OH && q.pool_kw <= g[l].OW, "pooling window larger than the convolution output");
         g[l].pool_kh = q.pool_kh; g[l].pool_kw = q.pool_kw; g[l].pool_sh = q.pool_stride_h; g[l].pool_sw = q.pool_stride_w;
         g[l].PH = (g[l].OH - q.pool_kh) / q.pool_stride_h + 1;
         g[l].PW = (g[l].OW - q.pool_kw) / q.pool_stride_w + 1;
      }
      if (l + 1 < n_layers)
         SOFIE_REQUIRE(ctx, layers[l + 1].C == q.OC && layers[l + 1].H == g[l].PH && layers[l + 1].W == g[l].PW,
                       "a layer's input shape is not the output shape of the layer before it");
      in = q.y;
      in_layout = q.y_layout;
   }
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x, "null operand");
   for (int l = 0; l < n_layers;) {
      if (l + 1 < n_layers) {
         bool done = false;
         if (int rc = qconv_ring_pair(ctx, g[l], g[l + 1], &done)) return rc;
         if (done) {
            l += 2;
            continue;
         }
      }
      if (int rc = run<SOFIE_OUT_S8>(ctx, g[l])) return rc;
      ++l;
   }
   return SOFIE_HIP_OK;
}

extern "C" int sofie_hip_quantize_qconv2d_s8(sofie_hip_ctx *ctx, const float *x, float x_scale, int zp_x, const int8_t *w,
                                             int w_layout, const int32_t *bias, const float *scale, int8_t *y,
                                             int y_layout, int N, int C, int H, int W, int OC, int KH, int KW, int pad_top,
                                             int pad_left, int pad_bottom, int pad_right, int stride_h, int stride_w,
                                             int groups, int zp_y, int act,
                                             int pool_kh, int pool_kw, int pool_stride_h, int pool_stride_w)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, x_scale > 0.0f, "the input scale must be positive");
   QConvArgs g{};
   if (int rc = fill_args(ctx, g, nullptr, SOFIE_LAYOUT_NCHW, w, w_layout, bias, scale, y, y_layout, N, C, H, W, OC, KH, KW,
                          pad_top, pad_left, pad_bottom, pad_right, stride_h, stride_w, groups, zp_x, zp_y, act, SOFIE_OUT_S8))
      return rc;
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x, "null operand");
   const bool pool = pool_kh != 0 || pool_kw != 0;
   if (pool) {
      SOFIE_REQUIRE(ctx, pool_kh > 0 && pool_kw > 0 && pool_stride_h > 0 && pool_stride_w > 0, "bad pooling window");
      SOFIE_REQUIRE(ctx, pool_kh <= g.OH && pool_kw <= g.OW, "pooling window larger than the convolution output");
      g.pool_kh = pool_kh; g.pool_kw = pool_kw; g.pool_sh = pool_stride_h; g.pool_sw = pool_stride_w;
      g.PH = (g.OH - pool_kh) / pool_stride_h + 1;
      g.PW = (g.OW - pool_kw) / pool_stride_w + 1;
   }
   // the first-layer kernel quantizes while it copies the image into LDS
   g.xf = x;
   g.xscale = x_scale;
   bool done = false;
   if (int rc = qconv_first_layer(ctx, g, &done)) return rc;
   if (done) return SOFIE_HIP_OK;
   // otherwise: quantize into scratch memory, then the int8 path
   g.xf = nullptr;
   const size_t xbytes = up256((size_t)N * C * H * W);
   void *ws = nullptr;
   if (int rc = workspace(ctx, xbytes + run_scratch_bytes(g), &ws)) return rc;
   if (int rc = sofie_hip_quantize_f32_s8(ctx, x, static_cast<int8_t *>(ws), (size_t)N * C * H * W, x_scale, zp_x)) return rc;
   g.x = static_cast<const int8_t *>(ws);
   return run<SOFIE_OUT_S8>(ctx, g, static_cast<int8_t *>(ws) + xbytes);
}
