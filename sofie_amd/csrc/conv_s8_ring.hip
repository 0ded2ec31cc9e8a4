// int8 3x3 stride-1 convolution on the matrix cores whose input travels global memory -> LDS without registers.
//
// k_qconv_ring: the implicit GEMM of conv_s8.hip (NHWC activations, weights [OC][3][3][C], C = 32 or 64, the
// workgroup's weight slice resident in LDS, 8 wavefronts of 2 x 2 accumulator tiles of 32 x 32, optionally the fused
// 2x2 pooling) with another way of getting the input there:
//   * a workgroup owns a CONTIGUOUS run of pixels of the linear (n, oh, ow) order, so the rows of the padded
//     images it needs ("virtual rows": image n, padded row r -> n*HP + r) form a window that slides down; they
//     live in a ring of R rows in LDS (row v in slot v % R). A tile only fetches the rows the previous tile did not
//     have, and they are fetched while the previous tile is multiplied: the ring has room for the rows of two
//     consecutive tiles.
//   * rows are fetched with buffer_load_dwordx4 ... lds: a wavefront instruction moves 64 x 16 bytes into 1 KB of
//     consecutive LDS, the global address is free per lane. A ring row is stored as C/16 planes
//     [16-byte channel chunk][padded column][16 bytes]; one instruction fills one plane of one row (lane = padded
//     column), or the whole row where all its planes fit the 64 lanes; lanes of padding columns are switched off.
//     The vector unit spends nothing on staging: no address arithmetic per 16 bytes, no registers, no LDS writes.
//     Padding columns are written once with the input zero-point when the kernel starts, padding rows by one LDS
//     write when such a row enters the ring. The weights arrive the same way.
//   * in a plane consecutive pixels are 16 bytes apart, so the 16-byte-per-lane operand read of consecutive pixels
//     covers consecutive banks; the row pitch is padded so that this also holds across the end of an output row.
//     The nine taps of a pixel are its base address (per kernel row and channel half) plus a constant. With the
//     pooling, where consecutive lanes are two columns apart, a plane holds its even columns first and its odd
//     columns behind them, to the same effect.
#include "common.h"
#include <type_traits>
#include "conv_s8.h"
#include "gemm_tile.h"

using namespace sofie;

namespace {

template <bool B> struct BoolTag { static constexpr bool value = B; };

struct QConvRingArgs {
   const int8_t *x;      // NHWC
   const int8_t *w;      // [OC][3][3][C]
   GemmArgs ep;          // Y, scale, bias, M = N*OH*OW, N = OC, ldy = OC, zp, lo, relu
   int H, W, C, ph, pw, OH, OW, HP, WP;
   int K, KS;            // bytes of one weight row, its LDS stride
   int RS, PL, R;        // ring: row pitch and plane pitch in bytes, rows
   int row_bytes;        // W * C: one image row in global memory
   int units_each, units_rem;   // 64-pixel (32 pooled pixel) units per workgroup of a channel block: quotient and remainder
   int gap;              // HP - OH * (rows per pixel): padded rows between the last window row of an image and the next image
   unsigned fill;        // zp_x replicated into four bytes
   unsigned xbytes;
   FastDiv dOW, dOH, dHP, dKS16, dR, dPL16;   // dPL16: by the 16-byte slots of a plane
};

// The block travels by value as the kernel's argument (and, when a call is recorded into a HIP graph, as a copy inside
// the graph's kernel node): plain data, far below the 4 KB a launch may pass.
static_assert(std::is_trivially_copyable<QConvRingArgs>::value && std::is_standard_layout<QConvRingArgs>::value &&
                 sizeof(QConvRingArgs) <= 512,
              "kernel argument block");

// C16: 16-byte chunks per pixel (2 or 4); WN: wavefronts along the output channels. The tile is (8/WN)*64 pixels x
// WN*64 channels. (Twelve wavefronts per workgroup, three per SIMD, and wavefront tiles of 96 pixels were measured
// on the 56x56 layer: the same time within 1 %.)
// ROWDMA: a whole padded row (all planes) has at most 64 16-byte slots and is fetched by one instruction; otherwise one
// instruction fetches one plane of a row.
// POOL: a 2x2 stride-2 max pooling is fused. A wavefront then owns 32 POOLED pixels; its four accumulator tiles along m
// are the four positions of the pooling window, the pooling is a register-wise maximum of the int32 accumulators (the
// requantisation is monotonic; for a negative scale the minimum is taken) and a quarter of the values is converted and
// stored. In that mode the "pixels" of tiles, runs and a.OH / a.OW / a.ep.M are pooled pixels.
template <int C16, int WN, bool ROWDMA, bool POOL>
__device__ __forceinline__ void qconv_ring_body(const QConvRingArgs &a, unsigned char *smem)
{
   constexpr int NB = 2;
   constexpr int MB = POOL ? 4 : 2;                 // accumulator tiles along m per wavefront
   constexpr int MBP = POOL ? 1 : 2;                // tiles of 32 (pooled) pixels per wavefront
   constexpr int RPP = POOL ? 2 : 1;                // convolution rows (and columns) per (pooled) pixel
   constexpr int NWAVE = 8, NT = NWAVE * 64;
   constexpr bool REGS = !POOL;                     // scales and bias tiles in registers
   // 64 input channels without pooling: v_mfma_i32_16x16x64_i8 (a tap's 64 channels are one instruction's K) instead of
   // two v_mfma_i32_32x32x32_i8. Same multiply-adds per cycle, less power, so a higher clock under the device's limit;
   // and a lane group's four channels of four 16-channel tiles transpose into 64 contiguous bytes per pixel and store.
   constexpr bool M16 = C16 == 4 && !POOL;
   constexpr int NBT = M16 ? 4 : NB, MBT = M16 ? 4 : MB;   // accumulator tiles of a wavefront along channels, pixels
   using AccT = std::conditional_t<M16, v4i, v16i>;
   constexpr int WM = NWAVE / WN;
   constexpr int TM = WM * MBP * 32;
   constexpr int OCT = WN * NB * 32;
   constexpr int CB = C16 / 2;                      // 32-channel blocks
   constexpr int NS = 9 * CB;                       // K steps of 32 bytes
   constexpr int NRL = ROWDMA ? NWAVE : NWAVE / C16;   // wavefronts that share the rows of a request among them
   unsigned char *const s_w = smem;                                        // [OCT][KS]
   float *const s_scale = reinterpret_cast<float *>(smem + OCT * a.KS);    // [OCT]
   int *const s_bias = reinterpret_cast<int *>(s_scale + OCT);             // [OCT]
   unsigned char *const s_ring = reinterpret_cast<unsigned char *>(s_bias + OCT);   // [R][C16][WP][16] (+ row pad)
   const unsigned ring0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)s_ring;

   const int tid = threadIdx.x, lane = tid & 63;
   const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int wn = wave % WN, wm = wave / WN;
   const int half = lane >> 5, l32 = lane & 31;
   const int kg = lane >> 4, l16 = lane & 15;           // 16 x 16 tiles: chunk of K and row / column of the lane
   const int nob = a.ep.N / OCT;
   const int ob = nob == 1 ? 0 : blockIdx.x % nob;
   const int wg = nob == 1 ? blockIdx.x : blockIdx.x / nob;
   // The workgroup's run of pixels, dealt out in units of the 64 pixels a wavefront multiplies: its tiles start at
   // m_begin, and of the last, partial one only the wavefronts whose pixels lie inside the run do any work.
   constexpr int UNIT = MBP * 32;
   // (the first units_rem workgroups of a channel block get units_each + 1 units, the others units_each: no division here)
   const int m_begin = (wg * a.units_each + (wg < a.units_rem ? wg : a.units_rem)) * UNIT;
   const int m_stop = m_begin + (a.units_each + (wg < a.units_rem ? 1 : 0)) * UNIT;
   const int mtot = m_stop < a.ep.M ? m_stop : a.ep.M;       // one past the last pixel of the run
   const int t0 = 0, t1 = (mtot - m_begin + TM - 1) / TM;
   GemmArgs ep = a.ep;
   ep.M = mtot;

   // ---- weights of this channel block: resident for the life of the workgroup. They travel like the input rows, straight
   // into LDS: an instruction fills 64 consecutive 16-byte slots of the padded LDS rows (a row of 36 chunks and its pad,
   // then the start of the next row), lanes on pad slots switched off, and all of a wavefront's requests are in flight
   // together.
   auto stage_weights = [&]() {
      const int K16 = a.K >> 4, KS16 = a.KS >> 4;
      const int slots = OCT * KS16;
      const rsrc_t wrs = make_rsrc(a.w + (size_t)ob * OCT * a.K, (unsigned)(OCT * a.K));
      const unsigned w0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)s_w;
      for (int s0 = wave * 64; s0 < slots; s0 += NWAVE * 64) {
         const int slot = s0 + lane;
         const int row = fdiv(slot, a.dKS16), chunk = slot - row * KS16;
         if (chunk < K16 && slot < slots) dma16(wrs, w0 + (unsigned)(s0 * 16), row * a.K + chunk * 16, 0);
      }
   };
   // The weights are requested before anything else is set up and the channels' scales and biases are fetched into
   // registers in front of them: both are on their way while the rows of the first tile are worked out and requested,
   // and nothing in the prologue waits for memory before its last line.
   const ColumnParams col_params = load_column_params(a.ep, tid, ob * OCT, OCT);
   stage_weights();
   // Slot of a padded column inside a plane. With the fused pooling the even columns come first, then the odd ones:
   // the pixels of consecutive lanes are two columns apart, and this keeps their 16 bytes next to each other.
   const int half_cols = (a.WP + 1) >> 1;
   auto column_slot = [&](int wp) { return POOL ? (wp >> 1) + (wp & 1) * half_cols : wp; };
   auto slot_column = [&](int pos) { return POOL ? (pos < half_cols ? 2 * pos : 2 * (pos - half_cols) + 1) : pos; };
   const v4i fillv = {(int)a.fill, (int)a.fill, (int)a.fill, (int)a.fill};
   // padding columns of every ring row hold the input zero-point for the life of the kernel
   auto fill_padding_columns = [&]() {
      const int npad = a.WP - a.W;
      for (int rc = tid; rc < a.R * C16; rc += NT) {       // one plane of one ring row per thread
         unsigned char *const plane = s_ring + (rc / C16) * a.RS + (rc % C16) * a.PL;
         for (int pc = 0; pc < npad; ++pc) {
            const int wp = pc < a.pw ? pc : pc + a.W;
            *reinterpret_cast<v4i *>(plane + column_slot(wp) * 16) = fillv;
         }
      }
   };

   // ---- rows of the padded images -> ring. The rows of a request are cut into NRL runs of consecutive rows, one per
   // wavefront (ROWDMA) or per group of C16 wavefronts, which take a plane each.
   const rsrc_t rs = make_rsrc(a.x, a.xbytes);
   const int my_plane = ROWDMA ? 0 : wave % C16, my_rl = ROWDMA ? wave : wave / C16;
   const int slot_c = ROWDMA ? fdiv(lane, a.dPL16) : my_plane;        // plane and padded column of the lane's 16 bytes
   const int slot_pos = ROWDMA ? lane - slot_c * (a.PL >> 4) : lane;  // (a plane may be longer than the row: see the launcher)
   const int slot_wp = slot_column(slot_pos);
   const int iw = slot_wp - a.pw;
   const bool slot_used = slot_pos < a.WP && (!ROWDMA || slot_c < C16);
   const bool col_data = slot_used && iw >= 0 && iw < a.W;
   const int voff = iw * a.C + slot_c * 16;
   // A request is scalar work plus one instruction per row; it is spread over the matrix loop of the present tile
   // (one row per call of req_step, between two K steps), where the scalar unit and the memory pipeline have nothing
   // else to do, instead of standing in front of it. The wavefront's rows inside one image are walked as a run: one
   // division per run, then additions only.
   const unsigned ring_end = ring0 + (unsigned)(a.R * a.RS) + (unsigned)(my_plane * a.PL);
   int rq_v = 0, rq_to = -1, rq_left = 0, rq_soff = 0;
   unsigned rq_dst = 0;
   auto req_begin = [&](int from, int to) {
      const int per = (to - from + NRL) / NRL;          // rows per run, rounded up
      rq_v = from + my_rl * per;
      rq_to = rq_v + per - 1 < to ? rq_v + per - 1 : to;
      rq_left = 0;
   };
   auto req_step = [&]() {
      if (rq_v > rq_to) return;
      if (rq_left == 0) {
         const int n = fdiv(rq_v, a.dHP);
         const int ih = rq_v - n * a.HP - a.ph;
         rq_dst = ring0 + (unsigned)((rq_v - fdiv(rq_v, a.dR) * a.R) * a.RS + my_plane * a.PL);
         if ((unsigned)ih < (unsigned)a.H) {
            const int in_image = a.H - 1 - ih, wanted = rq_to - rq_v;
            rq_left = (in_image < wanted ? in_image : wanted) + 1;
            rq_soff = (n * a.H + ih) * a.row_bytes;
         } else {
            // a padding row between two images (or above the first, below the last)
            if (slot_used) *reinterpret_cast<v4i *>(s_ring + (rq_dst - ring0) + lane * 16) = fillv;
            rq_v += 1;
            return;
         }
      }
      if (col_data) dma16(rs, rq_dst, voff, rq_soff);
      rq_soff += a.row_bytes;
      rq_dst += a.RS;
      if (rq_dst >= ring_end) rq_dst -= a.R * a.RS;
      rq_v += 1;
      --rq_left;
   };
   auto req_finish = [&]() {
      while (rq_v <= rq_to) req_step();
   };
   // first and last virtual row a tile reads
   auto first_row = [&](int t) {
      const int R0 = fdiv(m_begin + t * TM, a.dOW);
      const int n0 = fdiv(R0, a.dOH);
      return n0 * a.HP + (R0 - n0 * a.OH) * RPP;
   };
   auto last_row = [&](int t) {
      const int mlast = (m_begin + (t + 1) * TM < mtot ? m_begin + (t + 1) * TM : mtot) - 1;
      const int R1 = fdiv(mlast, a.dOW);
      const int n1 = fdiv(R1, a.dOH);
      return n1 * a.HP + (R1 - n1 * a.OH) * RPP + (RPP - 1) + 2;
   };

   int b_off[NBT];
#pragma unroll
   for (int i = 0; i < NBT; ++i)
      b_off[i] = M16 ? ((wn * NB * 32 + i * 16 + l16) * a.KS + kg * 16) : (((wn * NB + i) * 32 + l32) * a.KS + half * 16);
   const int nq = half * 4;
   const float *const w_scale = s_scale + wn * NB * 32;
   const int *const w_bias = s_bias + wn * NB * 32;
   const bool plain = a.ep.zp == -128 && a.ep.lo == -128;

   // LDS addresses of the wavefront's pixels in the ring, per kernel row and 32-channel block: the lane's half of the
   // block is plane 2*cb + half; the column tap kw is the constant kw*16 on top. With the fused pooling a lane's four
   // window positions share their rows: four ring rows per lane (window row + kernel row), the window column is
   // another constant.
   const unsigned char *pa[POOL ? 4 : 3][CB][2];   // last index: m tile, or parity of the column with the pooling
   const unsigned char *const lane_base = s_ring + half * a.PL;
   const unsigned char *pa16[M16 ? 3 : 1][M16 ? 4 : 1];   // 16 x 16 tiles: kernel row, pixel tile; the lane's plane is kg
   auto pixel_offsets = [&](int tt) {
      if constexpr (M16) {
#pragma unroll
         for (int j = 0; j < 4; ++j) {
            int m = m_begin + tt * TM + wm * 64 + j * 16 + l16;
            m = m < mtot ? m : mtot - 1;
            const int R = (int)(__umulhi((unsigned)m, a.dOW.magic) >> a.dOW.shift);
            const int ow = m - R * a.OW;
            const int n = (int)(__umulhi((unsigned)R, a.dOH.magic) >> a.dOH.shift);
            const int v = R + n * a.gap;
            const unsigned char *const colb = s_ring + kg * a.PL + ow * 16;
            unsigned slot = (unsigned)v - (__umulhi((unsigned)v, a.dR.magic) >> a.dR.shift) * (unsigned)a.R;
#pragma unroll
            for (int r = 0; r < 3; ++r) {
               pa16[r][j] = colb + slot * a.RS;
               slot = slot + 1;
               slot = slot < slot - (unsigned)a.R ? slot : slot - (unsigned)a.R;
            }
         }
         return;
      }
#pragma unroll
      for (int j = 0; j < MBP; ++j) {
         int m = m_begin + tt * TM + (wm * MBP + j) * 32 + l32;
         m = m < mtot ? m : mtot - 1;
         // OW and OH are at least 2 (the launcher sees to it): the divisions are a multiply-high and a shift
         const int R = (int)(__umulhi((unsigned)m, a.dOW.magic) >> a.dOW.shift);
         const int ow = m - R * a.OW;
         const int n = (int)(__umulhi((unsigned)R, a.dOH.magic) >> a.dOH.shift);
         const int v = R * RPP + n * a.gap;             // n * HP + (R - n * OH) * RPP
         const unsigned char *const colb = lane_base + ow * 16;   // pooled: column 2*ow is slot ow of the even columns
         // ring slots of the rows: v % R, then one step at a time with the wrap
         unsigned slot = (unsigned)v - (__umulhi((unsigned)v, a.dR.magic) >> a.dR.shift) * (unsigned)a.R;
#pragma unroll
         for (int r = 0; r < (POOL ? 4 : 3); ++r) {
            const unsigned char *const rowb = colb + slot * a.RS;
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
               if constexpr (POOL) {
                  pa[r][cb][0] = rowb + cb * 2 * a.PL;
                  pa[r][cb][1] = rowb + cb * 2 * a.PL + half_cols * 16;
               } else {
                  pa[r][cb][j] = rowb + cb * 2 * a.PL;
               }
            }
            slot = slot + 1;
            slot = slot < slot - (unsigned)a.R ? slot : slot - (unsigned)a.R;   // min(slot, slot - R): slot - R wraps below R
         }
      }
   };

   v16i r_bias[REGS && !M16 ? NB : 1];
   v4f r_scale[REGS && !M16 ? NB * 4 : 1];
   v4i r_bias16[M16 ? 4 : 1];       // 16 x 16 tiles: channels i * 16 + kg * 4 .. + 3 of tile i
   v4f r_scale16[M16 ? 4 : 1];
   // K loop of one tile: unrolled over its 9 * CB steps; the fragment reads run two steps ahead of the matrix
   // instructions and one read is issued behind each of a step's first matrix instructions
   auto kloop = [&](AccT (&acc)[NBT][MBT]) {
      if constexpr (M16) {
         // one step per tap: four weight and four pixel fragments, 16 matrix instructions; a read of the next tap's
         // fragments behind every second of them
         v4i fa[2][4], fb[2][4];
         const unsigned char *pb[4];
#pragma unroll
         for (int i = 0; i < 4; ++i) pb[i] = s_w + b_off[i];
#pragma unroll
         for (int s = 0; s < 9 + 1; ++s) {
            if (s < 9) {
               const int kh = s / 3, kw = s % 3;
#pragma unroll
               for (int i = 0; i < 4; ++i) {
                  fb[s & 1][i] = *reinterpret_cast<const v4i *>(pb[i] + s * 64);
                  fa[s & 1][i] = *reinterpret_cast<const v4i *>(pa16[kh][i] + kw * 16);
               }
            }
            if (s >= 1) {
               const int d = s - 1, buf = d & 1;
#pragma unroll
               for (int i = 0; i < 4; ++i)
#pragma unroll
                  for (int j = 0; j < 4; ++j)
                     acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[buf][i], fa[buf][j], d == 0 ? r_bias16[i] : acc[i][j], 0, 0, 0);
            }
            if (s < 9 && s >= 1) {
#pragma unroll
               for (int gidx = 0; gidx < 8; ++gidx) {
                  __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);   // two matrix instructions
                  __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
               }
            }
            __builtin_amdgcn_sched_barrier(0);
            // four chances per tile to send a row request (measured against one behind every tap: 53.8 against
            // 55.4 us on the 56x56 layer; the scalar bookkeeping of a request stands between two taps' instructions)
            if (s < 9 && (s & 1)) req_step();
         }
         req_finish();
         return;
      } else {
      constexpr int NBUF = POOL ? 2 : 3;
      v4i fa[NBUF][MB], fb[NBUF][NB];
      const unsigned char *pb[NB];
#pragma unroll
      for (int i = 0; i < NB; ++i) pb[i] = s_w + b_off[i];
      v16i bias_tile[NB];
      if constexpr (POOL) {
         // the pooled accumulators start from zero: the bias is added to the pooled quarter (max(a + b) = max(a) + b)
#pragma unroll
         for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) bias_tile[i][e] = 0;
      } else if constexpr (REGS) {
#pragma unroll
         for (int i = 0; i < NB; ++i) bias_tile[i] = r_bias[i];
      } else {
#pragma unroll
         for (int gi = 0; gi < NB * 4; ++gi) {
            const v4i bi = *reinterpret_cast<const v4i *>(w_bias + (gi >> 2) * 32 + (gi & 3) * 8 + nq);
#pragma unroll
            for (int e = 0; e < 4; ++e) bias_tile[gi >> 2][(gi & 3) * 4 + e] = bi[e];
         }
      }
#pragma unroll
      for (int s = 0; s < NS + NBUF - 1; ++s) {
         if (s < NS) {
            const int kh = s / (3 * CB), kw = (s / CB) % 3, cb = s % CB;
            fb[s % NBUF][0] = *reinterpret_cast<const v4i *>(pb[0] + s * 32);
#pragma unroll
            for (int j = 0; j < MB; ++j) {
               if constexpr (POOL) fa[s % NBUF][j] = *reinterpret_cast<const v4i *>(pa[(j >> 1) + kh][cb][((j & 1) + kw) & 1] + (((j & 1) + kw) >> 1) * 16);
               else fa[s % NBUF][j] = *reinterpret_cast<const v4i *>(pa[kh][cb][j] + kw * 16);
            }
#pragma unroll
            for (int i = 1; i < NB; ++i) fb[s % NBUF][i] = *reinterpret_cast<const v4i *>(pb[i] + s * 32);
         }
         if (s >= NBUF - 1) {
            const int d = s - (NBUF - 1), buf = d % NBUF;
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
               for (int j = 0; j < MB; ++j) {
                  if (d == 0) acc[i][j] = MmaI8::mma(fb[buf][i], fa[buf][j], bias_tile[i]);
                  else acc[i][j] = MmaI8::mma(fb[buf][i], fa[buf][j], acc[i][j]);
               }
         }
         if (s < NS && s >= NBUF - 1) {
#pragma unroll
            for (int gidx = 0; gidx < MB + NB; ++gidx) {
               __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one matrix instruction
               __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
            }
            if constexpr (MB * NB > MB + NB) __builtin_amdgcn_sched_group_barrier(0x008, MB * NB - (MB + NB), 0);
         }
         __builtin_amdgcn_sched_barrier(0);
         if (s < NS && (NS <= 9 || (s & 1))) req_step();   // 9 chances per tile
      }
      req_finish();
      }
   };
   // Requantisation and stores of one tile: a lane packs its four 4-channel groups of an accumulator tile into four
   // dwords, two swaps between the halves of the wavefront turn them into 16 consecutive channels, and two more
   // (store_pixels_64) sort the two tiles' halves into 64 contiguous bytes per pixel, 16 pixels per store instruction.
   // (Stored right after the first two swaps an instruction touched 32 pixels with 32 bytes each; moving the bytes
   // between lanes through a private block of LDS instead of by swaps cost what the wider stores gained.)
   auto epilogue_as = [&](AccT (&acc)[NBT][MBT], int tt, auto plain_tag) {
      constexpr bool PLAIN = decltype(plain_tag)::value;
      const int m_wave = m_begin + tt * TM + wm * MBP * 32, n_wave = ob * OCT + wn * NB * 32;
      const float zpo = (float)(ep.zp + 128), lof = (float)(ep.lo + 128);
      if constexpr (M16) {
         // A lane holds channels kg * 4 .. + 3 of each of the four 16-channel tiles of its pixel: packed, they are a
         // 4 x 4 matrix of dwords over the pixel's four lanes (16 lanes apart), and two rounds of swaps (between the
         // halves of the wavefront, then between neighbouring groups of 16 lanes) transpose it. Lane group kg then
         // has the 16 channels of tile kg in order, and a store instruction writes 64 contiguous bytes for each of 16 pixels.
#pragma unroll
         for (int j = 0; j < 4; ++j) {
            const int m = m_wave + j * 16 + l16;
            int8_t *const row = static_cast<int8_t *>(ep.Y) + (size_t)(m < ep.M ? m : 0) * ep.ldy + n_wave + kg * 16;
            unsigned d[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
               unsigned pk = 0;
#pragma unroll
               for (int e = 0; e < 4; ++e) {
                  float r = __fmul_rn(__int2float_rn(acc[i][j][e]), r_scale16[i][e]);
                  if constexpr (!PLAIN) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);
                  pk = __builtin_amdgcn_cvt_pk_u8_f32(r, e, pk);
               }
               d[i] = pk ^ 0x80808080u;
            }
            const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
            const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
            const auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
            const auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
            const v4i v = {(int)t01[0], (int)t01[1], (int)t23[0], (int)t23[1]};
            if (m < ep.M) store16_wt(row, v);
         }
         return;
      } else {
#pragma unroll
      for (int j = 0; j < MBP; ++j) {
         unsigned v[2][4];
#pragma unroll
         for (int i = 0; i < NB; ++i) {
            unsigned d[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
               const v4f sc = r_scale[REGS ? i * 4 + q : 0];
               unsigned pk = 0;
#pragma unroll
               for (int e = 0; e < 4; ++e) {
                  // the accumulators started from the bias; the byte conversion rounds half to even and saturates
                  float r = __fmul_rn(__int2float_rn(acc[i][j][q * 4 + e]), sc[e]);
                  if constexpr (!PLAIN) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);
                  pk = __builtin_amdgcn_cvt_pk_u8_f32(r, e, pk);
               }
               d[q] = pk ^ 0x80808080u;
            }
            const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
            const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
            v[i][0] = s02[0]; v[i][1] = s02[1]; v[i][2] = s13[0]; v[i][3] = s13[1];
         }
         store_pixels_64(ep, v, lane, m_wave + j * 32, n_wave);
      }
      }
   };
   bool any_negative = false;   // pooled variant: some scale of the workgroup's channels is negative (set below)
   auto epilogue = [&](AccT (&acc)[NBT][MBT], int tt) {
      if constexpr (POOL) {
         const int m_wave = m_begin + tt * TM + wm * 32, n_wave = ob * OCT + wn * NB * 32;
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
                  for (int e4 = 0; e4 < 4; ++e4) {
                     const int e = q * 4 + e4;
                     const int hi = max(max(acc[i][0][e], acc[i][1][e]), max(acc[i][2][e], acc[i][3][e]));
                     const int lo = min(min(acc[i][0][e], acc[i][1][e]), min(acc[i][2][e], acc[i][3][e]));
                     pooled[i][0][e] = sc[e4] < 0.0f ? lo : hi;
                  }
               }
         }
         // (two column tiles: they leave as 64 contiguous bytes per pooled pixel, written through the L2)
         if (plain) tile_epilogue_s8_direct<NB, 1, true, true>(ep, pooled, w_scale, w_bias, lane, m_wave, n_wave);
         else tile_epilogue_s8_direct<NB, 1, false, true>(ep, pooled, w_scale, w_bias, lane, m_wave, n_wave);
      } else {
         if (plain) epilogue_as(acc, tt, BoolTag<true>{});
         else epilogue_as(acc, tt, BoolTag<false>{});
      }
   };
   // whether the wavefront has pixels in tile tt (all tiles but the last are full)
   auto has_work = [&](int tt) { return m_begin + tt * TM + wm * MBP * 32 < mtot; };

   // The two wavefronts that share a SIMD (w and w + 4) do their parts of a tile in different order, so that the
   // matrix pipe always has a wavefront feeding it: wavefronts 0-3 multiply tile t first, then requantise it and
   // compute the addresses of tile t + 1; the others first requantise their tile t - 1 and compute the addresses of
   // tile t, and multiply last, up to the barrier that ends the tile.
   const bool mma_first = wave < 4;
   int t = t0, t_prev = -1, hi_cur = 0;
   if (t < t1) {
      hi_cur = last_row(t);
      req_begin(first_row(t), hi_cur);
      req_finish();
      if (mma_first) pixel_offsets(t);
   }
   fill_padding_columns();
   if (tid < OCT) {
      s_scale[tid] = col_params.scale;
      s_bias[tid] = col_params.bias;
   }
   wait_vmcnt<0>();
   __syncthreads();                          // weights, column parameters, padding columns and the first rows are in LDS
   if constexpr (POOL) {
      // whether any scale of the workgroup's channels is negative (uniform, so the common case pools with a maximum only)
      int neg = 0;
      for (int c = tid; c < OCT; c += NT) neg |= s_scale[c] < 0.0f;
      any_negative = __syncthreads_or(neg) != 0;
   }
   if constexpr (M16) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         r_scale16[i] = *reinterpret_cast<const v4f *>(w_scale + i * 16 + kg * 4);
         r_bias16[i] = *reinterpret_cast<const v4i *>(w_bias + i * 16 + kg * 4);
      }
   } else if constexpr (REGS) {
#pragma unroll
      for (int gi = 0; gi < NB * 4; ++gi) {
         r_scale[gi] = *reinterpret_cast<const v4f *>(w_scale + (gi >> 2) * 32 + (gi & 3) * 8 + nq);
         const v4i bi = *reinterpret_cast<const v4i *>(w_bias + (gi >> 2) * 32 + (gi & 3) * 8 + nq);
#pragma unroll
         for (int e = 0; e < 4; ++e) r_bias[gi >> 2][(gi & 3) * 4 + e] = bi[e];
      }
   }
   AccT acc[NBT][MBT];
   // rows tile t + 1 has and tile t does not: requested during tile t into slots that tile t does not read
   auto request_next = [&](bool more, int tn, int &hi_next) {
      if (more) {
         hi_next = last_row(tn);
         req_begin(hi_cur + 1, hi_next);
      }
   };
   // One loop per role, so that the accumulators of each have one home in the register file. All run t1 - t0
   // iterations with one workgroup barrier each: it says that the rows of the next tile are complete (every
   // wavefront has waited for its own requests) and that every wavefront is done reading the present tile.
   if (mma_first) {
      while (t < t1) {
         const int tn = t + 1;
         const bool more = tn < t1;
         int hi_next = hi_cur;
         request_next(more, tn, hi_next);
         if (has_work(t)) {
            kloop(acc);
            wait_vmcnt<0>();                 // before this tile's stores join the queue
            epilogue(acc, t);
         } else {
            req_finish();
            wait_vmcnt<0>();
         }
         if (more) pixel_offsets(tn);
         t = tn;
         hi_cur = hi_next;
         __syncthreads();
      }
   } else {
      while (t < t1) {
         const int tn = t + 1;
         const bool more = tn < t1;
         int hi_next = hi_cur;
         request_next(more, tn, hi_next);
         if (t_prev >= 0) epilogue(acc, t_prev);
         const bool work = has_work(t);
         if (work) {
            pixel_offsets(t);
            kloop(acc);
         } else {
            req_finish();
         }
         wait_vmcnt<0>();
         t_prev = work ? t : -1;
         t = tn;
         hi_cur = hi_next;
         __syncthreads();
      }
      if (t_prev >= 0) epilogue(acc, t_prev);
   }
}

template <int C16, int WN, bool ROWDMA, bool POOL>
__global__ void __launch_bounds__(512) k_qconv_ring(QConvRingArgs a)
{
   extern __shared__ __align__(16) unsigned char smem[];
   qconv_ring_body<C16, WN, ROWDMA, POOL>(a, smem);
}

// Two convolutions in one launch: layer a (64 output channels, one block of them) and layer b, which reads layer a's
// output, for launches in which every workgroup of both layers owns the same whole images. A workgroup then reads in
// layer b only what it wrote itself in layer a: its stores have reached the L2 once the vector-memory counter is down
// (a compute unit's L1 is written through and holds no line of a tensor nobody has read since the kernel began), so a
// wait and a workgroup barrier order the two layers and no kernel boundary stands between them: no wait for the
// slowest workgroup of layer a, no write-back of the L2s, no launch latency, and layer a's result is still in the
// workgroup's own L2 when layer b fetches it.
template <int C16A, bool POOLA, int WNB>
__global__ void __launch_bounds__(512) k_qconv_ring_pair(QConvRingArgs a, QConvRingArgs b)
{
   extern __shared__ __align__(16) unsigned char smem[];
   qconv_ring_body<C16A, 1, true, POOLA>(a, smem);
   wait_vmcnt<0>();
   __syncthreads();        // every wavefront is done with layer a's LDS, every store of the workgroup is in the L2
   qconv_ring_body<4, WNB, true, false>(b, smem);
}

}  // namespace

namespace sofie {

// 3x3, stride 1, 32 or 64 input channels, channels-last int8 in and out, rows of at most 64 padded columns; with or
// without a fused 2x2 stride-2 max pooling.
// What a launch of k_qconv_ring needs beside the argument block.
struct RingPlan {
   QConvRingArgs a;
   size_t lds;
   unsigned grid;
   int C16, WN, nob;
   bool row, pool;
   long long px_per_group;   // (pooled) pixels of a workgroup's run if every run has the same length, else 0
   int image_px;             // (pooled) pixels of one image
};

// Fills `plan` if the kernel takes the problem (*done).
static int plan_ring(sofie_hip_ctx *ctx, const QConvArgs &g, RingPlan &out, bool *done)
{
   *done = false;
   if (g.xf) return SOFIE_HIP_OK;
   const bool pool = g.pool_kh != 0;
   if (pool && !(g.pool_kh == 2 && g.pool_kw == 2 && g.pool_sh == 2 && g.pool_sw == 2)) return SOFIE_HIP_OK;
   if (g.groups != 1 || !(g.C == 32 || g.C == 64) || g.OC % 64 != 0 || !g.x_nhwc || !g.y_nhwc || !g.w_ohwi) return SOFIE_HIP_OK;
   if (g.KH != 3 || g.KW != 3 || g.sh != 1 || g.sw != 1) return SOFIE_HIP_OK;
   if (!aligned16(g.x) || !aligned16(g.w) || !aligned16(g.y)) return SOFIE_HIP_OK;
   // rows and columns the tiles count: pooled pixels when the pooling is fused
   const int TH = pool ? g.PH : g.OH, TW = pool ? g.PW : g.OW;
   const int rpp = pool ? 2 : 1;
   const long long mtot = (long long)g.N * TH * TW;
   const int HP = g.H + g.ph + g.pbh, WP = g.W + g.pw + g.pbw;
   // One instruction fetches a whole padded row if its C/16 planes are at most 64 16-byte slots, else one plane of a
   // row, with one lane per padded column: rows wider than 64 columns do not fit.
   if (mtot <= 0 || WP > 64 || TW < 2 || TH < 2) return SOFIE_HIP_OK;
   if (mtot >= (1ll << 31) - 1024 || (long long)g.N * HP >= (1ll << 31) - 4096) return SOFIE_HIP_OK;
   const size_t xbytes = (size_t)g.N * g.H * g.W * g.C;
   if (xbytes >= ((size_t)1 << 31)) return SOFIE_HIP_OK;
   const int WN = g.OC % 128 == 0 ? 2 : 1;
   const int OCT = WN * 64;
   const int C16 = g.C / 16;
   QConvRingArgs a{};
   a.x = g.x; a.w = g.w;
   a.ep.Y = g.y; a.ep.scale = g.scale; a.ep.bias = g.bias;
   a.ep.M = (int)mtot; a.ep.N = g.OC; a.ep.ldy = g.OC;
   a.ep.zp = g.zpy; a.ep.lo = g.lo; a.ep.relu = g.relu; a.ep.s = 1.0f;
   a.ep.vec_store = 1;
   a.H = g.H; a.W = g.W; a.C = g.C; a.ph = g.ph; a.pw = g.pw;
   a.OH = TH; a.OW = TW; a.HP = HP; a.WP = WP;
   a.gap = HP - TH * rpp;
   a.K = 9 * g.C;
   // The 64-channel layers without pooling run on 16 x 16 matrix instructions: a lane reads row (lane % 16) of a
   // tile and chunk (lane / 16) of K. The LDS serves a 16-byte read of a wavefront in four rounds of 16 lanes
   // (lanes 0-7 with 24-31, 8-15 with 16-23, and the same in the upper half), each free of conflicts if its lanes'
   // 16-byte slots differ modulo 256 bytes (measured: 4.4 cycles per read against 8.1). For the pixels that asks for
   // planes a multiple of 256 bytes apart, for the weights for a row pitch of 2, 6, 10 or 14 slots modulo 16.
   const bool m16 = C16 == 4 && !pool;
   a.KS = m16 ? a.K + 32 : (((a.K / 16) % 2 == 0) ? a.K + 16 : a.K);
   a.row_bytes = g.W * g.C;
   a.fill = 0x01010101u * (unsigned)(g.zpx & 0xff);
   a.xbytes = (unsigned)xbytes;
   a.dOW = make_fastdiv(TW); a.dOH = make_fastdiv(TH); a.dHP = make_fastdiv(HP); a.dKS16 = make_fastdiv(a.KS / 16);
   // The ring holds the rows of two consecutive tiles of TM pixels: the rows 2*TM consecutive pixels can touch, the
   // padded rows between the images they can span and the two extra rows of the last window.
   const int unit = pool ? 32 : 64;
   const int TM = (8 / WN) * unit;
   const int rows2 = (2 * TM - 1) / TW + 2;
   int crossings = (rows2 - 1) / TH + 1;
   if (crossings > g.N - 1) crossings = g.N - 1;
   const int R = rows2 * rpp + a.gap * crossings + 2;
   // Plane pitch PL -> row pitch and LDS bytes. Row pitch: consecutive pixels of an output row are 16 bytes apart (with
   // the pooling too: even and odd columns are stored apart); padded so that the first pixel of the next output row
   // continues that sequence modulo the 256 bytes the LDS banks span.
   auto plan = [&](int PL) {
      a.PL = PL;
      a.RS = C16 * PL;
      // rpp ring rows lie between two output rows: rpp * RS = TW * 16 modulo 256, as nearly as a multiple of 16 allows
      int best = 0, best_miss = 1 << 30;
      for (int pad = 0; pad < 256; pad += 16) {
         const int miss = ((rpp * (a.RS + pad) - TW * 16) % 256 + 256) % 256;
         const int dist = miss < 256 - miss ? miss : 256 - miss;
         if (dist < best_miss) { best_miss = dist; best = pad; }
      }
      a.RS += best;
      return (size_t)OCT * a.KS + (size_t)OCT * 8 + (size_t)R * a.RS;
   };
   size_t lds = plan(m16 ? (WP * 16 + 255) / 256 * 256 : WP * 16);
   if (lds > 160 * 1024 && a.PL != WP * 16) lds = plan(WP * 16);   // the longer planes do not fit: the rows as they are
   if (lds > 160 * 1024) return SOFIE_HIP_OK;
   a.R = R;
   a.dR = make_fastdiv(R);
   a.dPL16 = make_fastdiv(a.PL / 16);
   if ((size_t)g.OC * a.K >= ((size_t)1 << 31)) return SOFIE_HIP_OK;
   const int nob = g.OC / OCT;
   int per = ctx->num_cus / nob;
   if (per < 1) per = 1;
   const int units = (int)((mtot + unit - 1) / unit);
   if (per > units) per = units;
   a.units_each = units / per;
   a.units_rem = units % per;
   out.a = a;
   out.lds = lds;
   out.grid = (unsigned)(per * nob);
   out.C16 = C16; out.WN = WN; out.nob = nob;
   out.row = C16 * (a.PL / 16) <= 64;
   out.pool = pool;
   out.px_per_group = a.units_rem == 0 ? (long long)a.units_each * unit : 0;
   out.image_px = TH * TW;
   *done = true;
   return SOFIE_HIP_OK;
}

int qconv_ring(sofie_hip_ctx *ctx, const QConvArgs &g, bool *done)
{
   RingPlan plan;
   if (int rc = plan_ring(ctx, g, plan, done)) return rc;
   if (!*done) return SOFIE_HIP_OK;
   const QConvRingArgs &a = plan.a;
   const size_t lds = plan.lds;
   const int C16 = plan.C16, WN = plan.WN;
   const bool pool = plan.pool;
   const dim3 grid(plan.grid), block(512);
#define SOFIE_QRING_LAUNCH(C16_, WN_, ROW_, POOL_)                                                             \
   do {                                                                                                        \
      constexpr auto kern = k_qconv_ring<C16_, WN_, ROW_, POOL_>;                                              \
      SOFIE_LARGE_LDS(kern);                                                                                   \
      hipLaunchKernelGGL(kern, grid, block, lds, ctx->stream, a);                                              \
   } while (0)
#define SOFIE_QRING_BY_ROW(C16_, WN_, POOL_)                                                                   \
   do {                                                                                                        \
      if (plan.row) SOFIE_QRING_LAUNCH(C16_, WN_, true, POOL_);                                                \
      else SOFIE_QRING_LAUNCH(C16_, WN_, false, POOL_);                                                        \
   } while (0)
#define SOFIE_QRING_BY_POOL(C16_, WN_)                                                                         \
   do {                                                                                                        \
      if (pool) SOFIE_QRING_BY_ROW(C16_, WN_, true);                                                           \
      else SOFIE_QRING_BY_ROW(C16_, WN_, false);                                                               \
   } while (0)
   if (C16 == 4) {
      if (WN == 2) SOFIE_QRING_BY_POOL(4, 2);
      else SOFIE_QRING_BY_POOL(4, 1);
   } else {
      if (WN == 2) SOFIE_QRING_BY_POOL(2, 2);
      else SOFIE_QRING_BY_POOL(2, 1);
   }
#undef SOFIE_QRING_BY_POOL
#undef SOFIE_QRING_BY_ROW
#undef SOFIE_QRING_LAUNCH
   return check_launch(ctx, pool ? "k_qconv_ring_pool" : "k_qconv_ring");
}

// Layer g1 (its fused pooling included) and layer g2, which reads g1's output, as one launch of k_qconv_ring_pair:
// both must be problems of k_qconv_ring with one block of output channels and a whole padded row per request, g1 with
// the fused pooling, and every workgroup must own the same whole images in both layers. *done tells whether the launch
// was made; if not, nothing was launched and the caller runs the layers one after the other.
int qconv_ring_pair(sofie_hip_ctx *ctx, const QConvArgs &g1, const QConvArgs &g2, bool *done)
{
   *done = false;
   if (g2.x != static_cast<const int8_t *>(g1.y) || g1.N != g2.N || g2.pool_kh != 0) return SOFIE_HIP_OK;
   RingPlan p1, p2;
   bool ok1 = false, ok2 = false;
   if (int rc = plan_ring(ctx, g1, p1, &ok1)) return rc;
   if (!ok1) return SOFIE_HIP_OK;
   if (int rc = plan_ring(ctx, g2, p2, &ok2)) return rc;
   if (!ok2) return SOFIE_HIP_OK;
   if (!p1.pool || p1.WN != 1 || p1.nob != 1 || !p1.row || p2.C16 != 4 || p2.nob != 1 || !p2.row || p1.grid != p2.grid) return SOFIE_HIP_OK;
   // the same whole images per workgroup in both layers
   if (p1.px_per_group == 0 || p2.px_per_group == 0 || p1.px_per_group % p1.image_px != 0 || p2.px_per_group % p2.image_px != 0 ||
       p1.px_per_group / p1.image_px != p2.px_per_group / p2.image_px)
      return SOFIE_HIP_OK;
   const size_t lds = p1.lds > p2.lds ? p1.lds : p2.lds;
   const dim3 grid(p1.grid), block(512);
#define SOFIE_QRING_PAIR(C16A_, WNB_)                                                                          \
   do {                                                                                                        \
      constexpr auto kern = k_qconv_ring_pair<C16A_, true, WNB_>;                                              \
      SOFIE_LARGE_LDS(kern);                                                                                   \
      hipLaunchKernelGGL(kern, grid, block, lds, ctx->stream, p1.a, p2.a);                                     \
   } while (0)
   if (p1.C16 == 2) {
      if (p2.WN == 2) SOFIE_QRING_PAIR(2, 2);
      else SOFIE_QRING_PAIR(2, 1);
   } else {
      if (p2.WN == 2) SOFIE_QRING_PAIR(4, 2);
      else SOFIE_QRING_PAIR(4, 1);
   }
#undef SOFIE_QRING_PAIR
   *done = true;
   return check_launch(ctx, "k_qconv_ring_pair");
}

}  // namespace sofie
