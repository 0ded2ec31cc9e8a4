// One-byte-element GEMMs on the gfx950 matrix cores: int8 x int8 -> int32 with fused
// requantisation (QLinearMatMul semantics) and FP8 e4m3 x e4m3 -> fp32 -> bf16/fp32.
//
// Kernel shape (k_gemm_bytes): 256 threads = 4 wavefronts in a 2x2 arrangement, each
// wavefront owning a (TI*32) x (TJ*32) block of the output built from 32x32 MFMA tiles
// (v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x64_f8f6f4). Both operands are staged in LDS
// as [row][K-bytes] with a 16-byte pad per row, which makes the 16-byte-per-lane operand
// reads bank-conflict free; global -> register -> LDS staging is double buffered so the
// loads of K-step t+1 are in flight while the MFMAs of step t issue. The MFMA row operand
// is the B^T tile (output column n), the column operand the A tile (output row m), so a lane
// holds four consecutive n for one m and the epilogue packs them into one 4*esize store; the
// packed results go through a per-wavefront LDS staging block and leave as 16-byte row
// segments. Workgroup ids are remapped so that each XCD (ids are dealt round-robin over the
// 8 XCDs) owns a compact rectangle of output tiles and its L2 sees each operand panel once.
#include "common.h"
#include "gemm_tile.h"

using namespace sofie;

namespace {


// Workgroup id -> output tile. Ids are dealt round-robin over the 8 XCDs, each with its own
// L2; the remap gives every XCD a contiguous run of ids and the grouped order turns that run
// into a compact rectangle of tiles, so an XCD's L2 sees each operand panel once.
template <int GM = 4>
__device__ __forceinline__ void tile_of_workgroup(int pid, int tiles_m, int tiles_n, int &tm, int &tn)
{
   const int tiles = tiles_m * tiles_n;
   {
      const int xcd = pid & 7, local = pid >> 3;
      const int base = tiles >> 3, rem = tiles & 7;
      pid = local + xcd * base + (xcd < rem ? xcd : rem);
   }
   const int width = GM * tiles_n;
   const int group = pid / width;
   const int first = group * GM;
   const int gsize = (tiles_m - first) < GM ? (tiles_m - first) : GM;
   tm = first + (pid % width) % gsize;
   tn = (pid % width) / gsize;
}

template <class Mma, int BK, int NSETS, int TI, int TJ, int OUT, bool B_KN, bool FULL>
__global__ void __launch_bounds__(256, (TI * TJ >= 16 || NSETS > 2) ? 1 : 2) k_gemm_bytes(GemmArgs g)
{
   constexpr int BN = 2 * TI * 32, BM = 2 * TJ * 32;
   constexpr int LDK = BK + 16;
   constexpr int CPR = BK / 16;
   constexpr int NSUB = BK / Mma::KB;
   constexpr int ESZ = OutSize<OUT>::value;
   constexpr bool IS_INT = __is_same(typename Mma::Acc, v16i);
   extern __shared__ __align__(16) unsigned char smem[];
   unsigned char *const sA = smem;                  // [2][BM][LDK]
   unsigned char *const sB = smem + 2 * BM * LDK;   // [2][BN][LDK]

   const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
   const int wm = wave >> 1, wn = wave & 1;

   int tm, tn;
   int pid = blockIdx.x;
   bool placed = false;
   if constexpr (IS_INT && OUT == SOFIE_OUT_S32) {
      if (g.splits > 1) {
         const int tiles = g.tiles_m * g.tiles_n;
         int ks;
         const int xps = 8 / g.splits;                 // XCDs per K slice
         if (8 % g.splits == 0 && tiles % xps == 0) {
            // Workgroup ids are dealt round-robin over the 8 XCDs. A K slice goes to 8 / splits XCDs of its own: the
            // slice of B is then read by those XCDs only (with rows of tiles spread over all XCDs every XCD reads all
            // of B), and the column tiles of a row panel of A sit next to each other on one XCD.
            const int xcd = pid & 7, idx = pid >> 3;
            ks = xcd / xps;
            const int tile = (xcd % xps) * (tiles / xps) + idx;
            tm = tile / g.tiles_n;
            tn = tile - tm * g.tiles_n;
            placed = true;
         } else {
            ks = pid / tiles;
            pid -= ks * tiles;
         }
         const int k_begin = ks * g.kslice;
         g.A += k_begin;
         g.B += B_KN ? (size_t)k_begin * g.ldb : (size_t)k_begin;
         g.K = (g.K - k_begin) < g.kslice ? (g.K - k_begin) : g.kslice;
         g.Y = static_cast<unsigned char *>(g.Y) + (size_t)ks * g.ysplit;
      }
   }
   if (!placed) tile_of_workgroup(pid, g.tiles_m, g.tiles_n, tm, tn);
   const int m0 = tm * BM, n0 = tn * BN;

   // --- global -> register staging -----------------------------------------------------
   // A thread owns A_CH 16-byte chunks of the A tile and B_CH of the B tile per K-step.
   // NSETS register sets are in flight: the chunk written to LDS during step t (tile t+1) is
   // re-requested for tile t+1+NSETS right behind its LDS write, so every request has NSETS
   // full K-steps to return.
   constexpr int A_CH = BM * CPR / 256;
   constexpr int B_UNITS = BN / 4 * CPR;                 // transposing loader: 16k x 4n units per tile
   constexpr int B_UPT = (B_UNITS + 255) / 256;          // units per thread
   constexpr int B_CH = B_KN ? B_UPT * 4 : BN * CPR / 256;
   constexpr int B_PARTS = B_KN ? B_UPT : B_CH;          // independently movable pieces of B
   struct Staged {
      v4i a[A_CH];
      v4i b[B_CH];
   };
   const v4i zero4 = {0, 0, 0, 0};

   // Row/column part of each thread's addresses is fixed for the whole K loop. Out-of-range
   // rows are clamped to a valid row and their data replaced by zero after the load, so the
   // loads themselves are never predicated.
   const unsigned char *pa[A_CH];
   bool oka[A_CH];
#pragma unroll
   for (int i = 0; i < A_CH; ++i) {
      const int c = i * 256 + tid;
      const int gm = m0 + c / CPR;
      oka[i] = FULL || gm < g.M;
      pa[i] = g.A + (size_t)(oka[i] ? gm : g.M - 1) * g.lda + (c % CPR) * 16;
   }
   const unsigned char *pb[B_PARTS];
   bool okb[B_PARTS];
#pragma unroll
   for (int i = 0; i < B_PARTS; ++i) {
      if constexpr (!B_KN) {
         const int c = i * 256 + tid;
         const int gn = n0 + c / CPR;
         okb[i] = FULL || gn < g.N;
         pb[i] = g.B + (size_t)(okb[i] ? gn : g.N - 1) * g.ldb + (c % CPR) * 16;
      } else {
         const int u = i * 256 + tid;
         const int kg = u % CPR, ng = u / CPR;
         const int gn = n0 + ng * 4;
         okb[i] = (B_UNITS % 256 == 0 || u < B_UNITS) && (FULL || gn < g.N);
         pb[i] = g.B + (size_t)(kg * 16) * g.ldb + (okb[i] ? gn : 0);
      }
   }
   const int kmax = g.K - 16;   // K is a multiple of 16 on this path

   auto fetch_a = [&](Staged &G, int k0, int i) {
      const int kc = ((i * 256 + tid) % CPR) * 16;
      const bool kin = FULL || k0 + kc <= kmax;
      const v4i v = *reinterpret_cast<const v4i *>(pa[i] + (kin ? k0 : kmax - kc));
      G.a[i] = (oka[i] && kin) ? v : zero4;
   };
   auto fetch_b = [&](Staged &G, int k0, int i) {
      const int kc = ((i * 256 + tid) % CPR) * 16;
      const bool kin = FULL || k0 + kc <= kmax;
      if constexpr (!B_KN) {
         const v4i v = *reinterpret_cast<const v4i *>(pb[i] + (kin ? k0 : kmax - kc));
         G.b[i] = (okb[i] && kin) ? v : zero4;
      } else {
         // B is [K,N]: a unit is 16 k-rows x 4 n-columns = 16 dwords, kept raw in registers and
         // transposed into four K-contiguous 16-byte chunks when written to LDS.
         const unsigned char *p = pb[i] + (size_t)(kin ? k0 : kmax - kc) * g.ldb;
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            v4i v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = *reinterpret_cast<const int *>(p + (size_t)(4 * q + e) * g.ldb);
            G.b[i * 4 + q] = (okb[i] && kin) ? v : zero4;
         }
      }
   };
   auto stash_a = [&](const Staged &G, int stage, int i) {
      const int c = i * 256 + tid;
      *reinterpret_cast<v4i *>(sA + stage * BM * LDK + (c / CPR) * LDK + (c % CPR) * 16) = G.a[i];
   };
   auto stash_b = [&](const Staged &G, int stage, int i) {
      unsigned char *b = sB + stage * BN * LDK;
      if constexpr (!B_KN) {
         const int c = i * 256 + tid;
         *reinterpret_cast<v4i *>(b + (c / CPR) * LDK + (c % CPR) * 16) = G.b[i];
      } else {
         const int u = i * 256 + tid;
         const bool live = B_UNITS % 256 == 0 || u < B_UNITS;
         const int kg = u % CPR, ng = u / CPR;
         unsigned o[4][4];   // o[column][k-quad]: 4x4 byte transposes with v_perm_b32
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            const v4i d = G.b[i * 4 + q];
            const unsigned t0 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u);
            const unsigned t1 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
            const unsigned t2 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
            const unsigned t3 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
            o[0][q] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
            o[1][q] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
            o[2][q] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
            o[3][q] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
         }
         if (live) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
               const v4i v = {(int)o[j][0], (int)o[j][1], (int)o[j][2], (int)o[j][3]};
               *reinterpret_cast<v4i *>(b + (ng * 4 + j) * LDK + kg * 16) = v;
            }
         }
      }
   };
   // Pieces of a tile pair are numbered 0..A_CH+B_PARTS-1 and dealt round-robin to the MFMA
   // groups of a K-step; group `grp` of `ngrp` moves the pieces p with p % ngrp == grp.
   auto move_pieces = [&](Staged &G, int stage, int k_next, int grp, int ngrp, bool do_stash, bool do_fetch) {
#pragma unroll
      for (int p = 0; p < A_CH + B_PARTS; ++p) {
         if (p % ngrp != grp) continue;
         if (p < A_CH) {
            if (do_stash) stash_a(G, stage, p);
            if (do_fetch) fetch_a(G, k_next, p);
         } else {
            if (do_stash) stash_b(G, stage, p - A_CH);
            if (do_fetch) fetch_b(G, k_next, p - A_CH);
         }
      }
   };

   typename Mma::Acc acc[TI][TJ];
#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
         for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

   const int frag_row = lane & 31;
   const int frag_k = (lane >> 5) * Mma::LANE_BYTES;
   const int a_off = (wm * TJ * 32 + frag_row) * LDK + frag_k;
   const int b_off = (wn * TI * 32 + frag_row) * LDK + frag_k;
   constexpr int TMAX = TI > TJ ? TI : TJ;
   static_assert(NSUB >= 2 && NSUB % 2 == 0, "the software pipeline needs an even number of MFMA K-substeps per stage");

   // Operand fragments: two register sets used alternately by consecutive MFMA K-substeps.
   typename Mma::Frag fn[2][TI], fm[2][TJ];
   auto read_pair = [&](int set, int stage, int sub, int i) {
      if (i < TI) fn[set][i] = Mma::load(sB + stage * BN * LDK + b_off + i * 32 * LDK + sub * Mma::KB);
      if (i < TJ) fm[set][i] = Mma::load(sA + stage * BM * LDK + a_off + i * 32 * LDK + sub * Mma::KB);
   };
   auto mma_row = [&](int set, int i) {
      if (i < TI) {
#pragma unroll
         for (int j = 0; j < TJ; ++j) acc[i][j] = Mma::mma(fn[set][i], fm[set][j], acc[i][j]);
      }
   };

   // One K-step on LDS stage `stage`. On entry fragment set 0 holds substep 0 of this stage.
   //   substeps 0..NSUB-2: multiply while the next substep's fragments are read, and while
   //                       register set G (tile of the next step) moves into the other stage
   //                       and is re-requested for tile `k_next`;
   //   barrier:            the other stage is complete and nobody reads this stage any more;
   //   substep NSUB-1:     multiply while set 0 is refilled from the other stage.
   // The instruction order is pinned with scheduling barriers so that every group of TJ MFMAs
   // has memory instructions issued right behind it to overlap with.
   auto kstep = [&](int stage, Staged &G, int k_next, bool more) {
      constexpr int NGRP = (NSUB - 1) * TMAX;
#pragma unroll
      for (int sub = 0; sub < NSUB - 1; ++sub) {
#pragma unroll
         for (int i = 0; i < TMAX; ++i) {
            read_pair((sub + 1) & 1, stage, sub + 1, i);
            mma_row(sub & 1, i);
            move_pieces(G, stage ^ 1, k_next, sub * TMAX + i, NGRP, more, true);
            __builtin_amdgcn_sched_barrier(0);
         }
      }
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TMAX; ++i) {
         if (more) read_pair(0, stage ^ 1, 0, i);
         mma_row((NSUB - 1) & 1, i);
         __builtin_amdgcn_sched_barrier(0);
      }
   };

   const int nk = (g.K + BK - 1) / BK;
   const int klast = nk > 0 ? (nk - 1) * BK : 0;
   auto kclamp = [&](int t) { return t * BK < klast ? t * BK : klast; };
   // Requests past the end of K re-read the last tile (never used): keeping every request
   // unconditional keeps the number of loads in flight identical on every path.
   Staged G[NSETS];
   if (nk > 0) {
      move_pieces(G[0], 0, 0, 0, 1, false, true);               // tile 0
#pragma unroll
      for (int s = 1; s < NSETS; ++s) move_pieces(G[s], 0, kclamp(s), 0, 1, false, true);   // tiles 1 .. NSETS-1
      // (the later tiles are requested before tile 0 is waited for: their way from memory runs under its)
      move_pieces(G[0], 0, 0, 0, 1, true, false);               // tile 0 -> stage 0
      move_pieces(G[0], 0, kclamp(NSETS), 0, 1, false, true);   // tile NSETS
      __syncthreads();
#pragma unroll
      for (int i = 0; i < TMAX; ++i) read_pair(0, 0, 0, i);
      __builtin_amdgcn_sched_barrier(0);
   }
   // step t multiplies stage t&1, moves tile t+1 (register set (t+1) % NSETS) into stage (t+1)&1
   // and re-requests that set for tile t+1+NSETS; the loop is unrolled over the stages and the sets
   constexpr int UNR = NSETS > 2 ? NSETS : 2;
   static_assert(UNR % 2 == 0 && UNR % NSETS == 0, "the unrolled loop covers whole cycles of stages and register sets");
   int kt = 0;
   for (; kt + UNR <= nk; kt += UNR) {
#pragma unroll
      for (int u = 0; u < UNR; ++u) kstep(u & 1, G[(u + 1) % NSETS], kclamp(kt + u + 1 + NSETS), kt + u + 1 < nk);
   }
#pragma unroll
   for (int u = 0; u < UNR - 1; ++u)
      if (kt + u < nk) kstep(u & 1, G[(u + 1) % NSETS], klast, kt + u + 1 < nk);
   __syncthreads();

   tile_epilogue<Mma, TI, TJ, OUT, 4>(g, acc, smem, tid, m0 + wm * (TJ * 32), n0, wn, BN);
}

// ---------------------------------------------------------------------------------------
// k_gemm_dma: both operands K-contiguous (A [M,K], B^T [N,K]).
//
// 512 threads = 8 wavefronts, two per SIMD, on a 256x256 output tile; a wavefront owns
// 128 columns x 64 rows (4x2 MFMA tiles of 32x32). The operand tiles of a K-step (64 bytes
// of K) travel HBM/L2 -> LDS with buffer_load_dwordx4 ... lds: no registers and no
// ds_write are spent on staging, and NST LDS stages keep NST-1 K-steps of requests in
// flight. A 1 KB load block holds 16 rows x 64 bytes; the 16-byte chunk c of row r sits in
// slot c ^ ((r >> 2) & 3), which makes the 16-byte-per-lane MFMA operand reads of 16
// consecutive rows hit 16 distinct bank groups without any padding (the DMA writes LDS
// linearly, so the permutation is applied to the global address of each lane instead).
// Out-of-range rows come back as zeros through the buffer descriptor's size check.
// The LDS-DMA instructions are issued from inline assembly so that their completion is
// waited for explicitly (s_waitcnt vmcnt) one stage at a time.
#ifndef SOFIE_DMA_BK
#define SOFIE_DMA_BK 128   // bytes of K per LDS stage of k_gemm_dma
#define SOFIE_DMA_NST 2    // LDS stages
#endif
#ifndef SOFIE_GEMM16
#define SOFIE_GEMM16 1
#endif
// Ablation builds of k_gemm_dma16 for timing only (make ABLATE=...; the results are wrong by construction): bit 0 leaves
// out the LDS-DMA requests after the first two K-steps, bit 1 the fragment reads after the first K-step, bit 2 the matrix
// instructions. Waits, barriers, prologue and epilogue stay. 0 in the library that is shipped.
#ifndef SOFIE_GEMM_ABLATE
#define SOFIE_GEMM_ABLATE 0
#endif
template <int S> struct StageTag { static constexpr int value = S; };

// LDS of k_gemm_dma: [A stage 0][A stage 1][B stage 0][B stage 1], BM*BK (BN*BK) bytes each. Both stages of an
// operand lie within 64 KB of its first byte, so a fragment read is one per-lane base register plus a constant in the
// instruction's 16-bit offset field for either stage, and the K loop (unrolled over the two stages) holds no
// address arithmetic in the vector unit.
// LOOP: the persistent form for launches with more tiles than compute units. A workgroup walks over the tiles
// blockIdx.x, blockIdx.x + gridDim.x, ... (each XCD keeps its compact rectangle of tiles) and the K loop runs on
// across the tile boundary: the last K-step of a tile requests the first K-step of the next one instead of a dummy, the
// second follows as soon as its stage is free, and the epilogue in between works in LDS of its own (a 64-byte-wide
// staging block per wavefront and the tile's scales and biases, behind the 128 KB of operand stages), so that the next
// tile's operands land while the present tile is converted and stored, the stores of a tile drain under the next
// tile's matrix instructions, and a compute unit never waits for a workgroup to end and the next one to start.
// Needs an even number of K-steps (the stages keep their roles from tile to tile) and 1- or 2-byte outputs.
template <class Mma, int BK, int NST, int OUT, bool B_KN, bool LOOP = false>
__global__ void __launch_bounds__(512, 2) k_gemm_dma(GemmArgs g)
{
   static_assert(!B_KN || BK == 128, "the [K,N] operand path is laid out for 128-byte stages");
   static_assert(NST == 2, "two stages per operand");
   constexpr int BM = 256, BN = 256;
   constexpr int TI = 4, TJ = 2;                      // wavefront tile: 128 n x 64 m
   constexpr int ABYTES = BM * BK, BBYTES = BN * BK;  // one stage of an operand
   constexpr int BREG = NST * ABYTES;                 // first byte of the B region
   constexpr int NSUB = BK / Mma::KB;
   constexpr int CPR = BK / 16;                       // 16-byte chunks per row
   constexpr int RPB = 1024 / BK;                     // rows per 1 KB load block
   constexpr int SWS = BK == 64 ? 2 : 1;              // swizzle: chunk ^ ((row >> SWS) & (CPR-1))
   static_assert(BK == 64 || BK == 128, "stage depth");
   static_assert(ABYTES * NST <= 65536 && BBYTES * NST <= 65536, "both stages of an operand within reach of the offset field");
   extern __shared__ __align__(16) unsigned char smem[];
   const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;

   const int tid = threadIdx.x, lane = tid & 63;
   // the wavefront index is uniform: as a scalar it keeps everything derived from it (operand choice, load
   // blocks, LDS destinations, descriptor) in scalar registers and the branches on it scalar branches
   const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int wn = wave & 1, wm = wave >> 1;

   // --- loads: wavefronts 0-3 request the A tile, 4-7 the B^T tile -------------------------
   constexpr int LPW = (BM + BN) / RPB / 8;           // load blocks per wavefront and stage
   const bool uses_a = wave < 4;
   const bool rows_are_k = B_KN && !uses_a;            // B [K,N]: a load block is 4 rows of k x 256 bytes of n
   const int ld = uses_a ? g.lda : g.ldb;
   const int rows_total = uses_a ? g.M : g.N;
   // What changes from tile to tile: the first row and column, and the descriptor of this wavefront's operand panel.
   struct Tile {
      rsrc_t rs;
      int m0, n0;
   };
   auto describe = [&](int pid) {
      Tile T;
      int tm, tn;
      tile_of_workgroup(pid, g.tiles_m, g.tiles_n, tm, tn);
      T.m0 = tm * BM;
      T.n0 = tn * BN;
      const int row0 = uses_a ? T.m0 : T.n0;
      const int rows_left = (rows_total - row0) < 256 ? (rows_total - row0) : 256;
      const unsigned char *tile_base = rows_are_k ? g.B + T.n0 : (uses_a ? g.A : g.B) + (size_t)row0 * ld;
      // rows of k past K lie beyond the descriptor and read as zeros
      T.rs = make_rsrc(tile_base, rows_are_k ? (unsigned)((size_t)(g.K - 1) * ld + (g.N - T.n0))
                                             : (unsigned)((size_t)(rows_left - 1) * ld + g.K));
      return T;
   };
   Tile cur = describe(blockIdx.x);
   const int blk0 = (wave & 3) * LPW;                  // first load block of this wavefront inside its operand's stage
   const int lrow = lane / CPR;                        // row inside a block
   // K-chunk this lane fetches in load block i: slot ^ swizzle(row); for BK = 128 the row
   // bits that enter the swizzle include the parity of the block
   int chunk[2], voff[2];
#pragma unroll
   for (int par = 0; par < 2; ++par) {
      const int row_in_tile = par * RPB + lrow;        // low bits only matter
      chunk[par] = (lane % CPR) ^ ((row_in_tile >> SWS) & (CPR - 1));
      voff[par] = (blk0 * RPB + lrow) * ld + chunk[par] * 16;
   }
   if (rows_are_k) {
      // [K,N] stage: row k holds 256 bytes of n as eight 32-byte pairs, pair p stored in slot p ^ (k & 7),
      // so that the transposing LDS reads (eight rows of k, 32 bytes of n each) cover every bank once
#pragma unroll
      for (int par = 0; par < 2; ++par) {
         const int krow = par * 4 + (lane >> 4);
         const int slot = lane & 15;
         chunk[par] = (((slot >> 1) ^ (krow & 7)) << 1) | (slot & 1);
         voff[par] = (blk0 * 4 + (lane >> 4)) * ld + chunk[par] * 16;
      }
   }
   const bool ktail = !LOOP && (g.K % BK) != 0;     // (the persistent form is launched on whole K-steps only)
   const int nk = (g.K + BK - 1) / BK;
   // per-lane offsets of the last, partial K-step: chunks at or past K point beyond the descriptor and read as zeros
   int voff_tail[2] = {voff[0], voff[1]};
   if (ktail && !rows_are_k) {
#pragma unroll
      for (int par = 0; par < 2; ++par)
         if ((nk - 1) * BK + chunk[par] * 16 >= g.K) voff_tail[par] = 0x7ffffff0;
   }
   const unsigned dst0 = lds0 + (uses_a ? 0 : BREG) + blk0 * 1024;   // this wavefront's first block in stage 0
   const int row_step = rows_are_k ? 4 * ld : RPB * ld;
   const int k_step = rows_are_k ? BK * ld : BK;
   // tile of K-step t -> stage S of its operand; steps past the end repeat the last tile into a stage nobody reads
   // any more, so the number of loads in flight never changes
   auto request = [&](const rsrc_t &rs, int t, int S) {
      const int tt = t < nk ? t : nk - 1;
      const bool tail = ktail && tt == nk - 1;
      const int v0 = tail ? voff_tail[0] : voff[0], v1 = tail ? voff_tail[1] : voff[1];
      const unsigned dst = dst0 + S * (uses_a ? ABYTES : BBYTES);
      const int k_off = tt * k_step;
#pragma unroll
      for (int i = 0; i < LPW; ++i) dma16(rs, dst + i * 1024, (BK == 128 && (i & 1)) ? v1 : v0, i * row_step + k_off);
   };
   // --- MFMA operand addresses ---------------------------------------------------------
   const int fr = lane & 31, half = lane >> 5;
   const int sw = (fr >> SWS) & (CPR - 1);
   // byte offset of this lane's first chunk inside a stage; later chunks differ by XOR
   // The order in which K is consumed is free as long as both operands agree, so the lower
   // and upper half of the wavefront always read chunks that differ in bit 1 (slot ^ 2):
   // with the row swizzle this keeps the two halves of one ds_read_b128 off each other's banks.
   const int first_chunk = half * 2;
   const int n_off = BREG + (wn * 128 + fr) * BK + ((first_chunk ^ sw) * 16);
   const int m_off = (wm * 64 + fr) * BK + ((first_chunk ^ sw) * 16);
   // The chunk of sub-step `sub` is the first one XOR a constant below 128 bytes: four patterns in all
   // (0, 16, 64, 80), one base register each per operand; tile index and stage are constants on top.
   const unsigned char *m_base[4], *n_base[4];
#pragma unroll
   for (int p = 0; p < 4; ++p) {
      const int pat = (p & 1) * 16 + (p >> 1) * 64;
      m_base[p] = smem + (m_off ^ pat);
      n_base[p] = smem + (n_off ^ pat);
   }
   // tile_off: i * 32 * BK (j * 32 * BK); stage_off: S * ABYTES (S * BBYTES)
   auto load_frag = [&](const unsigned char *const (&base)[4], int tile_off, int stage_off, int sub) -> typename Mma::Frag {
      if constexpr (Mma::LANE_BYTES == 16) {      // chunk = (sub/2)*4 + half*2 + sub%2: pattern index = sub
         return *reinterpret_cast<const v4i *>(base[sub] + tile_off + stage_off);
      } else {                                    // chunks sub*4 + half*2 + {0,1}: patterns 2*sub, 2*sub + 1
         const v4i lo = *reinterpret_cast<const v4i *>(base[2 * sub] + tile_off + stage_off);
         const v4i hi = *reinterpret_cast<const v4i *>(base[2 * sub + 1] + tile_off + stage_off);
         typename Mma::Frag f = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
         return f;
      }
   };

   // B [K,N]: ds_read_b64_tr_b8 hands a lane eight consecutive k of its column. Of a group of 16 lanes,
   // lane s points at row (s >> 1), bytes (s & 1) * 8 .. + 7 of the group's 16 columns; lane t of the
   // group then receives column t of those eight rows. A fragment is the same K slice the A operand reads.
   // The 32-byte pair of tile i is XORed into the address (bits 5-6): one base register per tile, with the
   // half-wavefront's two chunks of K folded in; chunk, row group and stage are constants on top.
   const int ts = lane & 15;
   const int kn_off = BREG + (ts >> 1) * 256 + ((((wn * 4) ^ (ts >> 1)) & 7) * 32) + ((lane >> 4) & 1) * 16 + (ts & 1) * 8 +
                      half * 2 * 16 * 256;
   const unsigned char *kn_base[TI];
#pragma unroll
   for (int i = 0; i < TI; ++i) kn_base[i] = smem + (kn_off ^ (i * 32));
   auto load_frag_kn = [&](int i, int stage_off, int sub) -> typename Mma::Frag {
      typedef int v2i_t __attribute__((ext_vector_type(2)));
      constexpr int NR = Mma::LANE_BYTES / 8;
      // first 16-byte chunk of K of sub-step `sub` without the half-wavefront's share (as in load_frag)
      const int ck = Mma::LANE_BYTES == 16 ? (sub >> 1) * 4 + (sub & 1) : sub * 4;
      const unsigned char *p = kn_base[i] + ck * 16 * 256 + stage_off;
      typename Mma::Frag f;
#pragma unroll
      for (int v = 0; v < NR; ++v) {
         const v2i_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (v2i_t __attribute__((address_space(3))) *)(p + v * 8 * 256));
         f[2 * v] = r[0];
         f[2 * v + 1] = r[1];
      }
      return f;
   };

   typename Mma::Acc acc[TI][TJ];
   auto clear_acc = [&]() {
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
         for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
   };
   clear_acc();
   // scale and bias of the thread's column, in registers across the K loop (the persistent form sends them to LDS
   // per tile instead, see below)
   ColumnParams col_params = {0.0f, 0};
   if constexpr (!LOOP) col_params = load_column_params(g, tid, cur.n0, BN);

   // --- LDS of the persistent form's epilogue, behind the operand stages: per wavefront a staging block of 32 rows x 64
   // bytes and the scales and biases of its 128 columns. Private to the wavefront: no workgroup barrier guards it.
   constexpr int ESZ = OutSize<OUT>::value;
   constexpr int TP = ESZ <= 2 ? 64 / (32 * ESZ) : 1;        // 32-column tiles per epilogue pass: 64 bytes of a row
   constexpr int WBX = EpilogueStaging<TP, OUT>::WAVE_BYTES;
   constexpr int XREG = NST * (ABYTES + BBYTES);
   unsigned char *const x_stg = smem + XREG + wave * WBX;
   float *const x_scale = reinterpret_cast<float *>(smem + XREG + 8 * WBX + wave * 1024);
   int *const x_bias = reinterpret_cast<int *>(x_scale + 128);
   constexpr bool IS_INT = __is_same(typename Mma::Acc, v16i);
   // stores of a full tile's epilogue and parameter loads of a tile per wavefront: the first wait of the next tile
   // counts past them instead of waiting for them
   constexpr int EPI_STORES = (TI / TP) * TJ * (32 * (TP * 32 * ESZ / 16) / 64);
   const int param_loads = ((IS_INT && g.scale) ? 2 : 0) + (g.bias ? 2 : 0);
   // The tile's per-column parameters travel straight into the wavefront's LDS block, one dword per lane and
   // instruction; columns past N lie beyond the descriptor and read as zero.
   // (the lane index is read off the hardware where the epilogue needs it: one register less across the K loop)
   auto lane_now = [&]() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); };
   auto request_params = [&](int n0) {
      const int nw = n0 + wn * 128;
      const int lane = lane_now();
      const unsigned xs = lds0 + XREG + 8 * WBX + wave * 1024;
      if (IS_INT && g.scale) {
         const rsrc_t srs = make_rsrc(g.scale, (unsigned)g.N * 4u);
         dma4(srs, xs, (nw + lane) * 4, 0);
         dma4(srs, xs + 256, (nw + 64 + lane) * 4, 0);
      }
      if (g.bias) {
         const rsrc_t brs = make_rsrc(g.bias, (unsigned)g.N * 4u);
         dma4(brs, xs + 512, (nw + lane) * 4, 0);
         dma4(brs, xs + 768, (nw + 64 + lane) * 4, 0);
      }
   };

   // --- ping-pong schedule -----------------------------------------------------------------
   // The two wavefronts of a SIMD run half a K-step apart: while one multiplies (MFMAs only,
   // operands already in registers) the other issues the LDS-DMA requests and reads its next
   // operands from LDS; a workgroup barrier ends every phase. Group 1 gets its phase shift
   // from one extra barrier at the start, group 0 pays it back after its last multiply.
   const int group = wave >> 2;
   auto barrier = [&]() {
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
   };
   // the first two K-steps are requested together: the second one's way from memory runs under the first one's
   if (nk > 0) {
      request(cur.rs, 0, 0);
      request(cur.rs, 1, 1);
      wait_vmcnt<LPW>();                // this wavefront's part of stage 0 has landed
   }
   if constexpr (LOOP) {
      // without a bias (or scales) the block reads as zeros for the life of the kernel
      x_scale[lane] = 0.0f; x_scale[64 + lane] = 0.0f;
      x_bias[lane] = 0; x_bias[64 + lane] = 0;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
   }
   barrier();
   const int tiles = g.tiles_m * g.tiles_n;
   int pid = blockIdx.x;
   bool stores_behind = false;          // the previous tile's epilogue left exactly EPI_STORES stores in the queue
   for (;;) {
      const int pid_next = pid + (int)gridDim.x;
      const bool has_next = LOOP && pid_next < tiles;
      Tile nxt = cur;
      if (has_next) nxt = describe(pid_next);
      if (group == 1) barrier();
      if constexpr (LOOP) request_params(cur.n0);
      // one K-step on the tile in stage S (a compile-time constant: the loop below is unrolled over the two stages)
      auto kstep = [&](int t, auto tag) {
         constexpr int S = decltype(tag)::value;
         // load phase: requests for K-step t+1 into the other stage (last read one phase ago), then
         // every operand fragment of stage S into registers. The requests go first: issued behind the fragment reads
         // they land later and the phase that waits for them grows (measured: 63.2 us instead of 59.9 us at 4096^3).
         if (t > 0) {
            if (!LOOP || t + 1 < nk) request(cur.rs, t + 1, 1 - S);
            else if (has_next) request(nxt.rs, 0, 1 - S);      // the next tile's first K-step
         }
         typename Mma::Frag fn[NSUB][TI], fm[NSUB][TJ];
#pragma unroll
         for (int sub = 0; sub < NSUB; ++sub) {
#pragma unroll
            for (int i = 0; i < TI; ++i) {
               if constexpr (B_KN) fn[sub][i] = load_frag_kn(i, S * BBYTES, sub);
               else fn[sub][i] = load_frag(n_base, i * 32 * BK, S * BBYTES, sub);
            }
#pragma unroll
            for (int j = 0; j < TJ; ++j) fm[sub][j] = load_frag(m_base, j * 32 * BK, S * ABYTES, sub);
         }
         __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): fragments are in registers
         // The other stage is first read by group 0 right after the barrier that ends its multiply
         // phase, which is the barrier that ends group 1's load phase: each group waits for its
         // own part of it just before that barrier. (Completion is reported in the order of issue: in the first
         // K-step of a later tile the requests of its second K-step are followed by the previous tile's stores
         // and this tile's parameter loads, which the wait counts past.)
         auto wait_requests = [&]() {
            if (LOOP && S == 0 && t == 0 && stores_behind) {
               if (param_loads == 4) wait_vmcnt<EPI_STORES + 4>();
               else if (param_loads == 2) wait_vmcnt<EPI_STORES + 2>();
               else wait_vmcnt<EPI_STORES>();
            } else {
               wait_vmcnt<0>();
            }
         };
         if (group == 1) wait_requests();
         barrier();
         // multiply phase
         // The n tiles of an m tile are walked back and forth: every instruction shares an operand with the one before
         // it (FP8 8192 x 8192 x 4096: 0.1 - 0.9 % in each of ten alternating comparisons).
#pragma unroll
         for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
               for (int ii = 0; ii < TI; ++ii) {
                  const int i = (j & 1) ? TI - 1 - ii : ii;
                  acc[i][j] = Mma::mma(fn[sub][i], fm[sub][j], acc[i][j]);
               }
         if (group == 0) wait_requests();
         if (group == 0 || t + 1 < nk) barrier();
      };
      for (int t = 0; t < nk; t += 2) {
         kstep(t, StageTag<0>{});
         if (t + 1 < nk) kstep(t + 1, StageTag<1>{});
      }
      if constexpr (!LOOP) break;
      // Both groups are past the barrier behind the last load phase: stage 1 is free, the next tile's first K-step
      // is complete in stage 0 (every wavefront waited for its part before that barrier).
      if (has_next) request(nxt.rs, 1, 1);
      {
         const int m_wave = cur.m0 + wm * 64, n_wave = cur.n0 + wn * 128;
         const bool full = g.vec_store && cur.m0 + BM <= g.M && cur.n0 + BN <= g.N;
         const int mode = (OUT == SOFIE_OUT_S8 && g.zp == -128 && g.lo == -128) ? 1 : (OUT == SOFIE_OUT_S8 && g.lo == -128) ? 2 : 0;
         // The epilogue's per-lane addresses are worked out afresh for every tile, from a lane index the compiler cannot
         // trace to the one above: as loop invariants they would be kept in registers (that is, in scratch memory) across
         // the K loop, which has none to spare.
         const int lane_e = lane_now();
#pragma unroll
         for (int i0 = 0; i0 < TI; i0 += TP) {
            typename Mma::Acc(&part)[TP][TJ] = reinterpret_cast<typename Mma::Acc(&)[TP][TJ]>(acc[i0]);
            // written through on the workgroup's last tile only: nothing follows that their way out could run under
            if (mode == 1) tile_epilogue_wave<Mma, TP, TJ, OUT, 1>(g, part, x_stg, x_scale + i0 * 32, x_bias + i0 * 32, lane_e, m_wave, n_wave + i0 * 32, nullptr, !has_next);
            else if (mode == 2) tile_epilogue_wave<Mma, TP, TJ, OUT, 2>(g, part, x_stg, x_scale + i0 * 32, x_bias + i0 * 32, lane_e, m_wave, n_wave + i0 * 32, nullptr, !has_next);
            else tile_epilogue_wave<Mma, TP, TJ, OUT, 0>(g, part, x_stg, x_scale + i0 * 32, x_bias + i0 * 32, lane_e, m_wave, n_wave + i0 * 32, nullptr, !has_next);
         }
         stores_behind = full;
      }
      if (!has_next) return;
      clear_acc();
      cur = nxt;
      pid = pid_next;
   }
   wait_vmcnt<0>();                         // the trailing dummy requests still target LDS
   __syncthreads();
   tile_epilogue<Mma, TI, TJ, OUT, 8>(g, acc, smem, tid, cur.m0 + wm * 64, cur.n0, wn, BN, &col_params);
}

// k_gemm_dma16: the int8 kernel above (B^T [N,K] or B [K,N]) on v_mfma_i32_16x16x64_i8 instead of v_mfma_i32_32x32x32_i8.
// Same tile, stages, requests and two-group schedule; a wavefront's 128 x 64 part is 8 x 4 accumulator tiles of
// 16 x 16. The instruction does the same multiply-adds per cycle, writes half as many accumulator values per
// multiply-add and draws less power: under the device's power limit a loop of it on random operands sustains about
// 13 % more than the 32 x 32 one (4.0 against 3.5 POP/s). A lane supplies row (lane % 16) of a tile and the 16 bytes of
// K number lane / 16 of a 64-byte sub-step, so its LDS address is the row's base plus chunk ((lane / 16) ^ swizzle)
// and the second sub-step of a 128-byte stage is that address XOR 64.
template <int OUT, bool B_KN>
__global__ void __launch_bounds__(512, 2) k_gemm_dma16(GemmArgs g)
{
   constexpr int BK = 128, NST = 2;
   constexpr int BM = 256, BN = 256;
   constexpr int NI = 8, MJ = 4;                      // wavefront tile: 128 n x 64 m
   constexpr int ABYTES = BM * BK, BBYTES = BN * BK;
   constexpr int BREG = NST * ABYTES;
   constexpr int NSUB = BK / 64;
   constexpr int CPR = BK / 16, RPB = 1024 / BK;
   extern __shared__ __align__(16) unsigned char smem[];
   const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
   const int tid = threadIdx.x, lane = tid & 63;
   const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int wn = wave & 1, wm = wave >> 1;
   int tm, tn;
   // an XCD's 32 tiles of a 4096^3 product: 8 m x 4 n with B [K,N] (49.4 - 50.9 against 49.7 - 51.6 us, eight of
   // eight alternating comparisons), 4 m x 8 n with B [N,K] (no difference there; 2 x 16 and 16 x 2 cost 1.5 - 2.5 %)
   tile_of_workgroup<B_KN ? 8 : 4>(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
   const int m0 = tm * BM, n0 = tn * BN;

   // --- loads: as in k_gemm_dma (wavefronts 0-3 request the A tile, 4-7 the B^T tile)
   constexpr int LPW = (BM + BN) / RPB / 8;
   const bool uses_a = wave < 4;
   const int ld = uses_a ? g.lda : g.ldb;
   const int rows_total = uses_a ? g.M : g.N;
   const int row0 = uses_a ? m0 : n0;
   const int rows_left = (rows_total - row0) < 256 ? (rows_total - row0) : 256;
   const bool rows_are_k = B_KN && !uses_a;            // B [K,N]: a load block is 4 rows of k x 256 bytes of n
   const unsigned char *tile_base = rows_are_k ? g.B + n0 : (uses_a ? g.A : g.B) + (size_t)row0 * ld;
   // rows of k past K lie beyond the descriptor and read as zeros
   const rsrc_t rs = make_rsrc(tile_base, rows_are_k ? (unsigned)((size_t)(g.K - 1) * ld + (g.N - n0))
                                                     : (unsigned)((size_t)(rows_left - 1) * ld + g.K));
   const int blk0 = (wave & 3) * LPW;
   const int lrow = lane / CPR;
   const bool ktail = (g.K % BK) != 0;
   const int nk = (g.K + BK - 1) / BK;
   int voff[2], voff_tail[2];
#pragma unroll
   for (int par = 0; par < 2; ++par) {
      const int chunk = (lane % CPR) ^ (((par * RPB + lrow) >> 1) & (CPR - 1));
      voff[par] = (blk0 * RPB + lrow) * ld + chunk * 16;
      voff_tail[par] = (ktail && (nk - 1) * BK + chunk * 16 >= g.K) ? 0x7ffffff0 : voff[par];
   }
   if (rows_are_k) {
      // [K,N] stage: row k holds 256 bytes of n as eight 32-byte pairs, pair p stored in slot p ^ (k & 7), so that
      // the transposing LDS reads (eight rows of k, 16 bytes of n each) of a group of 16 lanes cover distinct banks
#pragma unroll
      for (int par = 0; par < 2; ++par) {
         const int krow = par * 4 + (lane >> 4);
         const int slot = lane & 15;
         const int chunk = (((slot >> 1) ^ (krow & 7)) << 1) | (slot & 1);
         voff[par] = (blk0 * 4 + (lane >> 4)) * ld + chunk * 16;
         voff_tail[par] = voff[par];
      }
   }
   const unsigned dst0 = lds0 + (uses_a ? 0 : BREG) + blk0 * 1024;
   const int row_step = rows_are_k ? 4 * ld : RPB * ld;
   const int k_step = rows_are_k ? BK * ld : BK;
   auto request = [&](int t, int S) {
      const int tt = t < nk ? t : nk - 1;
      const bool tail = ktail && tt == nk - 1;      // B [K,N]: both offsets are the same
      const int v0 = tail ? voff_tail[0] : voff[0], v1 = tail ? voff_tail[1] : voff[1];
      const unsigned dst = dst0 + S * (uses_a ? ABYTES : BBYTES);
#pragma unroll
      for (int i = 0; i < LPW; ++i) dma16(rs, dst + i * 1024, (i & 1) ? v1 : v0, i * row_step + tt * k_step);
   };
   // --- operand addresses: row lane % 16 of a tile, chunk (lane / 16) of the sub-step, swizzled by the row
   const int fr = lane & 15, kg = lane >> 4;
   const int sw = (fr >> 1) & 7;
   const int n_off = BREG + (wn * 128 + fr) * BK + ((kg ^ sw) * 16);
   const int m_off = (wm * 64 + fr) * BK + ((kg ^ sw) * 16);
   const unsigned char *m_base[NSUB], *n_base[NSUB];
#pragma unroll
   for (int sub = 0; sub < NSUB; ++sub) {
      m_base[sub] = smem + (m_off ^ (sub * 64));
      n_base[sub] = smem + (n_off ^ (sub * 64));
   }
   // B [K,N]: ds_read_b64_tr_b8 hands a lane eight consecutive k of its column. Of a group of 16 lanes (one 16-byte
   // chunk of K), lane s points at row (s >> 1), bytes (s & 1) * 8 .. + 7 of the tile's 16 columns; lane t of the group
   // then receives column t of those eight rows. Two tiles share a 32-byte pair: the pair's slot is XORed into the
   // address, the half of the pair, the sub-step, the eight-row half and the stage are constants on top.
   const int ts = lane & 15;
   const int kn_off = BREG + (ts >> 1) * 256 + ((((wn * 4) ^ (ts >> 1)) & 7) * 32) + (ts & 1) * 8 + kg * 16 * 256;
   const unsigned char *kn_base[NI / 2];
#pragma unroll
   for (int ip = 0; ip < NI / 2; ++ip) kn_base[ip] = smem + (kn_off ^ (ip * 32));
   auto load_frag_kn = [&](int i, int stage_off, int sub) -> v4i {
      typedef int v2i_t __attribute__((ext_vector_type(2)));
      const unsigned char *p = kn_base[i >> 1] + (i & 1) * 16 + sub * 64 * 256 + stage_off;
      const v2i_t lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i_t __attribute__((address_space(3))) *)(p));
      const v2i_t hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i_t __attribute__((address_space(3))) *)(p + 8 * 256));
      return v4i{lo[0], lo[1], hi[0], hi[1]};
   };
   v4i acc[NI][MJ];
#pragma unroll
   for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < MJ; ++j) acc[i][j] = v4i{0, 0, 0, 0};
   const ColumnParams col_params = load_column_params(g, tid, n0, BN);

   const int group = wave >> 2;
   auto barrier = [&]() {
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
   };
   // the first two K-steps are requested together: the second one's way from memory runs under the first one's
   if (nk > 0) {
      request(0, 0);
      request(1, 1);
      wait_vmcnt<LPW>();               // this wavefront's part of stage 0 has landed
   }
   barrier();
   if (group == 1) barrier();
   constexpr bool NO_REQUESTS = (SOFIE_GEMM_ABLATE & 1) != 0, NO_READS = (SOFIE_GEMM_ABLATE & 2) != 0,
                  NO_MFMA = (SOFIE_GEMM_ABLATE & 4) != 0;
   v4i fn[NSUB][NI], fm[NSUB][MJ];          // (inside a K-step in effect: every step rewrites all of them)
   auto kstep = [&](int t, auto tag) {
      constexpr int S = decltype(tag)::value;
      if (t > 0 && !NO_REQUESTS) request(t + 1, 1 - S);
      if (!NO_READS || t == 0) {
#pragma unroll
         for (int sub = 0; sub < NSUB; ++sub) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
               if constexpr (B_KN) fn[sub][i] = load_frag_kn(i, S * BBYTES, sub);
               else fn[sub][i] = *reinterpret_cast<const v4i *>(n_base[sub] + i * 16 * BK + S * BBYTES);
            }
#pragma unroll
            for (int j = 0; j < MJ; ++j) fm[sub][j] = *reinterpret_cast<const v4i *>(m_base[sub] + j * 16 * BK + S * ABYTES);
         }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
      if (group == 1) wait_vmcnt<0>();
      barrier();
      if constexpr (NO_MFMA) {
         // the fragments stay "used", so that their reads are not removed with the instructions that consume them
#pragma unroll
         for (int sub = 0; sub < NSUB; ++sub) {
#pragma unroll
            for (int i = 0; i < NI; ++i) asm volatile("" ::"v"(fn[sub][i]));
#pragma unroll
            for (int j = 0; j < MJ; ++j) asm volatile("" ::"v"(fm[sub][j]));
         }
      } else {
         // The m tiles are walked back and forth (0..3 with an even n tile, 3..0 with an odd one): every instruction
         // then shares one operand with the one before it. 51.1 - 51.7 against 51.6 - 52.2 us (B [K,N]) and 48.8 - 49.4
         // against 49.6 - 50.4 us (B [N,K]) at 4096^3, alternating in one process; with the n tiles innermost, or the
         // two K halves of a tile one behind the other, nothing or a loss.
#pragma unroll
         for (int sub = 0; sub < NSUB; ++sub)
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
               for (int jj = 0; jj < MJ; ++jj) {
                  const int j = (i & 1) ? MJ - 1 - jj : jj;
                  acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fn[sub][i], fm[sub][j], acc[i][j], 0, 0, 0);
               }
      }
      if (group == 0) wait_vmcnt<0>();
      if (group == 0 || t + 1 < nk) barrier();
   };
   for (int t = 0; t < nk; t += 2) {
      kstep(t, StageTag<0>{});
      if (t + 1 < nk) kstep(t + 1, StageTag<1>{});
   }
   wait_vmcnt<0>();
   __syncthreads();
   // epilogue: staging blocks of the eight wavefronts, then scales and biases of the tile's columns
   constexpr int WB = EpilogueStaging<NI / 2, OUT>::WAVE_BYTES;
   float *s_scale = reinterpret_cast<float *>(smem + 8 * WB);
   int *s_bias = reinterpret_cast<int *>(s_scale + BN);
   if (tid < BN) {
      s_scale[tid] = col_params.scale;
      s_bias[tid] = col_params.bias;
   }
   __syncthreads();
   unsigned char *stg = smem + wave * WB;
   const int m_wave = m0 + wm * 64, n_wave = n0 + wn * 128;
   if constexpr (OUT == SOFIE_OUT_S8) {
      // Tiles whose columns all lie inside the matrix, rows that take 16-byte stores: no LDS staging (50.7 against
      // 51.4 us with B [K,N], 48.6 against 49.0 us with B [N,K] at 4096^3, alternating in one process). (Built on top
      // and not kept: the wavefronts' scales and biases by 4-byte LDS-DMA into blocks of their own, so that no workgroup
      // barrier stands between a wavefront's last matrix instruction and its epilogue: the same time within 0.4 us.)
      if (g.vec_store && n0 + BN <= g.N) {
         if (g.zp == -128 && g.lo == -128) tile_epilogue_wave16_direct<NI, MJ, 1>(g, acc, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
         else if (g.lo == -128 && !g.bias) tile_epilogue_wave16_direct<NI, MJ, 2, false>(g, acc, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
         else if (g.lo == -128) tile_epilogue_wave16_direct<NI, MJ, 2>(g, acc, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
         else tile_epilogue_wave16_direct<NI, MJ, 0>(g, acc, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
         return;
      }
   }
   if (OUT == SOFIE_OUT_S8 && g.zp == -128 && g.lo == -128)
      tile_epilogue_wave16<NI, MJ, OUT, 1>(g, acc, stg, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
   else if (OUT == SOFIE_OUT_S8 && g.lo == -128)
      tile_epilogue_wave16<NI, MJ, OUT, 2>(g, acc, stg, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
   else
      tile_epilogue_wave16<NI, MJ, OUT, 0>(g, acc, stg, s_scale + wn * 128, s_bias + wn * 128, lane, m_wave, n_wave);
}

// Byte-matrix transpose src [R, C] (ld_src) -> dst [C, R] (ld_dst), R % 16 == 0, C % 4 == 0.
// A thread takes 16 rows x 4 columns (16 dwords), transposes them in registers with
// v_perm_b32 and writes four 16-byte row segments; eight neighbouring lanes write 128
// contiguous bytes of one output row. HBM-bound: R*C bytes in, R*C bytes out.
__global__ void __launch_bounds__(256) k_transpose_bytes(const unsigned char *__restrict__ src, unsigned char *__restrict__ dst,
                                                         int R, int C, int ld_src, int ld_dst)
{
   const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
   const int rg = blockIdx.x * 8 + (lane & 7);                 // 16-row group
   const int cg = (blockIdx.y * 4 + wave) * 8 + (lane >> 3);   // 4-column group
   if (rg * 16 >= R || cg * 4 >= C) return;
   const unsigned char *p = src + (size_t)rg * 16 * ld_src + cg * 4;
   unsigned d[16];
#pragma unroll
   for (int r = 0; r < 16; ++r) d[r] = *reinterpret_cast<const unsigned *>(p + (size_t)r * ld_src);
   unsigned o[4][4];
#pragma unroll
   for (int q = 0; q < 4; ++q) {
      const unsigned t0 = __builtin_amdgcn_perm(d[4 * q + 1], d[4 * q + 0], 0x05010400u);
      const unsigned t1 = __builtin_amdgcn_perm(d[4 * q + 1], d[4 * q + 0], 0x07030602u);
      const unsigned t2 = __builtin_amdgcn_perm(d[4 * q + 3], d[4 * q + 2], 0x05010400u);
      const unsigned t3 = __builtin_amdgcn_perm(d[4 * q + 3], d[4 * q + 2], 0x07030602u);
      o[0][q] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
      o[1][q] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
      o[2][q] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
      o[3][q] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
   }
#pragma unroll
   for (int j = 0; j < 4; ++j) {
      const v4i v = {(int)o[j][0], (int)o[j][1], (int)o[j][2], (int)o[j][3]};
      *reinterpret_cast<v4i *>(dst + (size_t)(cg * 4 + j) * ld_dst + rg * 16) = v;
   }
}

int transpose_bytes(sofie_hip_ctx *ctx, const unsigned char *src, unsigned char *dst, int R, int C, int ld_src, int ld_dst)
{
   hipLaunchKernelGGL(k_transpose_bytes, dim3(cdiv(R, 128), cdiv(C, 128)), dim3(256), 0, ctx->stream, src, dst, R, C,
                      ld_src, ld_dst);
   return check_launch(ctx, "k_transpose_bytes");
}

// Any shape, any alignment: one thread per output element. Correctness path for operands
// the tiled kernel cannot take (K not a multiple of 16, unaligned rows).
template <bool IS_INT, int OUT>
__global__ void k_gemm_bytes_simple(GemmArgs g, int transB)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   if (idx >= (size_t)g.M * g.N) return;
   const int m = (int)(idx / g.N), n = (int)(idx % g.N);
   const uint8_t *a = g.A + (size_t)m * g.lda;
   constexpr int ESZ = OutSize<OUT>::value;
   unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + n) * ESZ;
   unsigned r;
   if constexpr (IS_INT) {
      int acc = 0;
      for (int k = 0; k < g.K; ++k) {
         const int b = (int)(int8_t)(transB ? g.B[(size_t)n * g.ldb + k] : g.B[(size_t)k * g.ldb + n]);
         acc += (int)(int8_t)a[k] * b;
      }
      r = epilogue_value<true, OUT>(g, g.scale ? g.scale[n] : 0.0f, g.bias ? static_cast<const int *>(g.bias)[n] : 0, acc, 0.0f);
   } else {
      float acc = 0.0f;
      for (int k = 0; k < g.K; ++k) {
         const unsigned b = transB ? g.B[(size_t)n * g.ldb + k] : g.B[(size_t)k * g.ldb + n];
         acc = __fadd_rn(acc, __fmul_rn(e4m3_to_f32(a[k]), e4m3_to_f32(b)));
      }
      r = epilogue_value<false, OUT>(g, 0.0f, g.bias ? static_cast<const int *>(g.bias)[n] : 0, 0, acc);
   }
   if constexpr (ESZ == 1) *out = (unsigned char)((int)fminf(__uint_as_float(r), 255.0f) - 128);
   else if constexpr (ESZ == 2) *reinterpret_cast<unsigned short *>(out) = (unsigned short)r;
   else *reinterpret_cast<unsigned *>(out) = r;
}

// int8 product with at most 16 output columns (the last layer of a classifier): B^T [N,K] is tiny and
// stays in cache, the work is streaming A. 16 lanes share a row of A, each takes every 16th 16-byte
// chunk of K and multiplies it into all N columns with v_dot4_i32_i8; the 16 partial sums of a column
// are added with four butterfly steps inside the 16-lane group. Four rows per wavefront.
template <int OUT, int NMAX>
__global__ void __launch_bounds__(256) k_qgemm_skinny(GemmArgs g)
{
   const int lane16 = threadIdx.x & 15;
   const int row = (int)(((size_t)blockIdx.x * 256 + threadIdx.x) >> 4);
   const int m = row < g.M ? row : g.M - 1;
   const uint8_t *a = g.A + (size_t)m * g.lda;
   int acc[NMAX];
#pragma unroll
   for (int n = 0; n < NMAX; ++n) acc[n] = 0;
   const int chunks = g.K >> 4;
   for (int c = lane16; c < chunks; c += 16) {
      const v4i av = *reinterpret_cast<const v4i *>(a + c * 16);
#pragma unroll
      for (int n = 0; n < NMAX; ++n) {
         if (n < g.N) {
            const v4i bv = *reinterpret_cast<const v4i *>(g.B + (size_t)n * g.ldb + c * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[n] = __builtin_amdgcn_sdot4(av[e], bv[e], acc[n], false);
         }
      }
   }
#pragma unroll
   for (int n = 0; n < NMAX; ++n) {
#pragma unroll
      for (int d = 1; d < 16; d <<= 1) acc[n] += __shfl_xor(acc[n], d, 16);
   }
   if (row >= g.M) return;
   constexpr int ESZ = OutSize<OUT>::value;
#pragma unroll
   for (int n = 0; n < NMAX; ++n) {
      if (n == lane16 && n < g.N) {
         const unsigned r = epilogue_value<true, OUT>(g, g.scale ? g.scale[n] : 0.0f,
                                                      g.bias ? static_cast<const int *>(g.bias)[n] : 0, acc[n], 0.0f);
         unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + n) * ESZ;
         if constexpr (ESZ == 1) *out = (unsigned char)((int)fminf(__uint_as_float(r), 255.0f) - 128);
         else *reinterpret_cast<unsigned *>(out) = r;
      }
   }
}

template <int OUT>
int launch_skinny(sofie_hip_ctx *ctx, GemmArgs &g)
{
   const dim3 grid((unsigned)(((size_t)g.M * 16 + 255) / 256)), block(256);
   if (g.N <= 8) hipLaunchKernelGGL((k_qgemm_skinny<OUT, 8>), grid, block, 0, ctx->stream, g);
   else hipLaunchKernelGGL((k_qgemm_skinny<OUT, 16>), grid, block, 0, ctx->stream, g);
   return check_launch(ctx, "k_qgemm_skinny");
}

template <class Mma, int OUT> struct IS_SPLITTABLE {
   static constexpr bool value = __is_same(typename Mma::Acc, v16i) && OUT == SOFIE_OUT_S32;
};

// Sum over the K slices of four consecutive int32 partial sums. The loads of four slices are issued together before
// the first addition (one after the other, each waiting for the one before, they were the length of the pass).
__device__ __forceinline__ v4i sum_slices(const int *__restrict__ p, size_t plane, int splits)
{
   v4i s = {0, 0, 0, 0};
   int k = 0;
   for (; k + 4 <= splits; k += 4) {
      const v4i a = *reinterpret_cast<const v4i *>(p + (size_t)k * plane);
      const v4i b = *reinterpret_cast<const v4i *>(p + (size_t)(k + 1) * plane);
      const v4i c = *reinterpret_cast<const v4i *>(p + (size_t)(k + 2) * plane);
      const v4i d = *reinterpret_cast<const v4i *>(p + (size_t)(k + 3) * plane);
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] += (a[e] + b[e]) + (c[e] + d[e]);
   }
   for (; k < splits; ++k) {
      const v4i v = *reinterpret_cast<const v4i *>(p + (size_t)k * plane);
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] += v[e];
   }
   return s;
}

// Sum of the K slices' int32 partial tiles, then bias and the output conversion of the unsplit kernel.
// One thread per four consecutive columns of one row; P is [splits][M][ldp], ldp a multiple of 4.
template <int OUT>
__global__ void __launch_bounds__(256) k_splitk_finish(GemmArgs g, const int *__restrict__ P, int splits, int ldp)
{
   const int quads = ldp >> 2;
   const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
   if (t >= (size_t)g.M * quads) return;
   const int m = (int)(t / quads), n = (int)(t % quads) * 4;
   const size_t plane = (size_t)g.M * ldp;
   const v4i s = sum_slices(P + (size_t)m * ldp + n, plane, splits);
   constexpr int ESZ = OutSize<OUT>::value;
   unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + n) * ESZ;
#pragma unroll
   for (int e = 0; e < 4; ++e) {
      if (n + e >= g.N) break;
      const unsigned r = epilogue_value<true, OUT>(g, g.scale ? g.scale[n + e] : 0.0f,
                                                   g.bias ? static_cast<const int *>(g.bias)[n + e] : 0, s[e], 0.0f);
      if constexpr (ESZ == 1) out[e] = (unsigned char)((int)fminf(__uint_as_float(r), 255.0f) - 128);
      else reinterpret_cast<unsigned *>(out)[e] = r;
   }
}

// The second, narrow layer of a pair behind a first layer whose K was cut into slices (a classifier's last two fully
// connected layers): the pass that adds the slices also requantises the first layer's row, multiplies it into the
// second layer's few columns and writes those; the first layer's output is never stored. g1 describes the first
// layer's requantisation (N = N1, scale, bias, zp, lo), g2 the second layer (B = its matrix [N2, ldb], N = N2 <= 8,
// K = N1, scale, bias, zp, lo, relu, Y, ldy). N1 / 4 threads share a row: a power of two of at most 64, so a row's
// threads are lanes of one wavefront and their partial dot products meet through lane shuffles.
// Sum of a value over the 64 lanes of a wavefront, delivered in lane 63: an inclusive scan inside each row of 16 lanes
// (row shifts by 1, 2, 4, 8), then the row totals travel to the following rows (lane 15 of a row to the next row,
// lane 31 to the upper half). Six vector instructions, no LDS.
__device__ __forceinline__ int wave_sum_in_lane63(int v)
{
   v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);
   v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);
   v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);
   v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);
   v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);
   v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);
   return v;
}

template <int OUT2, int QUADS>
__global__ void __launch_bounds__(256) k_splitk_finish_pair(GemmArgs g1, const int *__restrict__ P, int splits, int ldp, GemmArgs g2)
{
   constexpr int quads = QUADS;
   const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
   if (t >= (size_t)g1.M * quads) return;
   const int m = (int)(t / quads), c = (int)(t % quads), n = c * 4;
   const size_t plane = (size_t)g1.M * ldp;
   // everything the thread reads is requested before the first value is used
   float sc1[4];
   int b1[4], w2[8];
#pragma unroll
   for (int e = 0; e < 4; ++e) {
      sc1[e] = g1.scale[n + e];
      b1[e] = g1.bias ? static_cast<const int *>(g1.bias)[n + e] : 0;
   }
#pragma unroll
   for (int j = 0; j < 8; ++j) w2[j] = j < g2.N ? *reinterpret_cast<const int *>(g2.B + (size_t)j * g2.ldb + n) : 0;
   const v4i s = sum_slices(P + (size_t)m * ldp + n, plane, splits);
   unsigned packed = 0;
#pragma unroll
   for (int e = 0; e < 4; ++e) {
      const unsigned r = epilogue_value<true, SOFIE_OUT_S8>(g1, sc1[e], b1[e], s[e], 0.0f);
      packed |= ((unsigned)((int)fminf(__uint_as_float(r), 255.0f) - 128) & 0xffu) << (8 * e);
   }
   int dot[8];
#pragma unroll
   for (int j = 0; j < 8; ++j) {
      dot[j] = 0;
      if (j < g2.N) {      // uniform over the launch
         const int w = w2[j];
         dot[j] = __builtin_amdgcn_sdot4((int)packed, w, 0, false);
         if constexpr (QUADS == 64) {
            dot[j] = wave_sum_in_lane63(dot[j]);      // a row is a whole wavefront
         } else {
#pragma unroll
            for (int d = 1; d < quads; d <<= 1) dot[j] += __shfl_xor(dot[j], d);
         }
      }
   }
   // the thread that writes output j of the row: the last lane has every sum of a whole-wavefront row, otherwise
   // every lane of the row's group has them and lane j of the group writes
   const bool whole_wave = QUADS == 64;
   constexpr int ESZ = OutSize<OUT2>::value;
#pragma unroll
   for (int j = 0; j < 8; ++j) {
      if ((whole_wave ? c == 63 : j == c) && j < g2.N) {
         const unsigned r = epilogue_value<true, OUT2>(g2, g2.scale ? g2.scale[j] : 0.0f,
                                                       g2.bias ? static_cast<const int *>(g2.bias)[j] : 0, dot[j], 0.0f);
         unsigned char *out = static_cast<unsigned char *>(g2.Y) + ((size_t)m * g2.ldy + j) * ESZ;
         if constexpr (ESZ == 1) *out = (unsigned char)((int)fminf(__uint_as_float(r), 255.0f) - 128);
         else *reinterpret_cast<unsigned *>(out) = r;
      }
   }
}

template <class Mma, int BK, int NSETS, int TI, int TJ, int OUT, bool B_KN, bool FULL>
int launch_tiled_impl(sofie_hip_ctx *ctx, GemmArgs &g)
{
   constexpr int BN = 2 * TI * 32, BM = 2 * TJ * 32;
   constexpr int LDK = BK + 16;
   constexpr size_t stage_bytes = (size_t)2 * (BM + BN) * LDK;
   constexpr size_t epi_bytes = (size_t)4 * 32 * (TI * 32 * OutSize<OUT>::value + 16) + (size_t)2 * BN * 4;
   constexpr size_t lds = stage_bytes > epi_bytes ? stage_bytes : epi_bytes;
   static_assert(lds <= 160 * 1024, "tile does not fit the 160 KB LDS");
   g.tiles_m = cdiv(g.M, BM);
   g.tiles_n = cdiv(g.N, BN);
   constexpr auto kern = k_gemm_bytes<Mma, BK, NSETS, TI, TJ, OUT, B_KN, FULL>;
   SOFIE_LARGE_LDS(kern);
   const int splits = (IS_SPLITTABLE<Mma, OUT>::value && g.splits > 1) ? g.splits : 1;
   hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * splits), dim3(256), lds, ctx->stream, g);
   return check_launch(ctx, "k_gemm_bytes");
}

template <class Mma, int BK, int NSETS, int TI, int TJ, int OUT, bool B_KN>
int launch_tiled(sofie_hip_ctx *ctx, GemmArgs &g)
{
   constexpr int BN = 2 * TI * 32, BM = 2 * TJ * 32;
   if (g.M % BM == 0 && g.N % BN == 0 && g.K % BK == 0)
      return launch_tiled_impl<Mma, BK, NSETS, TI, TJ, OUT, B_KN, true>(ctx, g);
   return launch_tiled_impl<Mma, BK, NSETS, TI, TJ, OUT, B_KN, false>(ctx, g);
}

template <class Mma, int BK, int NST, int OUT, bool B_KN = false>
int launch_dma(sofie_hip_ctx *ctx, GemmArgs &g)
{
   constexpr size_t stage_bytes = (size_t)NST * 512 * BK;
   constexpr size_t epi_bytes = (size_t)8 * 32 * (128 * OutSize<OUT>::value + 16) + (size_t)2 * 256 * 4;
   constexpr size_t lds = stage_bytes > epi_bytes ? stage_bytes : epi_bytes;
   static_assert(lds <= 160 * 1024, "tile does not fit the 160 KB LDS");
   g.tiles_m = cdiv(g.M, 256);
   g.tiles_n = cdiv(g.N, 256);
   if constexpr (__is_same(Mma, MmaI8) && BK == 128 && SOFIE_GEMM16) {
      constexpr auto kern16 = k_gemm_dma16<OUT, B_KN>;
      SOFIE_LARGE_LDS(kern16);
      hipLaunchKernelGGL(kern16, dim3(g.tiles_m * g.tiles_n), dim3(512), lds, ctx->stream, g);
      return check_launch(ctx, "k_gemm_dma16");
   }
   // More tiles than compute units: one workgroup per compute unit walks over its tiles (see k_gemm_dma, LOOP).
   if constexpr (OutSize<OUT>::value <= 2) {
      const int nk = cdiv(g.K, BK);
      const int tiles = g.tiles_m * g.tiles_n;
      if (tiles > ctx->num_cus && g.K % (2 * BK) == 0) {
         constexpr size_t loop_lds = stage_bytes + (size_t)8 * EpilogueStaging<64 / (32 * OutSize<OUT>::value), OUT>::WAVE_BYTES + 8 * 1024;
         static_assert(loop_lds <= 160 * 1024, "stages and the epilogue's own blocks do not fit the 160 KB LDS");
         constexpr auto loop = k_gemm_dma<Mma, BK, NST, OUT, B_KN, true>;
         SOFIE_LARGE_LDS(loop);
         hipLaunchKernelGGL(loop, dim3(ctx->num_cus), dim3(512), loop_lds, ctx->stream, g);
         return check_launch(ctx, "k_gemm_dma_persistent");
      }
   }
   constexpr auto kern = k_gemm_dma<Mma, BK, NST, OUT, B_KN>;
   SOFIE_LARGE_LDS(kern);
   hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(512), lds, ctx->stream, g);
   return check_launch(ctx, "k_gemm_dma");
}

// Few rows of A (M <= 32: a quantised layer on a small batch) with B [N][K]: the product is a pass over B, bound by
// memory, and 64 x 64 tiles would give a handful of compute units all the work. A wavefront owns all rows of A (MT
// tiles of 16 rows, v_mfma_i32_16x16x64_i8) and 64 columns; B goes from global memory straight into the matrix
// instruction's operand registers: lane (j = lane % 16, kq = lane / 16) loads bytes k0 + 16 kq .. + 15 of column 16 q + j,
// which is its part of the operand of tile q as it stands, and the same bytes of its row of A. The grid is column
// blocks x slices of K; a wavefront takes a quarter of the slice in chunks of 64 k (consecutive chunks: the two halves
// of a 128-byte line are fetched one behind the other), three chunks of loads in flight while one is multiplied; the
// four wavefronts' sums meet in LDS and go to the scratch buffer [slice][M][ldp] that k_splitk_finish adds up and
// converts (integer sums: the result is that of the unsplit kernels bit for bit).
template <int MT>
__global__ void __launch_bounds__(256) k_qgemm_few_rows(GemmArgs g, int *partial, int ldp, int kslice)
{
   constexpr unsigned OUTSIDE = 0x80000000u;
   __shared__ int red[2 * MT * 4 * 4 * 64];
   const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int j = lane & 15, kq = lane >> 4;
   const int c0 = blockIdx.x * 64;
   const int k_begin = blockIdx.y * kslice + wave * (kslice >> 2);
   int k_end = k_begin + (kslice >> 2);
   if (k_end > g.K) k_end = g.K;
   const __amdgpu_buffer_rsrc_t ars = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t *>(g.A), 0, (int)((size_t)(g.M - 1) * g.lda + g.K), 0x00020000);
   const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t *>(g.B), 0, (int)((size_t)(g.N - 1) * g.ldb + g.K), 0x00020000);
   unsigned a_off[MT], b_off[4];
#pragma unroll
   for (int t = 0; t < MT; ++t) a_off[t] = t * 16 + j < g.M ? (unsigned)((t * 16 + j) * g.lda + 16 * kq) : OUTSIDE;
#pragma unroll
   for (int q = 0; q < 4; ++q) b_off[q] = c0 + 16 * q + j < g.N ? (unsigned)((c0 + 16 * q + j) * g.ldb + 16 * kq) : OUTSIDE;
   struct Chunk {
      v4i a[MT], b[4];
   };
   auto load = [&](Chunk &c, int k0) {
      const bool in = k0 + 16 * kq < k_end;     // K and the wavefronts' shares are multiples of 16: a lane's bytes are in or out together
#pragma unroll
      for (int t = 0; t < MT; ++t)
         c.a[t] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ars, in ? a_off[t] : OUTSIDE, k0, 0));
#pragma unroll
      for (int q = 0; q < 4; ++q)
         c.b[q] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(brs, in ? b_off[q] : OUTSIDE, k0, 0));
   };
   v4i acc[MT][4];
#pragma unroll
   for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[t][q] = v4i{0, 0, 0, 0};
   Chunk c0_, c1_, c2_, c3_;
   int k0 = k_begin;
   load(c0_, k0);
   load(c1_, k0 + 64);
   load(c2_, k0 + 128);
   for (; k0 < k_end; k0 += 64) {
      load(c3_, k0 + 192);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
         for (int t = 0; t < MT; ++t) acc[t][q] = __builtin_amdgcn_mfma_i32_16x16x64_i8(c0_.a[t], c0_.b[q], acc[t][q], 0, 0, 0);
      c0_ = c1_;
      c1_ = c2_;
      c2_ = c3_;
   }
   // wavefronts 2 and 3 hand their sums to 0 and 1, then 1 hands its to 0
   auto put = [&](int *dst) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
         for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[((t * 4 + q) * 4 + r) * 64 + lane] = acc[t][q][r];
   };
   auto add = [&](const int *src) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
         for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][q][r] += src[((t * 4 + q) * 4 + r) * 64 + lane];
   };
   constexpr int BLOCK = MT * 4 * 4 * 64;
   if (wave >= 2) put(red + (wave - 2) * BLOCK);
   __syncthreads();
   if (wave < 2) add(red + wave * BLOCK);
   __syncthreads();
   if (wave == 1) put(red);
   __syncthreads();
   if (wave != 0) return;
   add(red);
   // tile (t, q), register r: row t * 16 + kq * 4 + r, column c0 + 16 q + j
   int *const out = partial + (size_t)blockIdx.y * g.M * ldp;
#pragma unroll
   for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
         const int m = t * 16 + kq * 4 + r;
         if (m >= g.M) continue;
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            const int n = c0 + 16 * q + j;
            if (n < ldp) out[(size_t)m * ldp + n] = acc[t][q][r];
         }
      }
}

// The same pass over B for at most 16 rows of A and enough columns to give every compute unit a workgroup without
// cutting K across workgroups: a workgroup owns 16 columns and all of K, its eight wavefronts take an eighth of K
// each (up to eight chunks of 64 k in flight per wavefront: with K = 4096 everything the launch reads is requested
// before the first matrix instruction), their sums meet in LDS and the first wavefront converts and stores them. One
// launch and no partial sums in memory; integer sums, so the result is that of every other int8 kernel bit for bit.
template <int OUT>
__global__ void __launch_bounds__(512) k_qgemm_few_rows_whole(GemmArgs g, int kper)
{
   constexpr unsigned OUTSIDE = 0x80000000u;
   constexpr int NCH = 8;      // chunks whose loads are in flight together
   __shared__ int red[7 * 4 * 64];
   const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int j = lane & 15, kq = lane >> 4;
   const int c0 = blockIdx.x * 16;
   const int k_begin = wave * kper;
   int k_end = k_begin + kper;
   if (k_end > g.K) k_end = g.K;
   const __amdgpu_buffer_rsrc_t ars = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t *>(g.A), 0, (int)((size_t)(g.M - 1) * g.lda + g.K), 0x00020000);
   const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t *>(g.B), 0, (int)((size_t)(g.N - 1) * g.ldb + g.K), 0x00020000);
   const unsigned a_off = j < g.M ? (unsigned)(j * g.lda + 16 * kq) : OUTSIDE;
   const unsigned b_off = c0 + j < g.N ? (unsigned)((c0 + j) * g.ldb + 16 * kq) : OUTSIDE;
   v4i acc = {0, 0, 0, 0};
   for (int k0 = k_begin; k0 < k_end; k0 += 64 * NCH) {
      v4i a[NCH], b[NCH];
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
         const bool in = k0 + 64 * c + 16 * kq < k_end;      // K and the wavefronts' shares are multiples of 16
         b[c] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(brs, in ? b_off : OUTSIDE, k0 + 64 * c, 0));
         a[c] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ars, in ? a_off : OUTSIDE, k0 + 64 * c, 0));
      }
#pragma unroll
      for (int c = 0; c < NCH; ++c) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[c], b[c], acc, 0, 0, 0);
   }
   if (wave != 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) red[((wave - 1) * 4 + r) * 64 + lane] = acc[r];
   }
   __syncthreads();
   if (wave != 0) return;
#pragma unroll
   for (int w = 0; w < 7; ++w)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] += red[(w * 4 + r) * 64 + lane];
   // register r: row kq * 4 + r, column c0 + j
   const int n = c0 + j;
   if (n >= g.N) return;
   const float sc = g.scale ? g.scale[n] : 0.0f;
   const int bi = g.bias ? static_cast<const int *>(g.bias)[n] : 0;
   constexpr int ESZ = OutSize<OUT>::value;
#pragma unroll
   for (int r = 0; r < 4; ++r) {
      const int m = kq * 4 + r;
      if (m >= g.M) continue;
      const unsigned v = epilogue_value<true, OUT>(g, sc, bi, acc[r], 0.0f);
      unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + n) * ESZ;
      if constexpr (ESZ == 1) *out = (unsigned char)((int)fminf(__uint_as_float(v), 255.0f) - 128);
      else if constexpr (ESZ == 2) *reinterpret_cast<unsigned short *>(out) = (unsigned short)v;
      else *reinterpret_cast<unsigned *>(out) = v;
   }
}

// Slices of K so that about eight workgroups per compute unit exist, every wavefront with at least two chunks, and the
// partial sums a fraction of B's bytes.
template <int OUT>
int launch_few_rows(sofie_hip_ctx *ctx, GemmArgs &g)
{
   // enough columns for a workgroup of 16 columns on at least every second compute unit: one launch, K cut inside the
   // workgroups only (8 x 4096 x 4096: 5.7 against 9.3 us for the call; the second launch was a third of it)
   if (g.M <= 16 && cdiv(g.N, 16) * 2 >= ctx->num_cus) {
      const int kper = cdiv(cdiv(g.K, 8), 64) * 64;
      hipLaunchKernelGGL((k_qgemm_few_rows_whole<OUT>), dim3(cdiv(g.N, 16)), dim3(512), 0, ctx->stream, g, kper);
      return check_launch(ctx, "k_qgemm_few_rows_whole");
   }
   const int blocks = cdiv(g.N, 64);
   int splits = 8 * ctx->num_cus / blocks;
   if (splits > g.K / 512) splits = g.K / 512;
   if (splits > g.K / (16 * g.M)) splits = g.K / (16 * g.M);
   if (splits < 1) splits = 1;
   const int kslice = cdiv(cdiv(g.K, splits), 256) * 256;
   splits = cdiv(g.K, kslice);
   const int ldp = cdiv(g.N, 4) * 4;
   void *part = nullptr;
   if (int rc = workspace(ctx, (size_t)splits * g.M * ldp * sizeof(int), &part)) return rc;
   const dim3 grid(blocks, splits);
   if (g.M <= 16) hipLaunchKernelGGL(k_qgemm_few_rows<1>, grid, dim3(256), 0, ctx->stream, g, static_cast<int *>(part), ldp, kslice);
   else hipLaunchKernelGGL(k_qgemm_few_rows<2>, grid, dim3(256), 0, ctx->stream, g, static_cast<int *>(part), ldp, kslice);
   if (int rc = check_launch(ctx, "k_qgemm_few_rows")) return rc;
   const size_t threads = (size_t)g.M * (ldp / 4);
   hipLaunchKernelGGL((k_splitk_finish<OUT>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, ctx->stream, g,
                      static_cast<const int *>(part), splits, ldp);
   return check_launch(ctx, "k_splitk_finish");
}

// K cut into `splits` slices of `kslice` bytes (a multiple of BK): partial sums into the context's scratch
// buffer, then k_splitk_finish writes Y.
template <class Mma, int BK, int NSETS, int OUT>
int launch_split_k(sofie_hip_ctx *ctx, GemmArgs &g, int splits, int kslice, const GemmArgs *tail = nullptr,
                   int tail_out = SOFIE_OUT_S8)
{
   const int ldp = cdiv(g.N, 4) * 4;
   void *part = nullptr;
   if (int rc = workspace(ctx, (size_t)splits * g.M * ldp * sizeof(int), &part)) return rc;
   GemmArgs p = g;
   p.Y = part;
   p.ldy = ldp;
   p.scale = nullptr;
   p.bias = nullptr;
   p.relu = 0;
   p.vec_store = 1;
   p.splits = splits;
   p.kslice = kslice;
   p.ysplit = (long long)g.M * ldp * sizeof(int);
   if (int rc = launch_tiled<Mma, BK, NSETS, 2, 2, SOFIE_OUT_S32, false>(ctx, p)) return rc;
   const size_t threads = (size_t)g.M * (ldp / 4);
   const dim3 fgrid((unsigned)((threads + 255) / 256));
   if (tail) {
      if constexpr (OUT == SOFIE_OUT_S8) {
         const int *pp = static_cast<const int *>(part);
#define SOFIE_PAIR_LAUNCH(Q_)                                                                                              \
   do {                                                                                                                     \
      if (tail_out == SOFIE_OUT_F32)                                                                                        \
         hipLaunchKernelGGL((k_splitk_finish_pair<SOFIE_OUT_F32, Q_>), fgrid, dim3(256), 0, ctx->stream, g, pp, splits, ldp, *tail); \
      else                                                                                                                  \
         hipLaunchKernelGGL((k_splitk_finish_pair<SOFIE_OUT_S8, Q_>), fgrid, dim3(256), 0, ctx->stream, g, pp, splits, ldp, *tail);  \
   } while (0)
         switch (ldp / 4) {
         case 8: SOFIE_PAIR_LAUNCH(8); break;
         case 16: SOFIE_PAIR_LAUNCH(16); break;
         case 32: SOFIE_PAIR_LAUNCH(32); break;
         default: SOFIE_PAIR_LAUNCH(64); break;
         }
#undef SOFIE_PAIR_LAUNCH
         return check_launch(ctx, "k_splitk_finish_pair");
      }
   }
   hipLaunchKernelGGL((k_splitk_finish<OUT>), fgrid, dim3(256), 0, ctx->stream, g, static_cast<const int *>(part), splits, ldp);
   return check_launch(ctx, "k_splitk_finish");
}

template <bool IS_INT, int OUT>
int launch_simple(sofie_hip_ctx *ctx, GemmArgs &g, int transB)
{
   const size_t total = (size_t)g.M * g.N;
   hipLaunchKernelGGL((k_gemm_bytes_simple<IS_INT, OUT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                      ctx->stream, g, transB);
   return check_launch(ctx, "k_gemm_bytes_simple");
}

// Whether an int8 product with K-contiguous operands is cut into slices of K, and how: few 128 x 128 tiles and a long
// K (measured: pays from K = 8192 on; below that the second pass over the partial sums costs more).
bool split_k_plan(const sofie_hip_ctx *ctx, const GemmArgs &g, int &splits, int &kslice)
{
   const int tiles128 = cdiv(g.M, 128) * cdiv(g.N, 128);
   if (!(tiles128 * 2 <= ctx->num_cus && g.K >= 8192)) return false;
   splits = ctx->num_cus / tiles128;
   const int shortest = tiles128 * 8 <= ctx->num_cus ? 1024 : 2048;
   if (splits > g.K / shortest) splits = g.K / shortest;
   if (splits > 16) splits = 16;
   kslice = cdiv(cdiv(g.K, splits), 128) * 128;
   splits = cdiv(g.K, kslice);
   return splits > 1;
}

template <class Mma, int OUT>
int dispatch(sofie_hip_ctx *ctx, GemmArgs &g, int transB)
{
   constexpr bool IS_INT = __is_same(typename Mma::Acc, v16i);
   constexpr int ESZ = OutSize<OUT>::value;
   const bool a_ok = g.K % 16 == 0 && g.lda % 16 == 0 && aligned16(g.A);
   const bool b_nk_ok = transB && g.ldb % 16 == 0 && aligned16(g.B);
   const bool b_kn_ok = !transB && g.ldb % 4 == 0 && g.N % 4 == 0 && (reinterpret_cast<uintptr_t>(g.B) & 3u) == 0;
   g.vec_store = ((size_t)g.ldy * ESZ) % 16 == 0 && aligned16(g.Y);
   // K = 0 (an empty sum: the outputs are the epilogue of zero) takes the plain kernel, whose K loop runs zero times
   if (g.K == 0) return launch_simple<IS_INT, OUT>(ctx, g, transB);
   if constexpr (IS_INT && OUT != SOFIE_OUT_BF16) {
      if (transB && g.N <= 16 && a_ok && g.ldb % 16 == 0 && aligned16(g.B) && (size_t)g.M * 16 < ((size_t)1 << 40))
         return launch_skinny<OUT>(ctx, g);
   }
   if (!a_ok || !(b_nk_ok || b_kn_ok)) return launch_simple<IS_INT, OUT>(ctx, g, transB);
   if constexpr (IS_INT && OUT != SOFIE_OUT_BF16) {
      // a small batch on a layer of 2 MB or more: a pass over B with K in slices (8 x 4096 x 4096: 9.1 against 15.1 us; a
      // layer of 1 MB is faster on tiles in one launch: 6.0 against 7.2 us)
      if (transB && g.M <= 32 && g.N >= 64 && g.K >= 512 && (size_t)g.N * g.K >= ((size_t)2 << 20) &&
          (size_t)g.M * g.lda + g.K < (1u << 31) && (size_t)g.N * g.ldb + g.K < (1u << 31))
         return launch_few_rows<OUT>(ctx, g);
   }
   const bool big = (size_t)g.M * g.N >= (size_t)256 * 256 * 128 && g.M >= 256 && g.N >= 256;
   // 128 bytes of K per stage; int8 keeps two register sets in flight, fp8 (twice the
   // fragment registers) one.
   constexpr int BK = 128;
   constexpr int NSETS = IS_INT ? 2 : 1;
   if (transB) {
      // descriptor offsets are 32-bit: a 256-row panel plus K must stay below 2 GiB
      const bool fits = (size_t)256 * g.lda + g.K < (1u << 31) && (size_t)256 * g.ldb + g.K < (1u << 31);
      if (big && fits) return launch_dma<Mma, SOFIE_DMA_BK, SOFIE_DMA_NST, OUT>(ctx, g);
      if (big) return launch_tiled<Mma, BK, NSETS, 4, 4, OUT, false>(ctx, g);
      // a long K with few 128 x 128 tiles (a wide fully connected layer on a small batch x width):
      // 64 x 64 tiles put four times as many workgroups on the device
      if constexpr (IS_INT) {
         // ... and a longer one is cut into slices of K: 128 x 128 tiles write int32 partial sums per slice
         // (integer sums, so the result does not depend on the cut), a second kernel adds them and converts
         int splits = 1, kslice = 0;
         if (split_k_plan(ctx, g, splits, kslice)) return launch_split_k<Mma, BK, NSETS, OUT>(ctx, g, splits, kslice);
      }
      if (cdiv(g.M, 128) * cdiv(g.N, 128) * 2 <= ctx->num_cus && g.K >= 1024)
         return launch_tiled<Mma, BK, NSETS, 1, 1, OUT, false>(ctx, g);
      return launch_tiled<Mma, BK, NSETS, 2, 2, OUT, false>(ctx, g);
   }
   if (big && g.ldb % 16 == 0 && aligned16(g.B) && (size_t)256 * g.lda + g.K < (1u << 31) &&
       (size_t)(g.K + 128) * g.ldb < (1u << 31)) {
      // B [K,N] as it lies: rows of k go to LDS and the transposing LDS read builds the operand
      return launch_dma<Mma, SOFIE_DMA_BK, SOFIE_DMA_NST, OUT, true>(ctx, g);
   }
   if (big && g.K % 16 == 0 && (size_t)256 * g.lda + g.K < (1u << 31) && (size_t)257 * g.K < (1u << 31)) {
      // B [K,N] -> B^T [N,K] in the context's scratch buffer, then the K-contiguous kernel.
      // A caller that reuses B (weights) should transpose once and call with transB = 1.
      void *bt = nullptr;
      if (int rc = workspace(ctx, (size_t)g.N * g.K, &bt)) return rc;
      if (int rc = transpose_bytes(ctx, g.B, static_cast<unsigned char *>(bt), g.K, g.N, g.ldb, g.K)) return rc;
      g.B = static_cast<const uint8_t *>(bt);
      g.ldb = g.K;
      return launch_dma<Mma, SOFIE_DMA_BK, SOFIE_DMA_NST, OUT>(ctx, g);
   }
   if (big) return launch_tiled<Mma, BK, NSETS, 4, 4, OUT, true>(ctx, g);
   // Products of fewer tiles: a pass that transposes B in front (N * K bytes, into the context's scratch buffer, or once
   // per weight tensor when the caller promised constant weights) costs less than the byte transposes in every
   // workgroup's K loop, from one row of A upwards (2048^3: 20.2 against 23.7 us, 512 x 512 x 4096: 15.9 against 37.1,
   // 8 x 4096 x 4096: 28.7 against 45.3, 1 x 1024 x 1024: 9.4 against 16.1). A B^T of at most the fixed scratch array's
   // size, so that the no-allocation entry point takes the same path.
   if (g.K % 16 == 0 && (size_t)g.N * g.K <= (size_t)SOFIE_HIP_NOALLOC_SCRATCH_BYTES) {
      void *bt = nullptr;
      bool fresh = true;
      const int layout[] = {2, g.K, g.N, g.ldb};
      if (int rc = packed_weights(ctx, g.B, layout_key(layout, 4), (size_t)g.N * g.K, &bt, &fresh)) return rc;
      if (fresh)
         if (int rc = transpose_bytes(ctx, g.B, static_cast<unsigned char *>(bt), g.K, g.N, g.ldb, g.K)) return rc;
      g.B = static_cast<const uint8_t *>(bt);
      g.ldb = g.K;
      // a copy of its own (constant weights): every choice of the [N,K] case is open; a copy in the scratch buffer
      // leaves the kernels that need no scratch memory themselves
      if (bt != ctx->workspace && bt != ctx->static_scratch) return dispatch<Mma, OUT>(ctx, g, 1);
      if (cdiv(g.M, 128) * cdiv(g.N, 128) * 2 <= ctx->num_cus && g.K >= 1024)
         return launch_tiled<Mma, BK, NSETS, 1, 1, OUT, false>(ctx, g);
      return launch_tiled<Mma, BK, NSETS, 2, 2, OUT, false>(ctx, g);
   }
   return launch_tiled<Mma, BK, NSETS, 2, 2, OUT, true>(ctx, g);
}

}  // namespace

extern "C" {

int sofie_hip_qgemm_s8(sofie_hip_ctx *ctx, int transB, int M, int N, int K, const int8_t *A, int lda,
                       const int8_t *B, int ldb, const float *scale, const int32_t *bias, int zp_y,
                       int act, void *Y, int ldy, int out_kind)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, M >= 0 && N >= 0 && K >= 0, "negative dimension");
   if (M == 0 || N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, A && B && Y, "null operand");
   SOFIE_REQUIRE(ctx, lda >= K && ldb >= (transB ? K : N) && ldy >= N, "leading dimension too small");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   SOFIE_REQUIRE(ctx, out_kind == SOFIE_OUT_S8 || out_kind == SOFIE_OUT_F32 || out_kind == SOFIE_OUT_S32,
                 "output kind must be S8, F32 or S32");
   SOFIE_REQUIRE(ctx, scale || out_kind == SOFIE_OUT_S32, "scale is required for S8/F32 output");
   SOFIE_REQUIRE(ctx, zp_y >= -128 && zp_y <= 127, "zero-point out of int8 range");
   GemmArgs g{};
   g.A = reinterpret_cast<const uint8_t *>(A);
   g.B = reinterpret_cast<const uint8_t *>(B);
   g.Y = Y;
   g.scale = scale;
   g.bias = bias;
   g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldy = ldy;
   g.zp = zp_y;
   g.relu = act == SOFIE_ACT_RELU;
   g.lo = (g.relu && zp_y > -128) ? zp_y : -128;
   g.s = 1.0f;
   switch (out_kind) {
   case SOFIE_OUT_S8: return dispatch<MmaI8, SOFIE_OUT_S8>(ctx, g, transB);
   case SOFIE_OUT_F32: return dispatch<MmaI8, SOFIE_OUT_F32>(ctx, g, transB);
   default: return dispatch<MmaI8, SOFIE_OUT_S32>(ctx, g, transB);
   }
}

int sofie_hip_qgemm_s8_pair(sofie_hip_ctx *ctx, int M, int K, const int8_t *A, int lda, int N1, const int8_t *B1, int ldb1,
                            const float *scale1, const int32_t *bias1, int zp_mid, int act1, int8_t *mid, int ldmid,
                            int N2, const int8_t *B2, int ldb2, const float *scale2, const int32_t *bias2, int zp_y,
                            int act2, void *Y, int ldy, int out_kind)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, M >= 0 && K >= 0 && N1 >= 0 && N2 >= 0, "negative dimension");
   if (M == 0 || N2 == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, A && B1 && B2 && Y && scale1 && scale2 && mid, "null operand");
   SOFIE_REQUIRE(ctx, lda >= K && ldb1 >= K && ldmid >= N1 && ldb2 >= N1 && ldy >= N2, "leading dimension too small");
   SOFIE_REQUIRE(ctx, out_kind == SOFIE_OUT_S8 || out_kind == SOFIE_OUT_F32, "output kind must be S8 or F32");
   SOFIE_REQUIRE(ctx, (act1 == SOFIE_ACT_NONE || act1 == SOFIE_ACT_RELU) && (act2 == SOFIE_ACT_NONE || act2 == SOFIE_ACT_RELU),
                 "unknown activation");
   SOFIE_REQUIRE(ctx, zp_mid >= -128 && zp_mid <= 127 && zp_y >= -128 && zp_y <= 127, "zero-point out of int8 range");
   // One pass for both layers when the first one is cut into K slices anyway (its partial sums are added by a pass of
   // its own, which can as well multiply the finished row into a few more columns) and a row's quads of columns
   // are lanes of one wavefront.
   GemmArgs g{};
   g.A = reinterpret_cast<const uint8_t *>(A);
   g.B = reinterpret_cast<const uint8_t *>(B1);
   g.Y = mid;
   g.scale = scale1;
   g.bias = bias1;
   g.M = M; g.N = N1; g.K = K; g.lda = lda; g.ldb = ldb1; g.ldy = ldmid;
   g.zp = zp_mid;
   g.relu = act1 == SOFIE_ACT_RELU;
   g.lo = (g.relu && zp_mid > -128) ? zp_mid : -128;
   g.s = 1.0f;
   const int quads = N1 / 4;
   const bool lanes_ok = N1 % 4 == 0 && quads >= 8 && quads <= 64 && (quads & (quads - 1)) == 0;
   const bool operands_ok = K % 16 == 0 && lda % 16 == 0 && aligned16(A) && ldb1 % 16 == 0 && aligned16(B1) && ldb2 % 4 == 0 &&
                            (reinterpret_cast<uintptr_t>(B2) & 3u) == 0;
   int splits = 1, kslice = 0;
   if (N2 <= 8 && lanes_ok && operands_ok && N1 > 16 && split_k_plan(ctx, g, splits, kslice) &&
       !((size_t)M * N1 >= (size_t)256 * 256 * 128 && M >= 256 && N1 >= 256)) {
      GemmArgs t{};
      t.B = reinterpret_cast<const uint8_t *>(B2);
      t.Y = Y;
      t.scale = scale2;
      t.bias = bias2;
      t.M = M; t.N = N2; t.K = N1; t.ldb = ldb2; t.ldy = ldy;
      t.zp = zp_y;
      t.relu = act2 == SOFIE_ACT_RELU;
      t.lo = (t.relu && zp_y > -128) ? zp_y : -128;
      t.s = 1.0f;
      return launch_split_k<MmaI8, 128, 2, SOFIE_OUT_S8>(ctx, g, splits, kslice, &t, out_kind);
   }
   // otherwise the two layers one after the other, the first one's result in the caller's scratch tensor
   if (int rc = sofie_hip_qgemm_s8(ctx, 1, M, N1, K, A, lda, B1, ldb1, scale1, bias1, zp_mid, act1, mid, ldmid, SOFIE_OUT_S8))
      return rc;
   return sofie_hip_qgemm_s8(ctx, 1, M, N2, N1, mid, ldmid, B2, ldb2, scale2, bias2, zp_y, act2, Y, ldy, out_kind);
}

int sofie_hip_qgemm_s8_noalloc(sofie_hip_ctx *ctx, int transB, int M, int N, int K, const int8_t *A, int lda,
                               const int8_t *B, int ldb, const float *scale, const int32_t *bias, int zp_y,
                               int act, void *Y, int ldy, int out_kind)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   // Same kernels and the same choice among them as sofie_hip_qgemm_s8; the two paths that need memory beyond the
   // operands (partial sums of a K cut into slices, the transposed copy of a B [K,N] whose rows are not 16-byte
   // aligned) take it from the fixed array instead of the context's growable buffer.
   // Every context of a device shares the one array: the call takes its turn behind the one that used it last.
   scratch_turn_begin(ctx);
   ctx->no_alloc = true;
   const int rc = sofie_hip_qgemm_s8(ctx, transB, M, N, K, A, lda, B, ldb, scale, bias, zp_y, act, Y, ldy, out_kind);
   ctx->no_alloc = false;
   scratch_turn_end(ctx);
   return rc;
}

int sofie_hip_transpose_bytes(sofie_hip_ctx *ctx, const void *src, void *dst, int rows, int cols, int ld_src,
                               int ld_dst)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, rows >= 0 && cols >= 0, "negative dimension");
   if (rows == 0 || cols == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, src && dst && src != dst, "null or aliased operand");
   SOFIE_REQUIRE(ctx, ld_src >= cols && ld_dst >= rows, "leading dimension too small");
   SOFIE_REQUIRE(ctx, rows % 16 == 0 && cols % 4 == 0 && ld_src % 4 == 0 && ld_dst % 16 == 0 &&
                         (reinterpret_cast<uintptr_t>(src) & 3u) == 0 && aligned16(dst),
                 "needs rows % 16 == 0, cols % 4 == 0 and matching alignment");
   return transpose_bytes(ctx, static_cast<const unsigned char *>(src), static_cast<unsigned char *>(dst), rows, cols,
                          ld_src, ld_dst);
}

int sofie_hip_gemm_fp8(sofie_hip_ctx *ctx, int transB, int M, int N, int K, const uint8_t *A, int lda,
                       const uint8_t *B, int ldb, float scale_a, float scale_b, const float *bias, void *Y,
                       int ldy, int out_kind)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, M >= 0 && N >= 0 && K >= 0, "negative dimension");
   if (M == 0 || N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, A && B && Y, "null operand");
   SOFIE_REQUIRE(ctx, lda >= K && ldb >= (transB ? K : N) && ldy >= N, "leading dimension too small");
   SOFIE_REQUIRE(ctx, out_kind == SOFIE_OUT_BF16 || out_kind == SOFIE_OUT_F32, "output kind must be BF16 or F32");
   GemmArgs g{};
   g.A = A; g.B = B; g.Y = Y;
   g.scale = nullptr;
   g.bias = bias;
   g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldy = ldy;
   g.s = scale_a * scale_b;
   if (out_kind == SOFIE_OUT_BF16) return dispatch<MmaF8, SOFIE_OUT_BF16>(ctx, g, transB);
   return dispatch<MmaF8, SOFIE_OUT_F32>(ctx, g, transB);
}

}  // extern "C"
