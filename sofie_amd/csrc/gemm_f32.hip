// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32) with a fused
// alpha / beta*bias / ReLU epilogue.
//
// 256 threads = 4 wavefronts (2x2), each owning TI x TJ tiles of 32x32. Operands are staged
// in LDS k-major ([k][row]) so that the one-float-per-lane MFMA operand read is a conflict-free
// ds_read_b32 for either storage order of A and B; the accumulator layout puts 32 consecutive
// output columns in 32 consecutive lanes, so results are stored straight from registers as
// 128-byte row segments. Loads are guarded scalar loads: no alignment or size restrictions.
// Roofline: MFMA fp32 (256 flop/clk/CU); each K-step of 16 issues 8*TI*TJ MFMAs of 64 cycles
// per wavefront against 16 scalar loads per thread.
#include <cstdint>
#include <type_traits>

#include "common.h"
#include "gemm_tile.h"

using namespace sofie;

namespace {

struct GemmF32Args {
   const float *A, *B, *bias;
   float *Y;
   int M, N, K, lda, ldb, ldy;
   int transA, transB;
   float alpha, beta;
   int bias_kind, relu;
   // stacked products (blockIdx.z + z0 = index of the product, row-major over the n_lead leading dimensions):
   // element strides of A and B along each leading dimension (0 where the operand is broadcast), Y is dense
   int n_lead, z0;
   int lead[SOFIE_GEMM_MAX_LEAD];
   long long sa[SOFIE_GEMM_MAX_LEAD], sb[SOFIE_GEMM_MAX_LEAD];
   long long stride_y;
   // k_gemm_f32_dma with K in slices (gridDim.y > 1): a slice's raw sums go to partial [slice][M][N]
   float *partial;
};

constexpr int BK = 16;

// Stage a [rows x BK] block of a matrix into LDS as dst[k][row].
// k_major_src: the source is stored [K][rows] (row index contiguous); else [rows][K].
template <int ROWS, int LD>
__device__ __forceinline__ void fetch(float (&reg)[ROWS * BK / 256], const float *src, int ld, bool k_major_src,
                                      int row0, int k0, int nrows, int K, int tid)
{
#pragma unroll
   for (int i = 0; i < ROWS * BK / 256; ++i) {
      const int e = i * 256 + tid;
      int r, k;
      if (k_major_src) { k = e / ROWS; r = e % ROWS; }
      else { r = e / BK; k = e % BK; }
      const int gr = row0 + r, gk = k0 + k;
      float v = 0.0f;
      if (gr < nrows && gk < K) v = k_major_src ? src[(size_t)gk * ld + gr] : src[(size_t)gr * ld + gk];
      reg[i] = v;
   }
}

template <int ROWS, int LD>
__device__ __forceinline__ void stash(const float (&reg)[ROWS * BK / 256], float *dst, bool k_major_src, int tid)
{
#pragma unroll
   for (int i = 0; i < ROWS * BK / 256; ++i) {
      const int e = i * 256 + tid;
      int r, k;
      if (k_major_src) { k = e / ROWS; r = e % ROWS; }
      else { r = e / BK; k = e % BK; }
      dst[k * LD + r] = reg[i];
   }
}

template <int TI, int TJ>
__global__ void __launch_bounds__(256) k_gemm_f32(GemmF32Args g)
{
   constexpr int BM = 2 * TI * 32, BN = 2 * TJ * 32;
   constexpr int LDA = BM + 4, LDB = BN + 4;
   __shared__ float sA[2][BK * LDA];
   __shared__ float sB[2][BK * LDB];

   const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
   const int wm = wave >> 1, wn = wave & 1;
   const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
   if (g.n_lead > 0) {
      // this workgroup's product of the stack: its position along every leading dimension, last dimension fastest
      long long rem = (long long)blockIdx.z + g.z0, oa = 0, ob = 0;
      const long long index = rem;
      for (int d = g.n_lead - 1; d >= 0; --d) {
         const long long pos = rem % g.lead[d];
         rem /= g.lead[d];
         oa += pos * g.sa[d];
         ob += pos * g.sb[d];
      }
      g.A += oa;
      g.B += ob;
      g.Y += index * g.stride_y;
   }

   float ra[BM * BK / 256], rb[BN * BK / 256];
   v16f acc[TI][TJ];
#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
         for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

   const bool a_kmajor = g.transA != 0;   // A stored [K][M]
   const bool b_kmajor = g.transB == 0;   // B stored [K][N]
   const int nk = (g.K + BK - 1) / BK;

   fetch<BM, LDA>(ra, g.A, g.lda, a_kmajor, m0, 0, g.M, g.K, tid);
   fetch<BN, LDB>(rb, g.B, g.ldb, b_kmajor, n0, 0, g.N, g.K, tid);
   stash<BM, LDA>(ra, sA[0], a_kmajor, tid);
   stash<BN, LDB>(rb, sB[0], b_kmajor, tid);
   __syncthreads();

   const int fr = lane & 31, fk = lane >> 5;
   for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < nk) {
         fetch<BM, LDA>(ra, g.A, g.lda, a_kmajor, m0, (kt + 1) * BK, g.M, g.K, tid);
         fetch<BN, LDB>(rb, g.B, g.ldb, b_kmajor, n0, (kt + 1) * BK, g.N, g.K, tid);
      }
      const float *a = sA[cur] + fk * LDA + wm * TI * 32 + fr;
      const float *b = sB[cur] + fk * LDB + wn * TJ * 32 + fr;
#pragma unroll
      for (int s = 0; s < BK / 2; ++s) {
         float fa[TI], fb[TJ];
#pragma unroll
         for (int i = 0; i < TI; ++i) fa[i] = a[2 * s * LDA + i * 32];
#pragma unroll
         for (int j = 0; j < TJ; ++j) fb[j] = b[2 * s * LDB + j * 32];
#pragma unroll
         for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j)
               acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      if (kt + 1 < nk) {
         stash<BM, LDA>(ra, sA[cur ^ 1], a_kmajor, tid);
         stash<BN, LDB>(rb, sB[cur ^ 1], b_kmajor, tid);
      }
      __syncthreads();
   }

#pragma unroll
   for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
         const int n = n0 + wn * TJ * 32 + j * 32 + fr;
         if (n >= g.N) continue;
         float brow = 0.0f;
         if (g.bias_kind == SOFIE_BIAS_ROW) brow = __fmul_rn(g.beta, g.bias[n]);
#pragma unroll
         for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * TI * 32 + i * 32 + (r >> 2) * 8 + fk * 4 + (r & 3);
            if (m >= g.M) continue;
            float v = __fmul_rn(g.alpha, acc[i][j][r]);
            if (g.bias_kind == SOFIE_BIAS_ROW) v = __fadd_rn(v, brow);
            else if (g.bias_kind == SOFIE_BIAS_FULL) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[(size_t)m * g.ldy + n]));
            else if (g.bias_kind == SOFIE_BIAS_COL) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[m]));
            if (g.relu) v = v > 0.0f ? v : 0.0f;
            g.Y[(size_t)m * g.ldy + n] = v;
         }
      }
}

// The same product for operands that allow it (A [M][K] row-major, K a multiple of 32, 16-byte aligned rows), with
// both operand tiles travelling global memory -> LDS without registers (buffer_load_dwordx4 ... lds), two stages of
// 32 k, under the matrix loop of the stage before. Tile of 64 T x 64 T (T = 2: 128 x 128, two workgroups per CU; T = 1
// for products of few tiles: 64 x 64, four per CU), 4 wavefronts of T x T tiles of 32 x 32.
//   * An operand whose rows run along K (A; B given [N][K]) is staged as rows of 32 floats (8 chunks of 16 bytes) with
//     chunk c of row r in slot c ^ ((r >> 1) & 7): a lane reads 4 consecutive k of its row with one 16-byte read (lanes
//     0-31: k = 8s .. 8s+3, lanes 32-63: k = 8s+4 .. 8s+7, which is the pairing of four matrix instructions), and the 16
//     lanes the LDS serves together fall on 16 different slots of 256 bytes. The swizzle costs nothing: a lane of the
//     request asks for the chunk that belongs into its slot.
//   * B given [K][N] is staged as it is, rows of k with the tile's columns, and read 4 bytes per lane.
// A lane's read addresses do not depend on the K step (the stage is an immediate offset: the loop is unrolled over the
// two stages), so the loop holds LDS reads and matrix instructions and no vector arithmetic, which would take issue
// cycles from the matrix instructions. Rows behind M (or N) lie outside the tile's descriptor and arrive as zeros;
// outputs go through a descriptor too (columns behind N get an offset outside it and are dropped).
template <bool B_KMAJOR, int T>
__global__ void __launch_bounds__(256, T == 2 ? 2 : 4) k_gemm_f32_dma(GemmF32Args g)
{
   constexpr int BM = 64 * T, BN = 64 * T, BKD = 32;
   constexpr int STAGE = (BM + BN) * BKD;               // floats of one stage: the A tile, then the B tile
   constexpr unsigned OUTSIDE = 0x80000000u;            // an offset no descriptor of this kernel reaches
   extern __shared__ __align__(16) unsigned char smem_raw[];
   float *const lds = reinterpret_cast<float *>(smem_raw);
   const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem_raw;
   const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int wm = wave >> 1, wn = wave & 1;
   const int fr = lane & 31, fk = lane >> 5;
   // tiles in groups of 4 rows of tiles, so that the workgroups in flight share rows of A and columns of B in an L2
   int tm, tn;
   {
      const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
      // workgroups are dealt to the 8 XCDs in turn: renumbered so that an XCD (an L2) works on consecutive tiles
      int pid = blockIdx.x;
      {
         const int tiles = tiles_m * tiles_n, xcd = pid & 7, base = tiles >> 3, rem = tiles & 7;
         pid = (pid >> 3) + xcd * base + (xcd < rem ? xcd : rem);
      }
      const int width = 4 * tiles_n, group = pid / width, first = group * 4;
      const int gsize = tiles_m - first < 4 ? tiles_m - first : 4;
      tm = first + (pid % width) % gsize;
      tn = (pid % width) / gsize;
   }
   const int m0 = tm * BM, n0 = tn * BN;
   const int rows_a = g.M - m0 < BM ? g.M - m0 : BM, rows_b = g.N - n0 < BN ? g.N - n0 : BN;
   // K in slices (few tiles, long K): this workgroup's steps of 32 k, raw sums into its plane of the scratch buffer
   int kt_begin = 0, kt_end = g.K / BKD;
   if (gridDim.y > 1) {
      const int per = (kt_end + (int)gridDim.y - 1) / (int)gridDim.y;
      kt_begin = (int)blockIdx.y * per;
      kt_end = kt_end < kt_begin + per ? kt_end : kt_begin + per;
      g.Y = g.partial + (size_t)blockIdx.y * g.M * g.N;
      g.ldy = g.N;
      g.alpha = 1.0f;
      g.bias_kind = SOFIE_BIAS_NONE;
      g.relu = 0;
   }
   const rsrc_t ars = make_rsrc(g.A + (size_t)m0 * g.lda, (unsigned)((size_t)rows_a * g.lda * 4));
   const rsrc_t brs = B_KMAJOR ? make_rsrc(g.B, (unsigned)((size_t)g.K * g.ldb * 4))
                               : make_rsrc(g.B + (size_t)n0 * g.ldb, (unsigned)((size_t)rows_b * g.ldb * 4));
   // requests: 16 bytes per lane, 256 lanes per request. Row-major operand: lane -> (row tid/8 [+ 32 per request],
   // slot tid%8), it fetches chunk slot ^ swizzle(row); the swizzle is the same for every request of the lane.
   constexpr int NRQ = 2 * T;                           // requests per operand tile and stage (4 KB each)
   const int rq_row = tid >> 3, rq_slot = tid & 7;
   const unsigned rq_a = (unsigned)((rq_row * g.lda + ((rq_slot ^ ((rq_row >> 1) & 7)) << 2)) * 4);
   unsigned rq_b;
   if constexpr (B_KMAJOR) {
      // lane -> (k tid/(BN/4) [+ 1024/BN per request], columns 4*(tid%(BN/4)) .. +3); columns behind N ask for nothing
      const int col = n0 + (tid % (BN / 4)) * 4;
      rq_b = col < g.N ? (unsigned)(((tid / (BN / 4)) * g.ldb + col) * 4) : OUTSIDE;
   } else {
      rq_b = (unsigned)((rq_row * g.ldb + ((rq_slot ^ ((rq_row >> 1) & 7)) << 2)) * 4);
   }
   const unsigned step_a = (unsigned)(32 * g.lda * 4), step_b = (unsigned)((B_KMAJOR ? 1024 / BN : 32) * g.ldb * 4);
   auto request = [&](int kt, int stage) {
      const unsigned dst = lds0 + (unsigned)(stage * STAGE * 4) + (unsigned)(wave * 1024);
      const unsigned ka = (unsigned)(kt * BKD * 4), kb = B_KMAJOR ? (unsigned)kt * BKD * (unsigned)g.ldb * 4u : ka;
#pragma unroll
      for (int u = 0; u < NRQ; ++u) dma16(ars, dst + u * 4096, (int)rq_a, (int)(ka + u * step_a));
#pragma unroll
      for (int u = 0; u < NRQ; ++u) dma16(brs, dst + BM * BKD * 4 + u * 4096, (int)rq_b, (int)(kb + u * step_b));
   };
   // read addresses of the lane's fragments in stage 0 (floats from the start of the LDS block)
   int ra[T][4], rb[T][4];
#pragma unroll
   for (int i = 0; i < T; ++i) {
      const int row = wm * 32 * T + i * 32 + fr;
#pragma unroll
      for (int s = 0; s < 4; ++s) ra[i][s] = row * BKD + (((2 * s + fk) ^ ((row >> 1) & 7)) << 2);
   }
#pragma unroll
   for (int j = 0; j < T; ++j) {
      const int row = wn * 32 * T + j * 32 + fr;
#pragma unroll
      for (int s = 0; s < 4; ++s)
         rb[j][s] = BM * BKD + (B_KMAJOR ? (8 * s + 4 * fk) * BN + row : row * BKD + (((2 * s + fk) ^ ((row >> 1) & 7)) << 2));
   }
   v16f acc[T][T];
#pragma unroll
   for (int i = 0; i < T; ++i)
#pragma unroll
      for (int j = 0; j < T; ++j)
#pragma unroll
         for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

   auto multiply = [&](auto stage_c) {
      constexpr int OFF = decltype(stage_c)::value * STAGE;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
         v4f fa[T], fb[T];
#pragma unroll
         for (int i = 0; i < T; ++i) fa[i] = *reinterpret_cast<const v4f *>(lds + OFF + ra[i][s]);
#pragma unroll
         for (int j = 0; j < T; ++j) {
            if constexpr (B_KMAJOR) {
#pragma unroll
               for (int e = 0; e < 4; ++e) fb[j][e] = lds[OFF + rb[j][s] + e * BN];
            } else {
               fb[j] = *reinterpret_cast<const v4f *>(lds + OFF + rb[j][s]);
            }
         }
#pragma unroll
         for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < T; ++i)
#pragma unroll
               for (int j = 0; j < T; ++j)
                  acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][e], fb[j][e], acc[i][j], 0, 0, 0);
      }
   };
   const int nk = kt_end;
   if (kt_begin < nk) request(kt_begin, 0);
   wait_vmcnt<0>();
   __syncthreads();
   for (int kt = kt_begin; kt < nk; kt += 2) {
      if (kt + 1 < nk) request(kt + 1, 1);
      multiply(std::integral_constant<int, 0>{});
      wait_vmcnt<0>();
      __syncthreads();        // stage 1 has landed, everybody is done with stage 0
      if (kt + 1 >= nk) break;
      if (kt + 2 < nk) request(kt + 2, 0);
      multiply(std::integral_constant<int, 1>{});
      wait_vmcnt<0>();
      __syncthreads();
   }

   // epilogue: v = alpha * acc (+ beta * bias) (ReLU); a lane holds column n = fr of 16 rows per tile
   const rsrc_t yrs = make_rsrc(g.Y + (size_t)m0 * g.ldy, (unsigned)((size_t)rows_a * g.ldy * 4));
   const __amdgpu_buffer_rsrc_t col_bias = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(g.bias) + (g.bias_kind == SOFIE_BIAS_COL ? m0 : 0), 0, g.bias_kind == SOFIE_BIAS_COL ? rows_a * 4 : 0, 0x00020000);
   const unsigned ldy4 = (unsigned)g.ldy * 4u;
#pragma unroll
   for (int j = 0; j < T; ++j) {
      const int n = n0 + wn * 32 * T + j * 32 + fr;
      const float brow = g.bias_kind == SOFIE_BIAS_ROW && n < g.N ? __fmul_rn(g.beta, g.bias[n]) : 0.0f;
      const unsigned voff = n < g.N ? (unsigned)(n * 4) + (unsigned)fk * 4u * ldy4 : OUTSIDE;
#pragma unroll
      for (int i = 0; i < T; ++i)
#pragma unroll
         for (int r = 0; r < 16; ++r) {
            const int m_uniform = wm * 32 * T + i * 32 + (r >> 2) * 8 + (r & 3);      // + 4 * fk in the lane's offset
            float v = __fmul_rn(g.alpha, acc[i][j][r]);
            if (g.bias_kind == SOFIE_BIAS_ROW) v = __fadd_rn(v, brow);
            else if (g.bias_kind == SOFIE_BIAS_COL)
               v = __fadd_rn(v, __fmul_rn(g.beta, __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(col_bias, fk * 16, m_uniform * 4, 0))));
            if (g.relu) v = v > 0.0f ? v : 0.0f;
            store4_buf(yrs, v, voff, (unsigned)m_uniform * ldy4);
         }
   }
}

// Few rows of A (M <= 64: a layer on a small batch): the product is a pass over B, bound by memory, and tiles of
// 64 x 64 outputs would leave most of the device idle. Here a wavefront owns all rows of A (MT tiles of T = 16 rows,
// v_mfma_f32_16x16x4_f32) and 4 T = 64 columns: its accumulators are MT x 4 tiles of T x T (rows of A x columns), and B
// goes from global memory straight into the matrix instructions' operand registers, 16 bytes per lane, with no LDS on
// the way. With lane = (j = lane % T, kg = lane / T):
//   * B [K][N]: a lane loads columns 4 j .. 4 j + 3 of row k0 + 4 kg + u (a wavefront's load: 4 rows of 256
//     contiguous bytes); element e of the four feeds the tile of columns 4 j + e, so a lane ends up with 4 consecutive
//     columns of a row.
//   * B [N][K]: a lane loads k0 + 4 kg .. + 3 of column T q + j; element u feeds instruction u of tile q.
// A lane's 4 consecutive k of its row of A arrive the same way (k0 + 4 kg .. + 3, one instruction per element). The
// grid is column blocks x slices of K; the four wavefronts of a workgroup take the slice's chunks of 16 k in turn,
// each with the loads of the next three chunks in flight while it multiplies, and add their accumulators up through
// LDS. With more than one slice the sums go to a scratch buffer [slice][M][N] and k_gemm_f32_skinny_finish adds them
// in slice order and applies alpha, bias and ReLU (a fixed order: the result does not depend on timing). Rows behind
// M, columns behind N and k behind the slice get offsets outside the buffer descriptors and arrive as zeros.
template <int T> struct SkinnyTile;
template <> struct SkinnyTile<16> {
   typedef v4f Acc;
   static constexpr int NR = 4;
   static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
   static __device__ __forceinline__ int row(int r, int kg) { return kg * 4 + r; }
};

template <bool B_NK, int T, int MT>
__global__ void __launch_bounds__(256) k_gemm_f32_skinny(GemmF32Args g, float *partial, int kslice, int splits)
{
   typedef SkinnyTile<T> Tile;
   constexpr int NR = Tile::NR;
   constexpr int CHUNK = 256 / T;                      // k per chunk: 4 per lane, 64 / T groups of lanes
   constexpr int COLS = 4 * T;                         // columns of a workgroup
   constexpr unsigned OUTSIDE = 0x80000000u;
   __shared__ float red[2 * MT * 4 * NR * 64];
   const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
   const int fr = lane % T, fk = lane / T;
   const int c0 = blockIdx.x * COLS;
   const int k_begin = blockIdx.y * kslice;
   const int k_end = g.K < k_begin + kslice ? g.K : k_begin + kslice;
   const __amdgpu_buffer_rsrc_t ars = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(g.A), 0, (int)(((size_t)(g.M - 1) * g.lda + g.K) * 4), 0x00020000);
   const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(g.B), 0, (int)((B_NK ? (size_t)(g.N - 1) * g.ldb + g.K : (size_t)(g.K - 1) * g.ldb + g.N) * 4), 0x00020000);
   unsigned a_off[MT], b_off[B_NK ? 4 : 1];
#pragma unroll
   for (int t = 0; t < MT; ++t) a_off[t] = t * T + fr < g.M ? (unsigned)(((t * T + fr) * g.lda + 4 * fk) * 4) : OUTSIDE;
   if constexpr (B_NK) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
         const int n = c0 + T * q + fr;
         b_off[q] = n < g.N ? (unsigned)((n * g.ldb + 4 * fk) * 4) : OUTSIDE;
      }
   } else {
      const int n = c0 + 4 * fr;
      b_off[0] = n < g.N ? (unsigned)((4 * fk * g.ldb + n) * 4) : OUTSIDE;
   }
   struct Chunk {
      v4f a[MT], b[4];
   };
   auto load = [&](Chunk &c, int k0) {
      // a lane's four k lie inside the slice together or not at all (K and the slices are multiples of 4)
      const bool in = k0 + 4 * fk < k_end;
#pragma unroll
      for (int t = 0; t < MT; ++t)
         c.a[t] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(ars, in ? a_off[t] : OUTSIDE, k0 * 4, 0));
#pragma unroll
      for (int q = 0; q < 4; ++q) {
         if constexpr (B_NK)
            c.b[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(brs, in ? b_off[q] : OUTSIDE, k0 * 4, 0));
         else
            c.b[q] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(brs, in ? b_off[0] : OUTSIDE, (k0 + q) * g.ldb * 4, 0));
      }
   };
   typename Tile::Acc acc[MT][4];
#pragma unroll
   for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
         for (int r = 0; r < NR; ++r) acc[t][q][r] = 0.0f;
   auto multiply = [&](const Chunk &c) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
         for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
               // B [K][N]: load u is row k0 + 4 kg + u, its element q a column; B [N][K]: load q is a group of columns,
               // its element u a k
               const float b = B_NK ? c.b[q][u] : c.b[u][q];
               acc[t][q] = Tile::mma(c.a[t][u], b, acc[t][q]);
            }
   };
   // chunks wave, wave + 4, ... of the slice; three chunks ahead are in flight while one is multiplied (loads behind
   // the slice's end ask for nothing)
   constexpr int STEP = 4 * CHUNK;
   Chunk c0_, c1_, c2_, c3_;
   int k0 = k_begin + wave * CHUNK;
   load(c0_, k0);
   load(c1_, k0 + STEP);
   load(c2_, k0 + 2 * STEP);
   for (; k0 < k_end; k0 += STEP) {
      load(c3_, k0 + 3 * STEP);
      multiply(c0_);
      c0_ = c1_;
      c1_ = c2_;
      c2_ = c3_;
   }
   // the four wavefronts' sums meet in LDS: wavefronts 2 and 3 hand theirs to 0 and 1, then 1 hands its to 0
   // ((w0 + w2) + (w1 + w3): a fixed order)
   auto put = [&](float *dst) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
         for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < NR; ++r) dst[((t * 4 + q) * NR + r) * 64 + lane] = acc[t][q][r];
   };
   auto add = [&](const float *src) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
         for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < NR; ++r) acc[t][q][r] = __fadd_rn(acc[t][q][r], src[((t * 4 + q) * NR + r) * 64 + lane]);
   };
   constexpr int BLOCK = MT * 4 * NR * 64;
   if (wave >= 2) put(red + (wave - 2) * BLOCK);
   __syncthreads();
   if (wave < 2) add(red + wave * BLOCK);
   __syncthreads();
   if (wave == 1) put(red);
   __syncthreads();
   if (wave == 0) add(red);
   if (wave != 0) return;
   // tile (t, q), register r of a lane: row t * T + Tile::row(r, kg); column c0 + 4 j + q (B [K][N]) or c0 + T q + j
   const bool last = splits == 1;
   float *const out = last ? g.Y : partial + (size_t)blockIdx.y * g.M * g.N;
   const int ldo = last ? g.ldy : g.N;
   const bool vec_out = !last || (g.ldy % 4 == 0 && (reinterpret_cast<uintptr_t>(g.Y) & 15u) == 0);   // rows of whole 16-byte chunks
   auto finish = [&](float v, int m, int n) {
      if (!last) return v;
      v = __fmul_rn(g.alpha, v);
      if (g.bias_kind == SOFIE_BIAS_ROW) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[n]));
      else if (g.bias_kind == SOFIE_BIAS_FULL) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[(size_t)m * g.ldy + n]));
      else if (g.bias_kind == SOFIE_BIAS_COL) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[m]));
      if (g.relu) v = v > 0.0f ? v : 0.0f;
      return v;
   };
#pragma unroll
   for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < NR; ++r) {
         const int m = t * T + Tile::row(r, fk);
         if (m >= g.M) continue;
         if constexpr (B_NK) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
               const int n = c0 + T * q + fr;
               if (n < g.N) out[(size_t)m * ldo + n] = finish(acc[t][q][r], m, n);
            }
         } else {
            const int n = c0 + 4 * fr;     // N is a multiple of 4 on this path: the four columns are inside together
            if (n < g.N) {
               float *o = out + (size_t)m * ldo + n;
               const v4f v = {finish(acc[t][0][r], m, n), finish(acc[t][1][r], m, n + 1), finish(acc[t][2][r], m, n + 2),
                              finish(acc[t][3][r], m, n + 3)};
               if (vec_out) *reinterpret_cast<v4f *>(o) = v;
               else {
#pragma unroll
                  for (int q = 0; q < 4; ++q) o[q] = v[q];
               }
            }
         }
      }
}

// Sum of the K slices' partial products in slice order, then alpha, bias and ReLU: one thread per output. The loads of
// eight slices are in flight together; the additions keep the slices' order.
__global__ void __launch_bounds__(256) k_gemm_f32_skinny_finish(GemmF32Args g, const float *__restrict__ partial, int splits)
{
   const int idx = blockIdx.x * 256 + threadIdx.x;
   if (idx >= g.M * g.N) return;
   const int m = idx / g.N, n = idx - m * g.N;
   const size_t plane = (size_t)g.M * g.N;
   float v = 0.0f;
   int s = 0;
   for (; s + 8 <= splits; s += 8) {
      float p[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = partial[(size_t)(s + i) * plane + idx];
#pragma unroll
      for (int i = 0; i < 8; ++i) v = __fadd_rn(v, p[i]);
   }
   for (; s < splits; ++s) v = __fadd_rn(v, partial[(size_t)s * plane + idx]);
   v = __fmul_rn(g.alpha, v);
   if (g.bias_kind == SOFIE_BIAS_ROW) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[n]));
   else if (g.bias_kind == SOFIE_BIAS_FULL) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[(size_t)m * g.ldy + n]));
   else if (g.bias_kind == SOFIE_BIAS_COL) v = __fadd_rn(v, __fmul_rn(g.beta, g.bias[m]));
   if (g.relu) v = v > 0.0f ? v : 0.0f;
   g.Y[(size_t)m * g.ldy + n] = v;
}

// M <= 64 rows on k_gemm_f32_skinny. Slices of K so that about eight workgroups per compute unit exist, each wavefront
// with at least four chunks, and so that the partial sums stay below a quarter of B's bytes once they are more than a
// few megabytes (below that the launch is latency, not traffic).
template <bool B_NK, int T, int MT>
int launch_skinny_as(sofie_hip_ctx *ctx, GemmF32Args &g)
{
   constexpr int CHUNK = 256 / T;
   const int blocks = cdiv(g.N, 4 * T);
   int splits = 8 * ctx->num_cus / blocks;
   if (splits > g.K / (16 * CHUNK)) splits = g.K / (16 * CHUNK);
   if ((size_t)splits * g.M * g.N * 4 > ((size_t)4 << 20) && splits > g.K / (4 * g.M)) splits = g.K / (4 * g.M);
   if (splits < 1) splits = 1;
   const int kslice = cdiv(cdiv(g.K, splits), 4 * CHUNK) * 4 * CHUNK;
   splits = cdiv(g.K, kslice);
   float *partial = nullptr;
   if (splits > 1) {
      void *ws = nullptr;
      if (int rc = workspace(ctx, (size_t)splits * g.M * g.N * sizeof(float), &ws)) return rc;
      partial = static_cast<float *>(ws);
   }
   hipLaunchKernelGGL((k_gemm_f32_skinny<B_NK, T, MT>), dim3(blocks, splits), dim3(256), 0, ctx->stream, g, partial, kslice, splits);
   if (int rc = check_launch(ctx, "k_gemm_f32_skinny")) return rc;
   if (splits == 1) return SOFIE_HIP_OK;
   hipLaunchKernelGGL(k_gemm_f32_skinny_finish, dim3(cdiv(g.M * g.N, 256)), dim3(256), 0, ctx->stream, g, partial, splits);
   return check_launch(ctx, "k_gemm_f32_skinny_finish");
}

int launch_skinny(sofie_hip_ctx *ctx, GemmF32Args &g)
{
   if (g.M <= 16) return g.transB ? launch_skinny_as<true, 16, 1>(ctx, g) : launch_skinny_as<false, 16, 1>(ctx, g);
   // 17 to 64 rows as two or four tiles of 16 rows: 32 x 32 tiles (twice the columns per wavefront, twice the
   // accumulator registers) measured 9 - 13 % slower (64 x 4096 x 4096: 42.7 against 37.7 us)
   if (g.M <= 32) return g.transB ? launch_skinny_as<true, 16, 2>(ctx, g) : launch_skinny_as<false, 16, 2>(ctx, g);
   return g.transB ? launch_skinny_as<true, 16, 4>(ctx, g) : launch_skinny_as<false, 16, 4>(ctx, g);
}

}  // namespace

extern "C" int sofie_hip_gemm_f32(sofie_hip_ctx *ctx, int transA, int transB, int M, int N, int K, float alpha,
                                  const float *A, int lda, const float *B, int ldb, float beta, const float *bias,
                                  int bias_kind, float *Y, int ldy, int act)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, M >= 0 && N >= 0 && K >= 0, "negative dimension");
   if (M == 0 || N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, Y && (K == 0 || (A && B)), "null operand");
   SOFIE_REQUIRE(ctx, lda >= (transA ? M : K) && ldb >= (transB ? K : N) && ldy >= N, "leading dimension too small");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   SOFIE_REQUIRE(ctx, bias_kind >= SOFIE_BIAS_NONE && bias_kind <= SOFIE_BIAS_COL, "unknown bias kind");
   if (!bias || bias_kind == SOFIE_BIAS_NONE) {
      // Same rule as the reference emitter: without a bias tensor beta must be zero.
      if (beta != 0.0f)
         return sofie::set_error(ctx, SOFIE_HIP_EINVAL,
                                 "sofie_hip_gemm_f32: Bias tensor is not present but beta value in Gemm is not zero");
      bias = nullptr;
      bias_kind = SOFIE_BIAS_NONE;
   }
   GemmF32Args g{};
   g.A = A; g.B = B; g.bias = bias; g.Y = Y;
   g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldy = ldy;
   g.transA = transA != 0; g.transB = transB != 0;
   g.alpha = alpha; g.beta = beta; g.bias_kind = bias_kind; g.relu = act == SOFIE_ACT_RELU;
   const bool small = (size_t)cdiv(M, 128) * cdiv(N, 128) < 256;
   // operands by LDS-DMA: A row-major with rows of whole 16-byte chunks, K in whole stages, everything a descriptor
   // addresses below 2 GiB, a bias that is a row, a column or absent; 64 x 64 tiles where 128 x 128 ones would leave
   // compute units without a tile, and nothing for products of a handful of tiles
   const auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
   const int tile = small ? 64 : 128;
   const bool dma = (size_t)cdiv(M, 64) * cdiv(N, 64) >= 32 && !transA && K >= 32 && K % 32 == 0 && lda % 4 == 0 && ldb % 4 == 0 &&
                    (transB || N % 4 == 0) && aligned16(A) && aligned16(B) && bias_kind != SOFIE_BIAS_FULL &&
                    (size_t)128 * lda * 4 < (1u << 31) && (size_t)(transB ? 128 : K) * ldb * 4 < (1u << 31) &&
                    (size_t)128 * ldy * 4 < (1u << 31) && (size_t)cdiv(M, tile) * cdiv(N, tile) < (1u << 30);
   // a few rows of A on a B of some size: a pass over B (k_gemm_f32_skinny); needs whole 16-byte chunks per lane. With 33 to
   // 64 rows and thousands of column tiles the 64 x 64 tiles below fill the device and reuse B from LDS.
   const bool skinny = (M <= 32 || (M <= 64 && N < 8192)) && !transA && K >= 64 && K % 4 == 0 && (size_t)N * K >= 64 * 1024 && lda % 4 == 0 && ldb % 4 == 0 &&
                       (transB || N % 4 == 0) && aligned16(A) && aligned16(B) &&
                       (size_t)M * lda * 4 < (1u << 31) && (size_t)(transB ? N : K) * ldb * 4 < (1u << 31) &&
                       (size_t)M * ldy < (1u << 31);
   if (skinny) return launch_skinny(ctx, g);
   if (dma) {
      constexpr auto kern_nk2 = k_gemm_f32_dma<false, 2>, kern_kn2 = k_gemm_f32_dma<true, 2>;
      constexpr auto kern_nk1 = k_gemm_f32_dma<false, 1>, kern_kn1 = k_gemm_f32_dma<true, 1>;
      SOFIE_LARGE_LDS(kern_nk2);
      SOFIE_LARGE_LDS(kern_kn2);
      SOFIE_LARGE_LDS(kern_nk1);
      SOFIE_LARGE_LDS(kern_kn1);
      const auto kern = small ? (transB ? kern_nk1 : kern_kn1) : (transB ? kern_nk2 : kern_kn2);
      // tiles for less than half of the compute units and a K of 16 steps or more: K in slices (of at least 8 steps) so
      // that about two workgroups per compute unit exist; the slices' sums are added by the pass of the few-rows kernel
      // (128 x 1024 x 4096: 18.5 against 76.9 us; with a tile for every compute unit slices gain and lose: -6 % .. +14 %)
      const int tiles = cdiv(M, tile) * cdiv(N, tile), steps = K / 32;
      int splits = 1;
      if (small && tiles * 2 <= ctx->num_cus && steps >= 16) {
         splits = 2 * ctx->num_cus / tiles;
         if (splits > steps / 8) splits = steps / 8;
         if (splits > 16) splits = 16;
         splits = cdiv(steps, cdiv(steps, splits));
      }
      if (splits > 1) {
         void *ws = nullptr;
         if (int rc = workspace(ctx, (size_t)splits * M * N * sizeof(float), &ws)) return rc;
         g.partial = static_cast<float *>(ws);
      }
      hipLaunchKernelGGL(kern, dim3(tiles, splits), dim3(256), 2 * (tile + tile) * 32 * 4, ctx->stream, g);
      if (int rc = check_launch(ctx, small ? "k_gemm_f32_dma64" : "k_gemm_f32_dma")) return rc;
      if (splits == 1) return SOFIE_HIP_OK;
      hipLaunchKernelGGL(k_gemm_f32_skinny_finish, dim3(cdiv(M * N, 256)), dim3(256), 0, ctx->stream, g, g.partial, splits);
      return check_launch(ctx, "k_gemm_f32_skinny_finish");
   } else if (small) {
      hipLaunchKernelGGL((k_gemm_f32<1, 1>), dim3(cdiv(N, 64), cdiv(M, 64)), dim3(256), 0, ctx->stream, g);
   } else {
      hipLaunchKernelGGL((k_gemm_f32<2, 2>), dim3(cdiv(N, 128), cdiv(M, 128)), dim3(256), 0, ctx->stream, g);
   }
   return check_launch(ctx, "k_gemm_f32");
}

extern "C" int sofie_hip_gemm_f32_stacked(sofie_hip_ctx *ctx, int transA, int transB, int M, int N, int K, float alpha,
                                          const float *A, int lda, const float *B, int ldb, float *Y, int ldy, int n_lead,
                                          const int *lead, const long long *stride_a, const long long *stride_b, int act)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, M >= 0 && N >= 0 && K >= 0, "negative dimension");
   SOFIE_REQUIRE(ctx, n_lead >= 1 && n_lead <= SOFIE_GEMM_MAX_LEAD && lead && stride_a && stride_b, "bad leading dimensions");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   long long stack = 1;
   for (int d = 0; d < n_lead; ++d) {
      SOFIE_REQUIRE(ctx, lead[d] >= 0 && stride_a[d] >= 0 && stride_b[d] >= 0, "negative extent or stride");
      stack *= lead[d];
      SOFIE_REQUIRE(ctx, stack < (1ll << 31), "too many stacked products");
   }
   if (M == 0 || N == 0 || stack == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, Y && (K == 0 || (A && B)), "null operand");
   SOFIE_REQUIRE(ctx, lda >= (transA ? M : K) && ldb >= (transB ? K : N) && ldy >= N, "leading dimension too small");
   GemmF32Args g{};
   g.A = A; g.B = B; g.bias = nullptr; g.Y = Y;
   g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldb = ldb; g.ldy = ldy;
   g.transA = transA != 0; g.transB = transB != 0;
   g.alpha = alpha; g.beta = 0.0f; g.bias_kind = SOFIE_BIAS_NONE; g.relu = act == SOFIE_ACT_RELU;
   g.n_lead = n_lead;
   for (int d = 0; d < n_lead; ++d) { g.lead[d] = lead[d]; g.sa[d] = stride_a[d]; g.sb[d] = stride_b[d]; }
   g.stride_y = (long long)M * ldy;
   // the grid's third dimension holds at most 65535 products per launch
   for (long long z0 = 0; z0 < stack; z0 += 65535) {
      const unsigned nz = (unsigned)((stack - z0) < 65535 ? (stack - z0) : 65535);
      g.z0 = (int)z0;
      const bool small = (size_t)cdiv(M, 128) * cdiv(N, 128) * nz < 256;
      if (small) hipLaunchKernelGGL((k_gemm_f32<1, 1>), dim3(cdiv(N, 64), cdiv(M, 64), nz), dim3(256), 0, ctx->stream, g);
      else hipLaunchKernelGGL((k_gemm_f32<2, 2>), dim3(cdiv(N, 128), cdiv(M, 128), nz), dim3(256), 0, ctx->stream, g);
      if (int rc = check_launch(ctx, "k_gemm_f32_stacked")) return rc;
   }
   return SOFIE_HIP_OK;
}

// ------------------------------------------------------------------------------------------------------------
// A chain of small fully connected layers in one launch: y = act_L(... act_1(x W_1 + b_1) ... W_L + b_L).
// A multilayer perceptron on a few hundred rows is three kernel launches of a few microseconds each and nothing
// else: the matrix cores have nothing to chew on (8.65 MFLOP for 256 rows of 64 -> 128 -> 64 -> 8) and the time
// is the launches. Here a workgroup carries R rows through every layer with the activations in LDS; the weights
// (W_l [K_l, N_l], row-major) come straight from L2, one coalesced row of N_l per step of k. With N_l below the
// 256 threads of the workgroup the threads also split K: thread (o, part) sums its share of k for output o, the
// partial sums meet in LDS. Plain fp32 fused multiply-adds in a fixed order per output; no matrix instructions.
namespace {

struct MlpArgs {
   const float *W[SOFIE_MLP_MAX_LAYERS];
   const float *bias[SOFIE_MLP_MAX_LAYERS];
   int dims[SOFIE_MLP_MAX_LAYERS + 1];
   int relu[SOFIE_MLP_MAX_LAYERS];
   const float *x;
   float *y;
   int n_layers, M, ldx, ldy, maxd;
};

template <int R>
__global__ void __launch_bounds__(256) k_mlp_f32(MlpArgs a)
{
   extern __shared__ __align__(16) float s_mlp[];
   float *buf_in = s_mlp, *buf_out = s_mlp + R * a.maxd;     // activations of the rows, [R][maxd] each
   float *part = s_mlp + 2 * R * a.maxd;                     // [256][R] partial sums
   const int tid = threadIdx.x;
   const int row0 = blockIdx.x * R;
   {
      const int K0 = a.dims[0];
      for (int idx = tid; idx < R * K0; idx += 256) {
         const int r = idx / K0, k = idx - r * K0;
         buf_in[r * a.maxd + k] = row0 + r < a.M ? a.x[(size_t)(row0 + r) * a.ldx + k] : 0.0f;
      }
   }
   __syncthreads();
   for (int l = 0; l < a.n_layers; ++l) {
      const int K = a.dims[l], N = a.dims[l + 1];
      const float *__restrict__ W = a.W[l];
      const bool last = l + 1 == a.n_layers;
      // columns per pass (a power of two, at most 256) and the parts K is cut into
      int n2 = 1;
      while (n2 < N && n2 < 256) n2 <<= 1;
      const int parts = 256 / n2;
      const int kc = (K + parts - 1) / parts;
      const int oc = tid & (n2 - 1), pt = tid / n2;
      const int k0 = pt * kc, k1 = k0 + kc < K ? k0 + kc : K;
      for (int o0 = 0; o0 < N; o0 += n2) {
         const int o = o0 + oc;
         float acc[R];
#pragma unroll
         for (int r = 0; r < R; ++r) acc[r] = 0.0f;
         if (o < N) {
            const float *w = W + (size_t)k0 * N + o;
#pragma unroll 8
            for (int k = k0; k < k1; ++k) {
               const float wv = *w;
               w += N;
#pragma unroll
               for (int r = 0; r < R; ++r) acc[r] = fmaf(buf_in[r * a.maxd + k], wv, acc[r]);
            }
         }
         auto finish = [&](int r, int oo, float v) {
            if (a.bias[l]) v += a.bias[l][oo];
            if (a.relu[l]) v = fmaxf(v, 0.0f);
            if (last) {
               if (row0 + r < a.M) a.y[(size_t)(row0 + r) * a.ldy + oo] = v;
            } else {
               buf_out[r * a.maxd + oo] = v;
            }
         };
         if (parts == 1) {
            // 256 columns per pass: every thread holds the complete sums of its column
            if (o < N) {
#pragma unroll
               for (int r = 0; r < R; ++r) finish(r, o, acc[r]);
            }
         } else {
#pragma unroll
            for (int r = 0; r < R; ++r) part[tid * R + r] = acc[r];
            __syncthreads();
            // the parts of an output are added in order by one thread per (row, output)
            for (int idx = tid; idx < R * n2; idx += 256) {
               const int r = idx / n2, c = idx - r * n2;
               if (o0 + c >= N) continue;
               float v = 0.0f;
               for (int p = 0; p < parts; ++p) v += part[(p * n2 + c) * R + r];
               finish(r, o0 + c, v);
            }
         }
         if (parts > 1) __syncthreads();   // the partial sums are read before the next pass overwrites them
      }
      __syncthreads();
      float *t = buf_in; buf_in = buf_out; buf_out = t;
   }
}

}  // namespace

extern "C" int sofie_hip_mlp_f32(sofie_hip_ctx *ctx, int n_layers, const int *dims, const float *const *W,
                                 const float *const *bias, const int *act, const float *x, int ldx, float *y, int ldy,
                                 int M)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, n_layers >= 1 && n_layers <= SOFIE_MLP_MAX_LAYERS && dims && W && act, "bad layer list");
   SOFIE_REQUIRE(ctx, M >= 0, "negative dimension");
   MlpArgs a{};
   int maxd = 0;
   for (int l = 0; l <= n_layers; ++l) {
      SOFIE_REQUIRE(ctx, dims[l] >= 1 && dims[l] <= SOFIE_MLP_MAX_WIDTH, "layer width out of range");
      a.dims[l] = dims[l];
      if (dims[l] > maxd) maxd = dims[l];
   }
   for (int l = 0; l < n_layers; ++l) {
      SOFIE_REQUIRE(ctx, W[l], "null weight matrix");
      SOFIE_REQUIRE(ctx, act[l] == SOFIE_ACT_NONE || act[l] == SOFIE_ACT_RELU, "unknown activation");
      a.W[l] = W[l];
      a.bias[l] = bias ? bias[l] : nullptr;
      a.relu[l] = act[l] == SOFIE_ACT_RELU;
   }
   if (M == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   SOFIE_REQUIRE(ctx, ldx >= dims[0] && ldy >= dims[n_layers], "leading dimension too small");
   a.x = x; a.y = y; a.n_layers = n_layers; a.M = M; a.ldx = ldx; a.ldy = ldy;
   a.maxd = (maxd + 3) & ~3;
   // rows per workgroup: one while that still gives every CU a workgroup, more when there are rows to share the
   // weight traffic between
   const int cus = ctx->num_cus > 0 ? ctx->num_cus : 256;
   const int R = M <= 2 * cus ? 1 : M <= 8 * cus ? 4 : 8;
   const size_t lds = ((size_t)2 * R * a.maxd + (size_t)256 * R) * sizeof(float);
   const dim3 grid((unsigned)cdiv(M, R)), block(256);
   // (up to 72 KB of LDS at the widest layers: above the default limit of a launch)
   SOFIE_LARGE_LDS(k_mlp_f32<1>);
   SOFIE_LARGE_LDS(k_mlp_f32<4>);
   SOFIE_LARGE_LDS(k_mlp_f32<8>);
   if (R == 1) hipLaunchKernelGGL(k_mlp_f32<1>, grid, block, lds, ctx->stream, a);
   else if (R == 4) hipLaunchKernelGGL(k_mlp_f32<4>, grid, block, lds, ctx->stream, a);
   else hipLaunchKernelGGL(k_mlp_f32<8>, grid, block, lds, ctx->stream, a);
   return check_launch(ctx, "k_mlp_f32");
}
