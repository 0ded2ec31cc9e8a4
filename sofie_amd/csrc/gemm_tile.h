// Pieces shared by the tiled MFMA kernels of one-byte operands (GEMM and implicit-GEMM convolution):
// the matrix-instruction traits, the argument block of an output tile and the epilogue that turns
// accumulator tiles into packed, row-contiguous stores.
#pragma once
#include "common.h"

namespace sofie {

struct MmaI8 {
   typedef v16i Acc;
   typedef v4i Frag;
   static constexpr int KB = 32;           // bytes of K consumed by one instruction
   static constexpr int LANE_BYTES = 16;   // bytes of K one lane supplies per operand
   static __device__ __forceinline__ Frag load(const unsigned char *p) { return *reinterpret_cast<const v4i *>(p); }
   static __device__ __forceinline__ Acc mma(Frag a, Frag b, Acc c)
   {
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
   }
};

struct MmaF8 {
   typedef v16f Acc;
   typedef v8i Frag;
   static constexpr int KB = 64;
   static constexpr int LANE_BYTES = 32;
   static __device__ __forceinline__ Frag load(const unsigned char *p)
   {
      const v4i lo = *reinterpret_cast<const v4i *>(p), hi = *reinterpret_cast<const v4i *>(p + 16);
      Frag f = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      return f;
   }
   static __device__ __forceinline__ Acc mma(Frag a, Frag b, Acc c)
   {
      // cbsz = blgp = 0 selects e4m3 for both operands; zero scale operands = unscaled.
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
   }
};

struct GemmArgs {
   const uint8_t *A;
   const uint8_t *B;
   void *Y;
   const float *scale;   // [N] (int8) or nullptr
   const void *bias;     // int32 [N] (int8) / float [N] (fp8) or nullptr
   int M, N, K, lda, ldb, ldy;
   int zp, lo;           // int8 output zero-point and lower clamp
   int relu;
   float s;              // fp8: scale_a * scale_b
   int tiles_m, tiles_n;
   int vec_store;        // rows of Y may be written with 16-byte stores
   // split K (int32 partial sums only): workgroup b works on K slice b / (tiles_m * tiles_n) of `kslice`
   // bytes and writes its tile into the slice's own copy of Y, `ysplit` bytes after the previous one
   int splits, kslice;
   long long ysplit;
};

template <int OUT> struct OutSize { static constexpr int value = 4; };
template <> struct OutSize<SOFIE_OUT_S8> { static constexpr int value = 1; };
template <> struct OutSize<SOFIE_OUT_BF16> { static constexpr int value = 2; };

__device__ __forceinline__ float e4m3_to_f32(unsigned v)
{
   const unsigned e = (v >> 3) & 15u, m = v & 7u;
   float r;
   if (e == 15u && m == 7u) return __uint_as_float(0x7fc00000u);
   if (e == 0u) r = (float)m * 0.001953125f;
   else r = __uint_as_float(((e + 120u) << 23) | (m << 20));
   return (v & 0x80u) ? -r : r;
}

// One output element of the epilogue from an int32 (int8 path) or fp32 (fp8 path) accumulator.
// `bias_bits` holds the column's int32 bias (int8 path) or fp32 bias bits (fp8 path), 0 if none.
template <bool IS_INT, int OUT>
__device__ __forceinline__ unsigned epilogue_value(const GemmArgs &g, float sc, int bias_bits, int raw_i, float raw_f)
{
   if constexpr (IS_INT) {
      const int a = raw_i + bias_bits;
      if constexpr (OUT == SOFIE_OUT_S32) return (unsigned)a;
      if constexpr (OUT == SOFIE_OUT_S8) return __float_as_uint(requant_biased(a, sc, g.zp, g.lo));
      float v = __fmul_rn(__int2float_rn(a), sc);
      if (g.relu && !(v > 0.0f)) v = 0.0f;
      return __float_as_uint(v);
   } else {
      float t = __fmul_rn(raw_f, g.s);
      if (g.bias) t = __fadd_rn(t, __int_as_float(bias_bits));
      if constexpr (OUT == SOFIE_OUT_BF16) return f32_to_bf16(t);
      return __float_as_uint(t);
   }
}

// Epilogue shared by the tiled kernels. Each wavefront owns TI x TJ accumulator tiles
// (rows = output columns n, columns = output rows m). Per pass j it converts TI tiles, packs
// four consecutive n of one m into a 4*esize store into its private LDS staging block
// [32 m][TI*32 n], then writes the block out as 16-byte row segments. The staging block is
// private to the wavefront and LDS operations of one wavefront complete in order, so no
// workgroup barrier is needed between the passes.
//   stg: this wavefront's staging block, 32 * (TI*32*esize + 16) bytes;
//   s_scale, s_bias: per-column scale and bias bits in LDS, already pointing at the
//     wavefront's first column, filled and made visible by the caller;
//   m_wave, n_wave: first output row and column of this wavefront.
// ADD_BIAS false: the accumulators already include the bias.
// PLAIN = 2: int8 output with lower clamp -128 and any zero-point: the byte conversion's saturation at 0 is the clamp.
// PLAIN = 1: int8 output with zero-point -128 and lower clamp -128: the byte conversion rounds half to
// even and saturates, so it is the whole requantisation after the multiply.
template <int TI, int OUT> struct EpilogueStaging {
   static constexpr int ESZ = OutSize<OUT>::value;
   static constexpr int SROW = TI * 32 * ESZ + 16;   // staging row stride in bytes
   static constexpr int WAVE_BYTES = 32 * SROW;
};

// FULLN: every 16-byte row segment lies inside the matrix and rows may be written with 16-byte
// stores (no column checks). reg_scale: if not null, the lane's TI*4 scale vectors held in
// registers (group gi = i*4 + q covers columns i*32 + q*8 + (lane/32)*4 .. +3); s_scale is then unused.
template <class Mma, int TI, int TJ, int OUT, int PLAIN, bool ADD_BIAS = true, bool FULLN = false>
__device__ __forceinline__ void tile_epilogue_wave(const GemmArgs &g, typename Mma::Acc (&acc)[TI][TJ],
                                                   unsigned char *stg, const float *s_scale, const int *s_bias,
                                                   int lane, int m_wave, int n_wave,
                                                   const v4f (*reg_scale)[TI * 4] = nullptr, bool write_through = true)
{
   constexpr int ESZ = OutSize<OUT>::value;
   constexpr bool IS_INT = __is_same(typename Mma::Acc, v16i);
   constexpr int WN = TI * 32;                       // output columns of one wavefront
   constexpr int SROW = EpilogueStaging<TI, OUT>::SROW;
   constexpr int CR = WN * ESZ / 16;                 // 16-byte chunks per staging row
   constexpr int NG = TI * 4;                        // groups of four columns per lane and pass
   const int m_local = lane & 31;
   const int nq = (lane >> 5) * 4;
   const float zpo = (float)(g.zp + 128), lof = (float)(g.lo + 128);
#pragma unroll
   for (int j = 0; j < TJ; ++j) {
      // scale and bias of group gi+1 are read while group gi is converted
      v4f sc_next = {0.0f, 0.0f, 0.0f, 0.0f};
      v4i bi_next = {0, 0, 0, 0};
      if (!reg_scale) sc_next = *reinterpret_cast<const v4f *>(s_scale + nq);
      if (ADD_BIAS || !IS_INT) bi_next = *reinterpret_cast<const v4i *>(s_bias + nq);
#pragma unroll
      for (int gi = 0; gi < NG; ++gi) {
         const int i = gi >> 2, q = gi & 3;
         const int nl = i * 32 + q * 8 + nq;
         const v4f sc = reg_scale ? (*reg_scale)[gi] : sc_next;
         const v4i bi = bi_next;
         if (gi + 1 < NG) {
            const int nn = ((gi + 1) >> 2) * 32 + ((gi + 1) & 3) * 8 + nq;
            if (!reg_scale) sc_next = *reinterpret_cast<const v4f *>(s_scale + nn);
            if (ADD_BIAS || !IS_INT) bi_next = *reinterpret_cast<const v4i *>(s_bias + nn);
         }
         unsigned char *dst = stg + m_local * SROW + nl * ESZ;
         if constexpr (IS_INT && ESZ == 1) {
            // rint(float(acc) * scale) + zp + 128, clamped below at lo + 128; the byte conversion
            // saturates at 0 and 255, i.e. at q = -128 and q = 127
            unsigned pk = 0;
            float e[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
               float r = __fmul_rn(__int2float_rn(acc[i][j][q * 4 + t] + (ADD_BIAS ? bi[t] : 0)), sc[t]);
               // v_cvt_pk_u8_f32 itself rounds to nearest even: with nothing to add, the product goes in as it is
               if constexpr (PLAIN == 0) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);
               if constexpr (PLAIN == 2) r = __fadd_rn(rintf(r), zpo);
               e[t] = r;
            }
            pk = __builtin_amdgcn_cvt_pk_u8_f32(e[0], 0, pk);
            pk = __builtin_amdgcn_cvt_pk_u8_f32(e[1], 1, pk);
            pk = __builtin_amdgcn_cvt_pk_u8_f32(e[2], 2, pk);
            pk = __builtin_amdgcn_cvt_pk_u8_f32(e[3], 3, pk);
            *reinterpret_cast<unsigned *>(dst) = pk ^ 0x80808080u;
         } else if constexpr (!IS_INT && OUT == SOFIE_OUT_BF16) {
            // acc * (scale_a * scale_b) [+ bias], then the hardware's packed conversion (round to nearest even)
            float e[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
               e[t] = __fmul_rn(acc[i][j][q * 4 + t], g.s);
               if (g.bias) e[t] = __fadd_rn(e[t], __int_as_float(bi[t]));
            }
            v2i p = {(int)f32x2_to_bf16x2(e[0], e[1]), (int)f32x2_to_bf16x2(e[2], e[3])};
            *reinterpret_cast<v2i *>(dst) = p;
         } else {
            unsigned e[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
               if constexpr (IS_INT)
                  e[t] = epilogue_value<true, OUT>(g, sc[t], ADD_BIAS ? bi[t] : 0, acc[i][j][q * 4 + t], 0.0f);
               else
                  e[t] = epilogue_value<false, OUT>(g, sc[t], bi[t], 0, acc[i][j][q * 4 + t]);
            }
            if constexpr (ESZ == 2) {
               v2i p = {(int)(e[0] | (e[1] << 16)), (int)(e[2] | (e[3] << 16))};
               *reinterpret_cast<v2i *>(dst) = p;
            } else {
               v4i p = {(int)e[0], (int)e[1], (int)e[2], (int)e[3]};
               *reinterpret_cast<v4i *>(dst) = p;
            }
         }
      }
      __builtin_amdgcn_wave_barrier();
      constexpr int ITERS = 32 * CR / 64;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
         const int c = it * 64 + lane;
         const int row = c / CR, cc = c % CR;
         const int m = m_wave + j * 32 + row;
         const int nfirst = n_wave + cc * (16 / ESZ);
         if (m < g.M && (FULLN || nfirst < g.N)) {
            const v4i v = *reinterpret_cast<const v4i *>(stg + row * SROW + cc * 16);
            unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + nfirst) * ESZ;
            if (FULLN || (g.vec_store && nfirst + 16 / ESZ <= g.N)) {
               if (write_through) store16_wt(out, v);
               else *reinterpret_cast<v4i *>(out) = v;
            } else {
               const unsigned char *src = stg + row * SROW + cc * 16;
               const int cnt = (g.N - nfirst) < (16 / ESZ) ? (g.N - nfirst) : (16 / ESZ);
               for (int b = 0; b < cnt * ESZ; ++b) out[b] = src[b];
            }
         }
      }
      __builtin_amdgcn_wave_barrier();
   }
}

// v[i] holds, per lane (half, l32), the 16 consecutive columns half * 16 .. + 15 of 32-column tile i of row
// m_first + l32 (what two v_permlane32_swap make of a 32 x 32 accumulator tile's packed bytes; for the convolutions a
// row is a pixel and the columns are its channels). One more swap between the halves of the wavefront and one
// between neighbouring groups of 16 lanes sort the four 16-byte quarters of a row's 64 columns onto the four lane
// groups, so that a store instruction writes the whole 64 bytes of 16 rows and can go through the L2 (store16_wt).
__device__ __forceinline__ void store_pixels_64(const GemmArgs &g, const unsigned (&v)[2][4], int lane, int m_first, int n_wave)
{
   const int kg = lane >> 4, l16 = lane & 15;
   // lane groups of 16 hold (pixels 0-15, 16-31 | quarter 0 resp. 2) in the lower half and (.. | quarter 1 resp. 3) in the
   // upper half of v[0] resp. v[1]; after the two swaps a[] has quarter kg of pixel l16, b[] quarter kg of pixel 16 + l16
   unsigned a[4], b[4];
#pragma unroll
   for (int e = 0; e < 4; ++e) {
      const auto x = __builtin_amdgcn_permlane32_swap(v[0][e], v[1][e], false, false);
      const auto y = __builtin_amdgcn_permlane16_swap(x[0], x[1], false, false);
      a[e] = y[0];
      b[e] = y[1];
   }
   const int ma = m_first + l16, mb = ma + 16;
   int8_t *const col = static_cast<int8_t *>(g.Y) + n_wave + kg * 16;
   if (ma < g.M) store16_wt(col + (size_t)ma * g.ldy, v4i{(int)a[0], (int)a[1], (int)a[2], (int)a[3]});
   if (mb < g.M) store16_wt(col + (size_t)mb * g.ldy, v4i{(int)b[0], (int)b[1], (int)b[2], (int)b[3]});
}

// int8 epilogue without LDS staging, for tiles whose columns are all inside the matrix: a lane packs its
// four 4-column groups of a 32 x 32 accumulator tile into four dwords; two v_permlane32_swap between the
// halves of the wavefront turn them into 16 consecutive columns per lane (lanes 0-31: columns 0-15 of
// the tile, lanes 32-63: columns 16-31), which leave as one 16-byte store, or, with an even number of column tiles,
// as 64 contiguous bytes per row of two neighbouring tiles (store_pixels_64). Rows need ldy % 16 == 0 and
// a 16-byte aligned Y. reg_scale as in tile_epilogue_wave (may be null: scales are then read from s_scale).
template <int TI, int TJ, bool PLAIN, bool ADD_BIAS>
__device__ __forceinline__ void tile_epilogue_s8_direct(const GemmArgs &g, v16i (&acc)[TI][TJ], const float *s_scale,
                                                        const int *s_bias, int lane, int m_wave, int n_wave,
                                                        const v4f (*reg_scale)[TI * 4] = nullptr)
{
   const int l32 = lane & 31, half = lane >> 5;
   const int nq = half * 4;
   const float zpo = (float)(g.zp + 128), lof = (float)(g.lo + 128);
#pragma unroll
   for (int j = 0; j < TJ; ++j) {
      const int m = m_wave + j * 32 + l32;
      int8_t *row = static_cast<int8_t *>(g.Y) + (size_t)(m < g.M ? m : 0) * g.ldy + n_wave + half * 16;
      unsigned pair[2][4];
#pragma unroll
      for (int i = 0; i < TI; ++i) {
         unsigned d[4];
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            const v4f sc = reg_scale ? (*reg_scale)[i * 4 + q] : *reinterpret_cast<const v4f *>(s_scale + i * 32 + q * 8 + nq);
            v4i bi = {0, 0, 0, 0};
            if (ADD_BIAS) bi = *reinterpret_cast<const v4i *>(s_bias + i * 32 + q * 8 + nq);
            unsigned pk = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
               float r = __fmul_rn(__int2float_rn(acc[i][j][q * 4 + t] + bi[t]), sc[t]);
               if constexpr (!PLAIN) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);   // the byte conversion rounds half to even
               pk = __builtin_amdgcn_cvt_pk_u8_f32(r, t, pk);
            }
            d[q] = pk ^ 0x80808080u;
         }
         const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
         const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
         if constexpr (TI % 2 == 0) {
            // two neighbouring 32-column tiles leave together, as 64 contiguous bytes per row
            pair[i & 1][0] = s02[0]; pair[i & 1][1] = s02[1]; pair[i & 1][2] = s13[0]; pair[i & 1][3] = s13[1];
            if (i & 1) store_pixels_64(g, pair, lane, m_wave + j * 32, n_wave + (i - 1) * 32);
         } else {
            const v4i v = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
            if (m < g.M) *reinterpret_cast<v4i *>(row + i * 32) = v;
         }
      }
   }
}

// Per-column scale and bias bits of a workgroup's BN columns starting at n0 -> LDS.
__device__ __forceinline__ void stage_column_params(const GemmArgs &g, float *s_scale, int *s_bias, int tid, int n0,
                                                    int BN)
{
   if (tid < BN) {
      const int n = n0 + tid;
      // both loads are issued before either value is stored
      const float sc = (g.scale && n < g.N) ? g.scale[n] : 0.0f;
      const int bi = (g.bias && n < g.N) ? static_cast<const int *>(g.bias)[n] : 0;
      s_scale[tid] = sc;
      s_bias[tid] = bi;
   }
}

// Whole-workgroup form: smem is reused ([NWAVES staging blocks][BN scales][BN biases]), so all
// wavefronts must have finished reading operand stages before the call.
//   m_wave: first output row of this wavefront; n0: first output column of the workgroup;
//   wn: index of the wavefront's column block; BN: columns of the workgroup tile.
// Scale and bias bits of column n0 + tid, loaded ahead of the K loop by the kernels that can spare two registers:
// the epilogue then starts without a round trip to memory.
struct ColumnParams {
   float scale;
   int bias;
};
__device__ __forceinline__ ColumnParams load_column_params(const GemmArgs &g, int tid, int n0, int BN)
{
   ColumnParams p = {0.0f, 0};
   if (tid < BN) {
      const int n = n0 + tid;
      p.scale = (g.scale && n < g.N) ? g.scale[n] : 0.0f;
      p.bias = (g.bias && n < g.N) ? static_cast<const int *>(g.bias)[n] : 0;
   }
   return p;
}

template <class Mma, int TI, int TJ, int OUT, int NWAVES>
__device__ __forceinline__ void tile_epilogue(const GemmArgs &g, typename Mma::Acc (&acc)[TI][TJ], unsigned char *smem,
                                              int tid, int m_wave, int n0, int wn, int BN,
                                              const ColumnParams *preloaded = nullptr)
{
   constexpr int WB = EpilogueStaging<TI, OUT>::WAVE_BYTES;
   constexpr int WN = TI * 32;
   const int lane = tid & 63, wave = tid >> 6;
   float *s_scale = reinterpret_cast<float *>(smem + NWAVES * WB);
   int *s_bias = reinterpret_cast<int *>(s_scale + BN);
   if (preloaded) {
      if (tid < BN) {
         s_scale[tid] = preloaded->scale;
         s_bias[tid] = preloaded->bias;
      }
   } else {
      stage_column_params(g, s_scale, s_bias, tid, n0, BN);
   }
   __syncthreads();
   unsigned char *stg = smem + wave * WB;
   if (OUT == SOFIE_OUT_S8 && g.zp == -128 && g.lo == -128)
      tile_epilogue_wave<Mma, TI, TJ, OUT, 1>(g, acc, stg, s_scale + wn * WN, s_bias + wn * WN, lane, m_wave,
                                              n0 + wn * WN);
   else if (OUT == SOFIE_OUT_S8 && g.lo == -128)
      tile_epilogue_wave<Mma, TI, TJ, OUT, 2>(g, acc, stg, s_scale + wn * WN, s_bias + wn * WN, lane, m_wave,
                                              n0 + wn * WN);
   else
      tile_epilogue_wave<Mma, TI, TJ, OUT, 0>(g, acc, stg, s_scale + wn * WN, s_bias + wn * WN, lane, m_wave,
                                              n0 + wn * WN);
}

// The same epilogue for accumulators of the 16 x 16 matrix instructions (v_mfma_i32_16x16x64_i8): a wavefront owns
// NI x MJ tiles; a lane holds output row m = lane % 16 of a tile and its columns (lane / 16) * 4 .. + 3. Two tiles
// along m (32 rows) go through the staging block [32 m][NI*16 n] per pass, then leave as 16-byte row segments.
// The staging block has the size of EpilogueStaging<NI / 2, OUT>.
template <int NI, int MJ, int OUT, int PLAIN>
__device__ __forceinline__ void tile_epilogue_wave16(const GemmArgs &g, v4i (&acc)[NI][MJ], unsigned char *stg,
                                                     const float *s_scale, const int *s_bias, int lane, int m_wave,
                                                     int n_wave)
{
   static_assert(MJ % 2 == 0, "passes of two tiles along m");
   constexpr int ESZ = OutSize<OUT>::value;
   static_assert(ESZ == 1 || ESZ == 4, "int8 or 32-bit outputs");
   constexpr int WN = NI * 16;
   constexpr int SROW = WN * ESZ + 16;
   constexpr int CR = WN * ESZ / 16;
   const int l16 = lane & 15;
   const int nq = (lane >> 4) * 4;
   const float zpo = (float)(g.zp + 128), lof = (float)(g.lo + 128);
#pragma unroll
   for (int jp = 0; jp < MJ; jp += 2) {
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
         const int nl = ni * 16 + nq;
         const v4f sc = *reinterpret_cast<const v4f *>(s_scale + nl);
         const v4i bi = *reinterpret_cast<const v4i *>(s_bias + nl);
#pragma unroll
         for (int jj = 0; jj < 2; ++jj) {
            const v4i a = acc[ni][jp + jj];
            unsigned char *dst = stg + (jj * 16 + l16) * SROW + nl * ESZ;
            if constexpr (ESZ == 1) {
               unsigned pk = 0;
#pragma unroll
               for (int t = 0; t < 4; ++t) {
                  float r = __fmul_rn(__int2float_rn(a[t] + bi[t]), sc[t]);
                  if constexpr (PLAIN == 0) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);
                  if constexpr (PLAIN == 2) r = __fadd_rn(rintf(r), zpo);
                  pk = __builtin_amdgcn_cvt_pk_u8_f32(r, t, pk);     // rounds half to even, saturates at 0 and 255
               }
               *reinterpret_cast<unsigned *>(dst) = pk ^ 0x80808080u;
            } else {
               v4i p;
#pragma unroll
               for (int t = 0; t < 4; ++t) p[t] = (int)epilogue_value<true, OUT>(g, sc[t], bi[t], a[t], 0.0f);
               *reinterpret_cast<v4i *>(dst) = p;
            }
         }
      }
      __builtin_amdgcn_wave_barrier();
      constexpr int ITERS = 32 * CR / 64;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
         const int c = it * 64 + lane;
         const int row = c / CR, cc = c % CR;
         const int m = m_wave + jp * 16 + row;
         const int nfirst = n_wave + cc * (16 / ESZ);
         if (m < g.M && nfirst < g.N) {
            const v4i v = *reinterpret_cast<const v4i *>(stg + row * SROW + cc * 16);
            unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + nfirst) * ESZ;
            if (g.vec_store && nfirst + 16 / ESZ <= g.N) {
               store16_wt(out, v);
            } else {
               const unsigned char *src = stg + row * SROW + cc * 16;
               const int cnt = (g.N - nfirst) < (16 / ESZ) ? (g.N - nfirst) : (16 / ESZ);
               for (int b = 0; b < cnt * ESZ; ++b) out[b] = src[b];
            }
         }
      }
      __builtin_amdgcn_wave_barrier();
   }
}

// The int8 epilogue of 16 x 16 accumulator tiles without LDS staging, for wavefront tiles whose columns all lie inside
// the matrix and rows that take 16-byte stores. A lane holds columns (lane / 16) * 4 .. + 3 of each 16-column tile of
// its row: packed, the dwords of four neighbouring tiles are a 4 x 4 matrix over the row's four lanes (16 lanes
// apart), and two rounds of swaps (between the halves of the wavefront, then between neighbouring groups of 16 lanes)
// transpose it. Lane group kg then has the 16 columns of tile kg in order, and a store instruction writes 64
// contiguous bytes for each of 16 rows (written through the L2).
// BIAS false: the call has no bias tensor, and the 128 additions of a zero per lane are left out.
template <int NI, int MJ, int PLAIN, bool BIAS = true>
__device__ __forceinline__ void tile_epilogue_wave16_direct(const GemmArgs &g, v4i (&acc)[NI][MJ], const float *s_scale,
                                                            const int *s_bias, int lane, int m_wave, int n_wave)
{
   static_assert(NI % 4 == 0, "groups of four column tiles");
   const int l16 = lane & 15, kg = lane >> 4;
   const float zpo = (float)(g.zp + 128), lof = (float)(g.lo + 128);
#pragma unroll
   for (int ig = 0; ig < NI; ig += 4) {
      v4f sc[4];
      v4i bi[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
         sc[i] = *reinterpret_cast<const v4f *>(s_scale + (ig + i) * 16 + kg * 4);
         if constexpr (BIAS) bi[i] = *reinterpret_cast<const v4i *>(s_bias + (ig + i) * 16 + kg * 4);
      }
#pragma unroll
      for (int j = 0; j < MJ; ++j) {
         const int m = m_wave + j * 16 + l16;
         int8_t *const row = static_cast<int8_t *>(g.Y) + (size_t)(m < g.M ? m : 0) * g.ldy + n_wave + ig * 16 + kg * 16;
         unsigned d[4];
#pragma unroll
         for (int i = 0; i < 4; ++i) {
            unsigned pk = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
               float r = __fmul_rn(__int2float_rn(BIAS ? acc[ig + i][j][t] + bi[i][t] : acc[ig + i][j][t]), sc[i][t]);
               if constexpr (PLAIN == 0) r = fmaxf(__fadd_rn(rintf(r), zpo), lof);
               if constexpr (PLAIN == 2) r = __fadd_rn(rintf(r), zpo);
               pk = __builtin_amdgcn_cvt_pk_u8_f32(r, t, pk);     // rounds half to even, saturates at 0 and 255
            }
            d[i] = pk ^ 0x80808080u;
         }
         const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
         const auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
         const auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
         const auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
         const v4i v = {(int)t01[0], (int)t01[1], (int)t23[0], (int)t23[1]};
         if (m < g.M) store16_wt(row, v);
      }
   }
}

// ---- global memory -> LDS without registers (buffer_load ... lds), shared by the GEMM and the convolution
typedef int rsrc_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ rsrc_t make_rsrc(const void *base, unsigned bytes)
{
   // every component is wave-uniform; readfirstlane tells the compiler so (SGPR operands)
   const unsigned long long a = reinterpret_cast<unsigned long long>(base);
   rsrc_t r = {__builtin_amdgcn_readfirstlane((int)(unsigned)a),
               __builtin_amdgcn_readfirstlane((int)(unsigned)((a >> 32) & 0xffffu)),
               __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
   return r;
}

// 16 bytes per lane from global (descriptor + per-lane offset + uniform offset) to
// LDS address lds_base + lane*16.
__device__ __forceinline__ void dma16(rsrc_t rs, unsigned lds_base, int voff, int soff)
{
   asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                :
                : "s"(__builtin_amdgcn_readfirstlane((int)lds_base)), "v"(voff), "s"(rs),
                  "s"(__builtin_amdgcn_readfirstlane(soff))
                : "memory");
}

// 4 bytes per lane from global to LDS address lds_base + lane*4 (per-column parameters of a tile).
__device__ __forceinline__ void dma4(rsrc_t rs, unsigned lds_base, int voff, int soff)
{
   asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                :
                : "s"(__builtin_amdgcn_readfirstlane((int)lds_base)), "v"(voff), "s"(rs),
                  "s"(__builtin_amdgcn_readfirstlane(soff))
                : "memory");
}

// 4 bytes per lane to global memory through a descriptor (per-lane offset + uniform offset): an address of a few
// instructions less than a flat store's, and a lane whose offset lies outside the descriptor's range stores nothing.
__device__ __forceinline__ void store4_buf(rsrc_t rs, float v, unsigned voff, unsigned soff)
{
   asm volatile("buffer_store_dword %0, %1, %2, %3 offen"
                :
                : "v"(v), "v"(voff), "s"(rs), "s"(__builtin_amdgcn_readfirstlane((int)soff))
                : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
   // s_waitcnt with only the vector-memory counter constrained
   __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

}  // namespace sofie
