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
// [32 m][TI*32 n], then the wavefront writes the block out as 16-byte row segments.
// smem is reused: all waves must have finished reading operand stages before the call.
//   m_wave: first output row of this wavefront; n0: first output column of the workgroup;
//   wn: index of the wavefront's column block; BN: columns of the workgroup tile.
template <class Mma, int TI, int TJ, int OUT, int NWAVES>
__device__ __forceinline__ void tile_epilogue(const GemmArgs &g, typename Mma::Acc (&acc)[TI][TJ], unsigned char *smem,
                                              int tid, int m_wave, int n0, int wn, int BN)
{
   constexpr int ESZ = OutSize<OUT>::value;
   constexpr bool IS_INT = __is_same(typename Mma::Acc, v16i);
   constexpr int WN = TI * 32;                       // output columns of one wavefront
   constexpr int SROW = WN * ESZ + 16;               // staging row stride in bytes
   constexpr int CR = WN * ESZ / 16;                 // 16-byte chunks per staging row
   const int lane = tid & 63, wave = tid >> 6;
   unsigned char *stg = smem + wave * (32 * SROW);
   float *s_scale = reinterpret_cast<float *>(smem + NWAVES * 32 * SROW);   // [BN] per-column scale
   int *s_bias = reinterpret_cast<int *>(s_scale + BN);                     // [BN] per-column bias bits
   if (tid < BN) {
      const int n = n0 + tid;
      s_scale[tid] = (g.scale && n < g.N) ? g.scale[n] : 0.0f;
      s_bias[tid] = (g.bias && n < g.N) ? static_cast<const int *>(g.bias)[n] : 0;
   }
   __syncthreads();
   const int m_local = lane & 31;
   const int nq = (lane >> 5) * 4;
#pragma unroll
   for (int j = 0; j < TJ; ++j) {
#pragma unroll
      for (int i = 0; i < TI; ++i) {
#pragma unroll
         for (int q = 0; q < 4; ++q) {
            const int nl = i * 32 + q * 8 + nq;
            unsigned e[4];
            const v4f sc = *reinterpret_cast<const v4f *>(s_scale + wn * WN + nl);
            const v4i bi = *reinterpret_cast<const v4i *>(s_bias + wn * WN + nl);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
               if constexpr (IS_INT)
                  e[t] = epilogue_value<true, OUT>(g, sc[t], bi[t], acc[i][j][q * 4 + t], 0.0f);
               else
                  e[t] = epilogue_value<false, OUT>(g, sc[t], bi[t], 0, acc[i][j][q * 4 + t]);
            }
            unsigned char *dst = stg + m_local * SROW + nl * ESZ;
            if constexpr (ESZ == 1) {
               // e[] hold q+128 as floats in [0,255]: convert-and-insert, then flip the sign bits
               unsigned pk = 0;
               pk = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(e[0]), 0, pk);
               pk = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(e[1]), 1, pk);
               pk = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(e[2]), 2, pk);
               pk = __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(e[3]), 3, pk);
               *reinterpret_cast<unsigned *>(dst) = pk ^ 0x80808080u;
            } else if constexpr (ESZ == 2) {
               v2i p = {(int)(e[0] | (e[1] << 16)), (int)(e[2] | (e[3] << 16))};
               *reinterpret_cast<v2i *>(dst) = p;
            } else {
               v4i p = {(int)e[0], (int)e[1], (int)e[2], (int)e[3]};
               *reinterpret_cast<v4i *>(dst) = p;
            }
         }
      }
      __syncthreads();
      constexpr int ITERS = 32 * CR / 64;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
         const int c = it * 64 + lane;
         const int row = c / CR, cc = c % CR;
         const int m = m_wave + j * 32 + row;
         const int nfirst = n0 + wn * WN + cc * (16 / ESZ);
         if (m < g.M && nfirst < g.N) {
            const v4i v = *reinterpret_cast<const v4i *>(stg + row * SROW + cc * 16);
            unsigned char *out = static_cast<unsigned char *>(g.Y) + ((size_t)m * g.ldy + nfirst) * ESZ;
            if (g.vec_store && nfirst + 16 / ESZ <= g.N) {
               *reinterpret_cast<v4i *>(out) = v;
            } else {
               const unsigned char *src = stg + row * SROW + cc * 16;
               const int cnt = (g.N - nfirst) < (16 / ESZ) ? (g.N - nfirst) : (16 / ESZ);
               for (int b = 0; b < cnt * ESZ; ++b) out[b] = src[b];
            }
         }
      }
      __syncthreads();
   }
}

}  // namespace sofie
