// Internal helpers shared by the kernel translation units of libsofie_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "sofie_hip.h"

struct sofie_hip_ctx {
   int device = 0;
   int num_cus = 256;           // compute units of the device (persistent kernels size their grid by it)
   hipStream_t stream = nullptr;
   bool owns_stream = false;
   hipEvent_t ev_start = nullptr, ev_stop = nullptr;
   void *workspace = nullptr;   // scratch owned by the context (layout changes, B transposes)
   size_t workspace_bytes = 0;
   bool capturing = false;      // between sofie_hip_capture_begin and _end: nothing may allocate or synchronise
   bool no_alloc = false;       // inside sofie_hip_qgemm_s8_noalloc: workspace() hands out the fixed array, never allocates
   void *static_scratch = nullptr;   // this device's address of the fixed scratch array (looked up in sofie_hip_create)
   int live_graphs = 0;         // recorded graphs not yet destroyed: they hold the scratch buffer's address
   // between sofie_hip_trace_begin and _end: an event behind every launch (check_launch records it), with the kernel's name
   bool tracing = false;
   int trace_seen = 0;
   struct TracePoint {
      const char *what;
      hipEvent_t done;
   };
   TracePoint *trace = nullptr;   // [SOFIE_HIP_TRACE_MAX + 1], entry 0 is the start
   int trace_len = 0;
   // sofie_hip_constant_weights: copies of weight tensors in the layout a kernel wants, kept per tensor and geometry
   bool constant_weights = false;
   struct PackedWeights {
      const void *w;
      unsigned long long key;
      size_t bytes;
      void *packed;
   };
   PackedWeights *packed = nullptr;   // [SOFIE_HIP_PACKED_MAX]
   int packed_len = 0;
   char err[512] = {0};
};

namespace sofie {

int set_error(sofie_hip_ctx *ctx, int code, const char *fmt, ...);
// Grow-only scratch buffer of the context. Never shrinks; freed in sofie_hip_destroy.
int workspace(sofie_hip_ctx *ctx, size_t bytes, void **ptr);
int check_launch(sofie_hip_ctx *ctx, const char *what);
// Where a kernel's own layout of the weight tensor `w` goes: the context's scratch buffer (*fresh = true: fill it now), or,
// when the caller has promised that its weights do not change (sofie_hip_constant_weights), a buffer kept for this
// tensor and `key` (a hash of everything the layout depends on), filled by the first call only.
int packed_weights(sofie_hip_ctx *ctx, const void *w, unsigned long long key, size_t bytes, void **ptr, bool *fresh);
unsigned long long layout_key(const int *values, int n);
// Bracket of a call that uses the device's fixed scratch array (sofie_hip_qgemm_s8_noalloc): orders it behind the call
// that used the array before it, on whatever context and stream that was.
void scratch_turn_begin(sofie_hip_ctx *ctx);
void scratch_turn_end(sofie_hip_ctx *ctx);

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// Requantisation shared by every int8 epilogue:
//   rint_half_even(float(acc) * scale) + zp, clamped to [lo, 127].
// One int->fp32 conversion (RNE), one fp32 multiply, one round-to-nearest-even.
__device__ __forceinline__ int requant(int acc, float scale, int zp, int lo)
{
   float r = rintf(__fmul_rn(__int2float_rn(acc), scale));
   r = fminf(fmaxf(r, -1024.0f), 1024.0f);
   int q = (int)r + zp;
   return min(127, max(lo, q));
}

// The same requantisation, returned as the float (q + 128) in [0, 255] for epilogues that
// pack with v_cvt_pk_u8_f32: rint(float(acc)*scale) + zp + 128, clamped below at lo + 128;
// the clamp at 255 (q = 127) and at 0 (q = -128) is the saturation of the u8 conversion.
// All quantities are integers well inside fp32's exact range after the first clamp.
__device__ __forceinline__ float requant_biased(int acc, float scale, int zp, int lo)
{
   float r = rintf(__fmul_rn(__int2float_rn(acc), scale));
   r = fminf(fmaxf(r, -1024.0f), 1024.0f);
   return fmaxf(r + (float)(zp + 128), (float)(lo + 128));
}

// fp32 -> bf16 bits, round to nearest even, NaN quieted.
__device__ __forceinline__ unsigned f32_to_bf16(float x)
{
   unsigned u = __float_as_uint(x);
   if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
   u += 0x7fffu + ((u >> 16) & 1u);
   return u >> 16;
}

// Two fp32 -> two bf16 in one dword (lo in bits 0-15), round to nearest even: v_cvt_pk_bf16_f32 of gfx950.
__device__ __forceinline__ unsigned f32x2_to_bf16x2(float lo, float hi)
{
   typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
   typedef float f32x2_t __attribute__((ext_vector_type(2)));
   const f32x2_t v = {lo, hi};
   return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
}

// Layout change of an int8 activation tensor (defined with the element-wise kernels).
int relayout_s8(sofie_hip_ctx *ctx, const int8_t *x, int8_t *y, int N, int C, int H, int W, int from, int to);

// floor(x / d) for 0 <= x < 2^31 as a multiply-high and a shift (shift < 0: d == 1).
struct FastDiv {
   unsigned magic;
   int shift;
};

inline FastDiv make_fastdiv(unsigned d)
{
   if (d <= 1) return {0u, -1};
   int s = 0;
   while ((1u << s) < d) ++s;
   const unsigned long long num = 1ull << (31 + s);
   return {(unsigned)((num + d - 1) / d), s - 1};
}

__device__ __forceinline__ int fdiv(int x, FastDiv f)
{
   return f.shift < 0 ? x : (int)(__umulhi((unsigned)x, f.magic) >> f.shift);
}

// A 16-byte store that is written through the XCD's L2 (system scope) instead of staying there as a dirty line.
// A kernel ends with a write-back of all eight L2s, during which nothing computes; a kernel that runs as a single
// round of workgroups writes most of its output in its last microseconds, so most of it would still be dirty then.
// Written through, the lines are on their way (into the memory-side cache, where the next kernel finds them) while
// the other workgroups still compute. Measured in one process against ordinary stores: int8 GEMM 4096^3 55.8 ->
// 53.5 us, 3x3 int8 convolution on 256 images of 56x56 54.9 -> 52.7 us, on 4096 images of 10x10 30.0 -> 27.3 us,
// first layer of 4096 images 23.7 -> 20.0 us, the int8 CNN Session 111.2 -> 105.5 us. For use where a store
// instruction writes whole 64-byte pieces: on the 32-byte pieces of the pooled epilogues it loses (they are merged
// in the L2), and so it does in kernels whose stores are spread over their whole run (fp32 convolution: +1.6 %).
// Non-temporal stores gain the same in the producer but bypass the memory-side cache: the consumer then reads from
// HBM and the Session as a whole loses 5 %.
__device__ __forceinline__ void store16_wt(void *p, v4i v)
{
   // the wait states behind it: the compiler does not know that this is a store of more than 8 bytes, whose data
   // registers must not be written by the next instruction
   asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

// Kernels that ask for more dynamic LDS than a launch may have by default need the limit raised with
// hipFuncSetAttribute. That is a driver call, so it is made once per kernel and device when a context is created
// (sofie_hip_create), never next to a launch and never while a stream is being captured: a launcher names its kernel
// with SOFIE_LARGE_LDS(kern), which puts the kernel on the library's list when the library is loaded.
void list_large_lds_kernel(const void *func);
template <auto Kern> struct LargeLdsKernel {
   static inline const bool listed = (list_large_lds_kernel(reinterpret_cast<const void *>(Kern)), true);
};
#define SOFIE_LARGE_LDS(kern) ((void)sofie::LargeLdsKernel<kern>::listed)
constexpr int kMaxDynamicLds = 160 * 1024;   // LDS of a gfx950 compute unit

inline int cdiv(int a, int b) { return (a + b - 1) / b; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace sofie

#define SOFIE_REQUIRE(ctx, cond, msg)                                             \
   do {                                                                           \
      if (!(cond)) return sofie::set_error((ctx), SOFIE_HIP_EINVAL, "%s: %s", __func__, (msg)); \
   } while (0)

#define SOFIE_HIP_CALL(ctx, expr)                                                 \
   do {                                                                           \
      hipError_t e_ = (expr);                                                     \
      if (e_ != hipSuccess)                                                       \
         return sofie::set_error((ctx), SOFIE_HIP_EHIP, "%s: %s failed: %s", __func__, #expr, \
                                 hipGetErrorString(e_));                          \
   } while (0)
