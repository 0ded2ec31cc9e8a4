// Einstein summation of fp32 operands for the equations that are not a (stacked) matrix product: one thread
// per output element, the summed labels run as nested loops in the order given (first label outermost), each
// product and each addition rounded on its own. That is the loop nest the reference emits as host code
// (ROperator_Einsum.hxx:236-278), so the sums associate the same way. Equations that are matrix products never
// get here: the emitter turns them into sofie_hip_gemm_f32 calls, as the reference turns them into sgemm_.
#include "common.h"

using namespace sofie;

namespace {

constexpr int MAX_IN = SOFIE_EINSUM_MAX_INPUTS;
constexpr int MAX_LABELS = SOFIE_EINSUM_MAX_LABELS;

struct EinsumArgs {
   const float *x[MAX_IN];
   float *y;
   int n_inputs, n_labels, n_out;
   int extent[MAX_LABELS];
   long long stride[MAX_IN][MAX_LABELS];
   long long outputs, terms;   // elements of y; summed terms per element
};

__global__ void __launch_bounds__(256) k_einsum_f32(EinsumArgs a)
{
   const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
   if (idx >= a.outputs) return;
   // position of the output element along the output labels -> offset into every operand
   long long base[MAX_IN];
#pragma unroll
   for (int i = 0; i < MAX_IN; ++i) base[i] = 0;
   long long rem = idx;
   for (int l = a.n_out - 1; l >= 0; --l) {
      const long long pos = rem % a.extent[l];
      rem /= a.extent[l];
#pragma unroll
      for (int i = 0; i < MAX_IN; ++i)
         if (i < a.n_inputs) base[i] += pos * a.stride[i][l];
   }
   // the summed labels as an odometer, last label fastest
   int pos[MAX_LABELS];
   for (int l = a.n_out; l < a.n_labels; ++l) pos[l] = 0;
   float sum = 0.0f;
   for (long long t = 0; t < a.terms; ++t) {
      float prod = a.x[0][base[0]];
#pragma unroll
      for (int i = 1; i < MAX_IN; ++i)
         if (i < a.n_inputs) prod = __fmul_rn(prod, a.x[i][base[i]]);
      sum = __fadd_rn(sum, prod);
      for (int l = a.n_labels - 1; l >= a.n_out; --l) {
#pragma unroll
         for (int i = 0; i < MAX_IN; ++i)
            if (i < a.n_inputs) base[i] += a.stride[i][l];
         if (++pos[l] < a.extent[l]) break;
#pragma unroll
         for (int i = 0; i < MAX_IN; ++i)
            if (i < a.n_inputs) base[i] -= (long long)a.extent[l] * a.stride[i][l];
         pos[l] = 0;
      }
   }
   a.y[idx] = sum;
}

}  // namespace

extern "C" int sofie_hip_einsum_f32(sofie_hip_ctx *ctx, int n_inputs, const float *const *inputs, int n_labels, int n_out,
                                    const int *extent, const long long *stride, float *y)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, n_inputs >= 1 && n_inputs <= MAX_IN, "between 1 and SOFIE_EINSUM_MAX_INPUTS operands");
   SOFIE_REQUIRE(ctx, n_labels >= 0 && n_labels <= MAX_LABELS && n_out >= 0 && n_out <= n_labels,
                 "at most SOFIE_EINSUM_MAX_LABELS labels, the output labels first");
   SOFIE_REQUIRE(ctx, inputs && y && (n_labels == 0 || (extent && stride)), "null operand");
   EinsumArgs a{};
   a.n_inputs = n_inputs;
   a.n_labels = n_labels;
   a.n_out = n_out;
   a.y = y;
   a.outputs = 1;
   a.terms = 1;
   for (int l = 0; l < n_labels; ++l) {
      SOFIE_REQUIRE(ctx, extent[l] >= 0, "negative extent");
      a.extent[l] = extent[l];
      if (l < n_out) a.outputs *= extent[l];
      else a.terms *= extent[l];
      SOFIE_REQUIRE(ctx, a.outputs < ((long long)1 << 38) && a.terms < ((long long)1 << 40), "operand too large");
   }
   for (int i = 0; i < n_inputs; ++i) {
      SOFIE_REQUIRE(ctx, inputs[i], "null operand");
      a.x[i] = inputs[i];
      for (int l = 0; l < n_labels; ++l) {
         SOFIE_REQUIRE(ctx, stride[(size_t)i * n_labels + l] >= 0, "negative stride");
         a.stride[i][l] = stride[(size_t)i * n_labels + l];
      }
   }
   if (a.outputs == 0) return SOFIE_HIP_OK;
   // an empty sum leaves zeros: the loop runs no term
   hipLaunchKernelGGL(k_einsum_f32, dim3((unsigned)((a.outputs + 255) / 256)), dim3(256), 0, ctx->stream, a);
   return check_launch(ctx, "k_einsum_f32");
}
