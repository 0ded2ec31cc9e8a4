// Memory-bound operators: ReLU, max pooling, quantize / dequantize, int8 layout changes.
// All are grid-stride-free flat launches with 16-byte accesses where the shape allows;
// their roofline is HBM bandwidth (bytes in + bytes out per element).
#include "common.h"

using namespace sofie;

namespace {

__global__ void k_relu_f32(const float *__restrict__ x, float *__restrict__ y, size_t len)
{
   const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
   if (i + 3 < len) {
      const v4f v = *reinterpret_cast<const v4f *>(x + i);
      v4f r;
#pragma unroll
      for (int t = 0; t < 4; ++t) r[t] = v[t] > 0.0f ? v[t] : 0.0f;
      *reinterpret_cast<v4f *>(y + i) = r;
   } else {
      for (size_t j = i; j < len; ++j) y[j] = x[j] > 0.0f ? x[j] : 0.0f;
   }
}

__global__ void k_relu_f32_scalar(const float *__restrict__ x, float *__restrict__ y, size_t len)
{
   const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   if (i < len) y[i] = x[i] > 0.0f ? x[i] : 0.0f;
}

// Inference BatchNormalization over [N*C planes][plane] elements: y = (x - mean[c]) * scale[c] + bias[c], each
// step rounded on its own as the reference's copy / axpy / multiply / axpy sequence does
// (ROperator_BatchNormalization.hxx:196-226); scale already holds scale / sqrt(var + eps). One workgroup row
// per plane (blockIdx.y), four elements per thread when the plane length allows it.
template <bool VEC>
__global__ void k_batchnorm_f32(const float *__restrict__ x, const float *__restrict__ scale, const float *__restrict__ mean,
                                const float *__restrict__ bias, float *__restrict__ y, int C, int plane, int relu,
                                int first_channel)
{
   const int pc = blockIdx.y;
   const int c = (pc + first_channel) % C;
   const float s = scale[c], m = mean[c], b = bias[c];
   const float *xp = x + (size_t)pc * plane;
   float *yp = y + (size_t)pc * plane;
   if constexpr (VEC) {
      for (int i = (blockIdx.x * blockDim.x + threadIdx.x) * 4; i < plane; i += gridDim.x * blockDim.x * 4) {
         const v4f v = *reinterpret_cast<const v4f *>(xp + i);
         v4f r;
#pragma unroll
         for (int t = 0; t < 4; ++t) {
            r[t] = __fadd_rn(__fmul_rn(__fsub_rn(v[t], m), s), b);
            if (relu) r[t] = r[t] > 0.0f ? r[t] : 0.0f;
         }
         *reinterpret_cast<v4f *>(yp + i) = r;
      }
   } else {
      for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < plane; i += gridDim.x * blockDim.x) {
         float r = __fadd_rn(__fmul_rn(__fsub_rn(xp[i], m), s), b);
         if (relu) r = r > 0.0f ? r : 0.0f;
         yp[i] = r;
      }
   }
}

template <typename T>
__device__ __forceinline__ T lowest();
template <>
__device__ __forceinline__ float lowest<float>() { return -__builtin_inff(); }
template <>
__device__ __forceinline__ int8_t lowest<int8_t>() { return -128; }

// One thread per output element. NHWC: channel is the fastest index.
template <typename T, bool NHWC>
__global__ void k_maxpool2d(const T *__restrict__ x, T *__restrict__ y, int N, int C, int H, int W, int OH, int OW,
                            int kh, int kw, int pt, int pl, int sh, int sw)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   const size_t total = (size_t)N * C * OH * OW;
   if (idx >= total) return;
   int n, c, oh, ow;
   size_t r = idx;
   if (NHWC) {
      c = (int)(r % C); r /= C;
      ow = (int)(r % OW); r /= OW;
      oh = (int)(r % OH); n = (int)(r / OH);
   } else {
      ow = (int)(r % OW); r /= OW;
      oh = (int)(r % OH); r /= OH;
      c = (int)(r % C); n = (int)(r / C);
   }
   T best = lowest<T>();
   for (int i = 0; i < kh; ++i) {
      const int ih = oh * sh - pt + i;
      if (ih < 0 || ih >= H) continue;
      for (int j = 0; j < kw; ++j) {
         const int iw = ow * sw - pl + j;
         if (iw < 0 || iw >= W) continue;
         const size_t off = NHWC ? (((size_t)n * H + ih) * W + iw) * C + c : (((size_t)n * C + c) * H + ih) * W + iw;
         const T v = x[off];
         if (v > best) best = v;
      }
   }
   y[idx] = best;
}

// NCHW fp32 average pooling, one thread per output element. The window's values are added in row-major order of
// the window (rows outside the image skipped), then divided once by the number of cells counted: the cells inside
// the image, or the whole window when padding cells count (count_include_pad).
__global__ void k_avgpool2d_f32(const float *__restrict__ x, float *__restrict__ y, int NC, int H, int W, int OH, int OW,
                                int kh, int kw, int pt, int pl, int sh, int sw, int include_pad)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   const size_t total = (size_t)NC * OH * OW;
   if (idx >= total) return;
   size_t r = idx;
   const int ow = (int)(r % OW); r /= OW;
   const int oh = (int)(r % OH);
   const size_t nc = r / OH;
   const float *xi = x + nc * H * W;
   float sum = 0.0f;
   int count = 0;
   for (int i = 0; i < kh; ++i) {
      const int ih = oh * sh - pt + i;
      if (ih < 0 || ih >= H) continue;
      for (int j = 0; j < kw; ++j) {
         const int iw = ow * sw - pl + j;
         if (iw < 0 || iw >= W) continue;
         sum = __fadd_rn(sum, xi[(size_t)ih * W + iw]);
         ++count;
      }
   }
   y[idx] = __fdiv_rn(sum, (float)(include_pad ? kh * kw : count));
}

// fp32 pooling over three spatial axes [NC][D0][D1][D2], one thread per output element, the window walked in
// row-major order (last axis fastest) with the cells outside the volume skipped: the maximum, or the sum divided once
// by the number of cells counted (those inside the volume, or the whole window when padding cells count).
struct Pool3dArgs {
   int NC, D[3], O[3], k[3], pad[3], s[3];
};

template <bool AVERAGE>
__global__ void k_pool3d_f32(const float *__restrict__ x, float *__restrict__ y, Pool3dArgs a, int include_pad)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   const size_t total = (size_t)a.NC * a.O[0] * a.O[1] * a.O[2];
   if (idx >= total) return;
   size_t r = idx;
   const int o2 = (int)(r % a.O[2]); r /= a.O[2];
   const int o1 = (int)(r % a.O[1]); r /= a.O[1];
   const int o0 = (int)(r % a.O[0]);
   const size_t nc = r / a.O[0];
   const float *xi = x + nc * a.D[0] * a.D[1] * a.D[2];
   float acc = AVERAGE ? 0.0f : -INFINITY;
   int count = 0;
   for (int i = 0; i < a.k[0]; ++i) {
      const int d0 = o0 * a.s[0] - a.pad[0] + i;
      if (d0 < 0 || d0 >= a.D[0]) continue;
      for (int j = 0; j < a.k[1]; ++j) {
         const int d1 = o1 * a.s[1] - a.pad[1] + j;
         if (d1 < 0 || d1 >= a.D[1]) continue;
         for (int l = 0; l < a.k[2]; ++l) {
            const int d2 = o2 * a.s[2] - a.pad[2] + l;
            if (d2 < 0 || d2 >= a.D[2]) continue;
            const float v = xi[((size_t)d0 * a.D[1] + d1) * a.D[2] + d2];
            if (AVERAGE) {
               acc = __fadd_rn(acc, v);
               ++count;
            } else if (v > acc) {
               acc = v;
            }
         }
      }
   }
   y[idx] = AVERAGE ? __fdiv_rn(acc, (float)(include_pad ? a.k[0] * a.k[1] * a.k[2] : count)) : acc;
}

// Channels-last int8 max pooling, 16 channels (one 16-byte vector) of one output pixel per thread.
// Signed bytes are compared as unsigned after flipping the sign bit, four at a time.
__device__ __forceinline__ unsigned max_u8x4(unsigned a, unsigned b)
{
   unsigned r = 0;
#pragma unroll
   for (int i = 0; i < 4; ++i) {
      const unsigned x = (a >> (8 * i)) & 0xffu, y = (b >> (8 * i)) & 0xffu;
      r |= (x > y ? x : y) << (8 * i);
   }
   return r;
}

__global__ void k_maxpool2d_s8_nhwc16(const int8_t *__restrict__ x, int8_t *__restrict__ y, int N, int C16, int H, int W,
                                      int OH, int OW, int kh, int kw, int pt, int pl, int sh, int sw)
{
   const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   const size_t total = (size_t)N * OH * OW * C16;
   if (idx >= total) return;
   size_t r = idx;
   const int c = (int)(r % C16); r /= C16;
   const int ow = (int)(r % OW); r /= OW;
   const int oh = (int)(r % OH);
   const int n = (int)(r / OH);
   v4i best = {0, 0, 0, 0};   // bytes with the sign bit flipped: 0 is the lowest value
   for (int i = 0; i < kh; ++i) {
      const int ih = oh * sh - pt + i;
      if (ih < 0 || ih >= H) continue;
      for (int j = 0; j < kw; ++j) {
         const int iw = ow * sw - pl + j;
         if (iw < 0 || iw >= W) continue;
         const v4i v = *reinterpret_cast<const v4i *>(x + ((((size_t)n * H + ih) * W + iw) * C16 + c) * 16);
#pragma unroll
         for (int e = 0; e < 4; ++e) best[e] = (int)max_u8x4((unsigned)best[e], (unsigned)v[e] ^ 0x80808080u);
      }
   }
#pragma unroll
   for (int e = 0; e < 4; ++e) best[e] ^= (int)0x80808080u;
   *reinterpret_cast<v4i *>(y + idx * 16) = best;
}

__global__ void k_quantize_f32_s8(const float *__restrict__ x, int8_t *__restrict__ q, size_t len, float scale, int zp)
{
   const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
   if (i >= len) return;
   unsigned packed = 0;
   const int cnt = (len - i) < 4 ? (int)(len - i) : 4;
   for (int t = 0; t < cnt; ++t) {
      float r = rintf(__fdiv_rn(x[i + t], scale));
      r = fminf(fmaxf(r, -1024.0f), 1024.0f);
      const int v = min(127, max(-128, (int)r + zp));
      packed |= ((unsigned)v & 0xffu) << (8 * t);
   }
   if (cnt == 4 && (reinterpret_cast<uintptr_t>(q + i) & 3u) == 0) {
      *reinterpret_cast<unsigned *>(q + i) = packed;
   } else {
      for (int t = 0; t < cnt; ++t) q[i + t] = (int8_t)(packed >> (8 * t));
   }
}

__global__ void k_dequantize_s8_f32(const int8_t *__restrict__ q, float *__restrict__ x, size_t len, float scale, int zp)
{
   const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   if (i < len) x[i] = __fmul_rn(__int2float_rn((int)q[i] - zp), scale);
}

// fp32 -> e4m3 (OCP), round to nearest even, saturating at +-448; NaN -> 0x7f.
__device__ __forceinline__ unsigned f32_to_e4m3_sat(float x)
{
   const unsigned u = __float_as_uint(x);
   const unsigned sign = (u >> 24) & 0x80u;
   const unsigned a = u & 0x7fffffffu;
   if (a > 0x7f800000u) return 0x7fu;
   const float af = __uint_as_float(a);
   if (af >= 448.0f) return sign | 0x7eu;
   // Scale so that the e4m3 grid becomes the integer grid, round, scale back.
   // Normal range (>= 2^-6): spacing 2^(e-3); subnormal: spacing 2^-9.
   int e = (int)(a >> 23) - 127;
   if (e < -6) e = -6;
   const float step = __uint_as_float((unsigned)(e - 3 + 127) << 23);
   const float q = rintf(__fdiv_rn(af, step));      // exact power-of-two division
   const float r = __fmul_rn(q, step);
   if (r >= 448.0f) return sign | 0x7eu;
   if (r < 0.015625f) return sign | (unsigned)(int)__fmul_rn(r, 512.0f);   // multiples of 2^-9
   const unsigned rb = __float_as_uint(r);
   const unsigned re = (rb >> 23) - 127u + 7u;
   return sign | (re << 3) | ((rb >> 20) & 7u);
}

__global__ void k_quantize_f32_e4m3(const float *__restrict__ x, uint8_t *__restrict__ q, size_t len, float inv_scale)
{
   const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
   if (i < len) q[i] = (uint8_t)f32_to_e4m3_sat(__fmul_rn(x[i], inv_scale));
}

// [N,C,HW] <-> [N,HW,C] through a 64x64 LDS tile so both sides move contiguous bytes.
__global__ void k_transpose_s8(const int8_t *__restrict__ x, int8_t *__restrict__ y, int R, int Ccols)
{
   // x is [batch][R][Ccols], y is [batch][Ccols][R]
   __shared__ int8_t tile[64][65];
   const size_t base = (size_t)blockIdx.z * R * Ccols;
   const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
   for (int i = threadIdx.y; i < 64; i += blockDim.y) {
      const int r = r0 + i, c = c0 + threadIdx.x;
      if (r < R && c < Ccols) tile[i][threadIdx.x] = x[base + (size_t)r * Ccols + c];
   }
   __syncthreads();
   for (int i = threadIdx.y; i < 64; i += blockDim.y) {
      const int c = c0 + i, r = r0 + threadIdx.x;
      if (r < R && c < Ccols) y[base + (size_t)c * R + r] = tile[threadIdx.x][i];
   }
}

inline unsigned blocks_for(size_t n, unsigned per) { return (unsigned)((n + per - 1) / per); }

}  // namespace

namespace sofie {
int relayout_s8(sofie_hip_ctx *ctx, const int8_t *x, int8_t *y, int N, int C, int H, int W, int from, int to)
{
   const size_t len = (size_t)N * C * H * W;
   if (len == 0) return SOFIE_HIP_OK;
   if (from == to) {
      if (x != y) SOFIE_HIP_CALL(ctx, hipMemcpyAsync(y, x, len, hipMemcpyDeviceToDevice, ctx->stream));
      return SOFIE_HIP_OK;
   }
   const int HW = H * W;
   // NCHW -> NHWC: per image transpose [C][HW] -> [HW][C]; the reverse swaps the roles.
   const int R = (from == SOFIE_LAYOUT_NCHW) ? C : HW;
   const int Cc = (from == SOFIE_LAYOUT_NCHW) ? HW : C;
   dim3 grid(cdiv(Cc, 64), cdiv(R, 64), N), block(64, 4);
   hipLaunchKernelGGL(k_transpose_s8, grid, block, 0, ctx->stream, x, y, R, Cc);
   return check_launch(ctx, "k_transpose_s8");
}
}  // namespace sofie

extern "C" {

int sofie_hip_relu_f32(sofie_hip_ctx *ctx, const float *x, float *y, size_t len)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (len == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   if (aligned16(x) && aligned16(y))
      hipLaunchKernelGGL(k_relu_f32, dim3(blocks_for(len, 1024)), dim3(256), 0, ctx->stream, x, y, len);
   else
      hipLaunchKernelGGL(k_relu_f32_scalar, dim3(blocks_for(len, 256)), dim3(256), 0, ctx->stream, x, y, len);
   return check_launch(ctx, "k_relu_f32");
}

int sofie_hip_batchnorm_f32(sofie_hip_ctx *ctx, const float *x, const float *scale, const float *mean, const float *bias,
                            float *y, int N, int C, int plane, int act)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C > 0 && plane > 0, "non-positive dimension");
   SOFIE_REQUIRE(ctx, act == SOFIE_ACT_NONE || act == SOFIE_ACT_RELU, "unknown activation");
   if (N == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && scale && mean && bias && y, "null operand");
   const size_t planes = (size_t)N * C;
   const bool vec = plane % 4 == 0 && aligned16(x) && aligned16(y);
   const int per_block = vec ? 1024 : 256;
   int bx = (plane + per_block - 1) / per_block;
   if (bx > 64) bx = 64;
   // planes ride in blockIdx.y (at most 65535 per launch)
   for (size_t p0 = 0; p0 < planes; p0 += 65535) {
      const unsigned np = (unsigned)((planes - p0) < 65535 ? (planes - p0) : 65535);
      const float *xs = x + p0 * plane;
      float *ys = y + p0 * plane;
      const int c0 = (int)(p0 % (size_t)C);
      if (vec)
         hipLaunchKernelGGL(k_batchnorm_f32<true>, dim3(bx, np), dim3(256), 0, ctx->stream, xs, scale, mean, bias, ys, C, plane,
                            act == SOFIE_ACT_RELU, c0);
      else
         hipLaunchKernelGGL(k_batchnorm_f32<false>, dim3(bx, np), dim3(256), 0, ctx->stream, xs, scale, mean, bias, ys, C, plane,
                            act == SOFIE_ACT_RELU, c0);
   }
   return check_launch(ctx, "k_batchnorm_f32");
}

static int pool_dims(sofie_hip_ctx *ctx, int H, int W, int kh, int kw, int pt, int pl, int pb, int pr, int sh,
                     int sw, int *OH, int *OW)
{
   SOFIE_REQUIRE(ctx, H > 0 && W > 0 && kh > 0 && kw > 0 && sh > 0 && sw > 0, "non-positive dimension");
   SOFIE_REQUIRE(ctx, pt >= 0 && pl >= 0 && pb >= 0 && pr >= 0, "negative padding");
   SOFIE_REQUIRE(ctx, H + pt + pb >= kh && W + pl + pr >= kw, "kernel larger than padded input");
   *OH = (H + pt + pb - kh) / sh + 1;
   *OW = (W + pl + pr - kw) / sw + 1;
   return SOFIE_HIP_OK;
}

int sofie_hip_maxpool2d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, int H, int W, int kh, int kw,
                            int pt, int pl, int pb, int pr, int sh, int sw)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, NC >= 0, "negative dimension");
   if (NC == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   int OH, OW;
   if (int rc = pool_dims(ctx, H, W, kh, kw, pt, pl, pb, pr, sh, sw, &OH, &OW)) return rc;
   const size_t total = (size_t)NC * OH * OW;
   hipLaunchKernelGGL((k_maxpool2d<float, false>), dim3(blocks_for(total, 256)), dim3(256), 0, ctx->stream, x, y, 1,
                      NC, H, W, OH, OW, kh, kw, pt, pl, sh, sw);
   return check_launch(ctx, "k_maxpool2d");
}

int sofie_hip_avgpool2d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, int H, int W, int kh, int kw,
                            int pt, int pl, int pb, int pr, int sh, int sw, int count_include_pad)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, NC >= 0, "negative dimension");
   if (NC == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   int OH, OW;
   if (int rc = pool_dims(ctx, H, W, kh, kw, pt, pl, pb, pr, sh, sw, &OH, &OW)) return rc;
   // a window that lies in the padding entirely would divide by zero cells
   SOFIE_REQUIRE(ctx, count_include_pad || (pt < kh && pl < kw && pb < kh && pr < kw), "a pooling window without a cell of the image");
   const size_t total = (size_t)NC * OH * OW;
   hipLaunchKernelGGL(k_avgpool2d_f32, dim3(blocks_for(total, 256)), dim3(256), 0, ctx->stream, x, y, NC, H, W, OH, OW, kh, kw,
                      pt, pl, sh, sw, count_include_pad != 0);
   return check_launch(ctx, "k_avgpool2d_f32");
}

static int pool3d(sofie_hip_ctx *ctx, bool average, const float *x, float *y, int NC, const int *dims, const int *kernel,
                  const int *pads, const int *strides, int count_include_pad)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, NC >= 0, "negative dimension");
   SOFIE_REQUIRE(ctx, dims && kernel && pads && strides, "null geometry");
   Pool3dArgs a;
   a.NC = NC;
   size_t total = (size_t)NC;
   for (int i = 0; i < 3; ++i) {
      SOFIE_REQUIRE(ctx, dims[i] > 0 && kernel[i] > 0 && strides[i] > 0, "non-positive dimension");
      SOFIE_REQUIRE(ctx, pads[i] >= 0 && pads[3 + i] >= 0, "negative padding");
      SOFIE_REQUIRE(ctx, dims[i] + pads[i] + pads[3 + i] >= kernel[i], "kernel larger than padded input");
      // a window that lies in the padding entirely would divide by zero cells
      SOFIE_REQUIRE(ctx, !average || count_include_pad || (pads[i] < kernel[i] && pads[3 + i] < kernel[i]),
                    "a pooling window without a cell of the volume");
      a.D[i] = dims[i];
      a.k[i] = kernel[i];
      a.pad[i] = pads[i];
      a.s[i] = strides[i];
      a.O[i] = (dims[i] + pads[i] + pads[3 + i] - kernel[i]) / strides[i] + 1;
      total *= (size_t)a.O[i];
   }
   if (NC == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   if (average)
      hipLaunchKernelGGL(k_pool3d_f32<true>, dim3(blocks_for(total, 256)), dim3(256), 0, ctx->stream, x, y, a, count_include_pad != 0);
   else
      hipLaunchKernelGGL(k_pool3d_f32<false>, dim3(blocks_for(total, 256)), dim3(256), 0, ctx->stream, x, y, a, 0);
   return check_launch(ctx, average ? "k_avgpool3d_f32" : "k_maxpool3d_f32");
}

int sofie_hip_maxpool3d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, const int *dims, const int *kernel,
                            const int *pads, const int *strides)
{
   return pool3d(ctx, false, x, y, NC, dims, kernel, pads, strides, 0);
}

int sofie_hip_avgpool3d_f32(sofie_hip_ctx *ctx, const float *x, float *y, int NC, const int *dims, const int *kernel,
                            const int *pads, const int *strides, int count_include_pad)
{
   return pool3d(ctx, true, x, y, NC, dims, kernel, pads, strides, count_include_pad);
}

int sofie_hip_maxpool2d_s8(sofie_hip_ctx *ctx, const int8_t *x, int8_t *y, int layout, int N, int C, int H, int W,
                           int kh, int kw, int pt, int pl, int pb, int pr, int sh, int sw)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C >= 0, "negative dimension");
   SOFIE_REQUIRE(ctx, layout == SOFIE_LAYOUT_NCHW || layout == SOFIE_LAYOUT_NHWC, "unknown layout");
   if (N == 0 || C == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   int OH, OW;
   if (int rc = pool_dims(ctx, H, W, kh, kw, pt, pl, pb, pr, sh, sw, &OH, &OW)) return rc;
   const size_t total = (size_t)N * C * OH * OW;
   if (layout == SOFIE_LAYOUT_NHWC && C % 16 == 0 && aligned16(x) && aligned16(y)) {
      hipLaunchKernelGGL(k_maxpool2d_s8_nhwc16, dim3(blocks_for(total / 16, 256)), dim3(256), 0, ctx->stream, x, y, N, C / 16,
                         H, W, OH, OW, kh, kw, pt, pl, sh, sw);
      return check_launch(ctx, "k_maxpool2d_s8_nhwc16");
   }
   if (layout == SOFIE_LAYOUT_NHWC)
      hipLaunchKernelGGL((k_maxpool2d<int8_t, true>), dim3(blocks_for(total, 256)), dim3(256), 0, ctx->stream, x, y,
                         N, C, H, W, OH, OW, kh, kw, pt, pl, sh, sw);
   else
      hipLaunchKernelGGL((k_maxpool2d<int8_t, false>), dim3(blocks_for(total, 256)), dim3(256), 0, ctx->stream, x, y,
                         N, C, H, W, OH, OW, kh, kw, pt, pl, sh, sw);
   return check_launch(ctx, "k_maxpool2d");
}

int sofie_hip_quantize_f32_s8(sofie_hip_ctx *ctx, const float *x, int8_t *q, size_t len, float scale, int zp)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (len == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && q, "null operand");
   SOFIE_REQUIRE(ctx, scale > 0.0f, "scale must be positive");
   SOFIE_REQUIRE(ctx, zp >= -128 && zp <= 127, "zero-point out of int8 range");
   hipLaunchKernelGGL(k_quantize_f32_s8, dim3(blocks_for(len, 1024)), dim3(256), 0, ctx->stream, x, q, len, scale, zp);
   return check_launch(ctx, "k_quantize_f32_s8");
}

int sofie_hip_dequantize_s8_f32(sofie_hip_ctx *ctx, const int8_t *q, float *x, size_t len, float scale, int zp)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (len == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && q, "null operand");
   SOFIE_REQUIRE(ctx, zp >= -128 && zp <= 127, "zero-point out of int8 range");
   hipLaunchKernelGGL(k_dequantize_s8_f32, dim3(blocks_for(len, 256)), dim3(256), 0, ctx->stream, q, x, len, scale, zp);
   return check_launch(ctx, "k_dequantize_s8_f32");
}

int sofie_hip_quantize_f32_e4m3(sofie_hip_ctx *ctx, const float *x, uint8_t *q, size_t len, float inv_scale)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (len == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && q, "null operand");
   hipLaunchKernelGGL(k_quantize_f32_e4m3, dim3(blocks_for(len, 256)), dim3(256), 0, ctx->stream, x, q, len, inv_scale);
   return check_launch(ctx, "k_quantize_f32_e4m3");
}

int sofie_hip_relayout_s8(sofie_hip_ctx *ctx, const int8_t *x, int8_t *y, int N, int C, int H, int W, int from,
                          int to)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, N >= 0 && C >= 0 && H >= 0 && W >= 0, "negative dimension");
   SOFIE_REQUIRE(ctx, (from == SOFIE_LAYOUT_NCHW || from == SOFIE_LAYOUT_NHWC) &&
                         (to == SOFIE_LAYOUT_NCHW || to == SOFIE_LAYOUT_NHWC), "unknown layout");
   if ((size_t)N * C * H * W == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, x && y, "null operand");
   SOFIE_REQUIRE(ctx, N <= 65535, "batch too large for one launch");
   return sofie::relayout_s8(ctx, x, y, N, C, H, W, from, to);
}

}  // extern "C"
