// Two sublayers side by side on one norm, each result scaled entry by entry before it joins the stream:
//     stream += s_a * a + s_b * b          (b and s_b may be missing)
// and, from the same launch, the RMS norm of the new stream for the layer that follows (weight ``wn``; missing: no
// norm is written). The stream, the scales, the sum and the norm's statistic are float32; a, b and the norm's result
// are float32 or bfloat16. A workgroup a row: the new row is kept in LDS between the sum and the norm. Where the
// width and the rows' distances are multiples of four (and the rows begin at multiples of 16 bytes) a thread takes
// four neighbours at a time.
// Also: the scale and soft cap of logits, y = cap tanh(x * scale / cap) (cap 0: y = x * scale), in place.
// The reference's block has one residual addition per sublayer, done by the norm that follows
// (vllm/kernels/layernorm_kernels.cu:41-68), and no scales.
#include "common.h"
#include "entry_points.h"

#include <math.h>

#define LS_THREADS 256

__device__ __forceinline__ void ls_load4(const float* p, float* x) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  x[0] = v.x, x[1] = v.y, x[2] = v.z, x[3] = v.w;
}
__device__ __forceinline__ void ls_load4(const bf16_t* p, float* x) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  x[0] = __uint_as_float(v.x << 16), x[1] = __uint_as_float(v.x & 0xffff0000u);
  x[2] = __uint_as_float(v.y << 16), x[3] = __uint_as_float(v.y & 0xffff0000u);
}
__device__ __forceinline__ void ls_store4(float* p, const float* x) {
  *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
}
__device__ __forceinline__ void ls_store4(bf16_t* p, const float* x) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(x[0], x[1]), pack2_bf16(x[2], x[3]));
}

// four neighbours a thread; W, a_stride and b_stride multiples of 4, every pointer a multiple of 16 bytes
template <typename T, typename TW>
__global__ __launch_bounds__(LS_THREADS) void scale_add_norm_vec_kernel(
    const T* __restrict__ a, long a_stride, const float* __restrict__ sa, const T* __restrict__ b, long b_stride,
    const float* __restrict__ sb, float* __restrict__ stream, const TW* __restrict__ wn, T* __restrict__ out, int W,
    float eps) {
  extern __shared__ float row[];      // [W] (+ 16 for the reduction)
  float* red = row + W;
  const long n = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x * 4; i < W; i += LS_THREADS * 4) {
    float r[4], x[4], s[4];
    ls_load4(stream + n * W + i, r);
    ls_load4(a + n * a_stride + i, x);
    ls_load4(sa + i, s);
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] += s[j] * x[j];
    if (b) {
      ls_load4(b + n * b_stride + i, x);
      ls_load4(sb + i, s);
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] += s[j] * x[j];
    }
    ls_store4(stream + n * W + i, r);
    ls_store4(row + i, r);
#pragma unroll
    for (int j = 0; j < 4; ++j) ss += r[j] * r[j];
  }
  if (!wn) return;
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x * 4; i < W; i += LS_THREADS * 4) {
    float r[4], w[4];
    ls_load4(row + i, r);
    ls_load4(wn + i, w);
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = r[j] * inv * w[j];
    ls_store4(out + n * W + i, r);
  }
}

template <typename T, typename TW>
__global__ __launch_bounds__(LS_THREADS) void scale_add_norm_kernel(
    const T* __restrict__ a, long a_stride, const float* __restrict__ sa, const T* __restrict__ b, long b_stride,
    const float* __restrict__ sb, float* __restrict__ stream, const TW* __restrict__ wn, T* __restrict__ out, int W,
    float eps) {
  extern __shared__ float row[];      // [W] (+ 16 for the reduction)
  float* red = row + W;
  const long n = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += LS_THREADS) {
    float r = stream[n * W + i] + sa[i] * to_f32<T>(a[n * a_stride + i]);
    if (b) r += sb[i] * to_f32<T>(b[n * b_stride + i]);
    stream[n * W + i] = r;
    row[i] = r;
    ss += r * r;
  }
  if (!wn) return;
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += LS_THREADS) out[n * W + i] = from_f32<T>(row[i] * inv * to_f32<TW>(wn[i]));
}

// a, b: [N, W] of ``dtype`` with unit column stride; sa, sb float32 [W]; stream contiguous float32 [N, W];
// wn [W] of ``wn_dtype`` or null; out contiguous [N, W] of ``dtype`` (ignored without wn).
extern "C" int lmsf_scale_add_norm(const void* a, long a_stride, const float* sa, const void* b, long b_stride,
                                   const float* sb, int dtype, float* stream, const void* wn, int wn_dtype, void* out,
                                   int n_rows, int W, float eps, hipStream_t stream_) {
  LMSF_CHECK(a && sa && stream && (!b || sb) && (!wn || out), "scale_add_norm: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "scale_add_norm: unknown dtype code %d", dtype);
  LMSF_CHECK(wn_dtype == LMSF_F32 || wn_dtype == LMSF_BF16, "scale_add_norm: unknown dtype code %d", wn_dtype);
  LMSF_CHECK(W > 0 && (size_t)(W + 16) * 4 <= 64 * 1024 && a_stride >= W && (!b || b_stride >= W),
             "scale_add_norm: bad sizes");
  if (n_rows <= 0) return 0;
  const size_t smem = (size_t)(W + 16) * 4;
  const bool vec = W % 4 == 0 && a_stride % 4 == 0 && (!b || b_stride % 4 == 0) && lmsf_aligned16(a) &&
                   lmsf_aligned16(sa) && lmsf_aligned16(b) && lmsf_aligned16(sb) && lmsf_aligned16(stream) &&
                   lmsf_aligned16(wn) && lmsf_aligned16(out);
#define LS_GO(T, TW)                                                                                                  \
  do {                                                                                                                \
    if (vec)                                                                                                          \
      hipLaunchKernelGGL((scale_add_norm_vec_kernel<T, TW>), dim3(n_rows), dim3(LS_THREADS), smem, stream_,           \
                         (const T*)a, a_stride, sa, (const T*)b, b_stride, sb, stream, (const TW*)wn, (T*)out, W,     \
                         eps);                                                                                        \
    else                                                                                                              \
      hipLaunchKernelGGL((scale_add_norm_kernel<T, TW>), dim3(n_rows), dim3(LS_THREADS), smem, stream_, (const T*)a,  \
                         a_stride, sa, (const T*)b, b_stride, sb, stream, (const TW*)wn, (T*)out, W, eps);            \
  } while (0)
  if (dtype == LMSF_F32) {
    if (wn_dtype == LMSF_F32) LS_GO(float, float); else LS_GO(float, bf16_t);
  } else {
    if (wn_dtype == LMSF_F32) LS_GO(bf16_t, float); else LS_GO(bf16_t, bf16_t);
  }
#undef LS_GO
  LMSF_LAUNCH_CHECK("scale_add_norm");
  return 0;
}

__global__ __launch_bounds__(256) void logit_cap_kernel(float* __restrict__ x, long stride, int V, float scale,
                                                        float cap) {
  float* row = x + (long)blockIdx.y * stride;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= V) return;
  const float y = row[i] * scale;
  row[i] = cap > 0.f ? cap * tanhf(y / cap) : y;
}

// float32 logits [R, V] (rows ``stride`` apart), in place
extern "C" int lmsf_logit_cap(float* logits, long stride, int R, int V, float scale, float cap, hipStream_t stream) {
  LMSF_CHECK(logits && V > 0 && stride >= V && R <= 65535, "logit_cap: bad arguments");
  if (R <= 0) return 0;
  hipLaunchKernelGGL(logit_cap_kernel, dim3((V + 255) / 256, R), dim3(256), 0, stream, logits, stride, V, scale, cap);
  LMSF_LAUNCH_CHECK("logit_cap");
  return 0;
}
