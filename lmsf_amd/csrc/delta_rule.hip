// The gated delta rule with one decay per head and key channel, a matrix memory S [dim, vdim] per head and request:
//
//   S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
//
// (the read-out sees the token's own write). What enters the recurrence is made here, in float32, from the
// projections' results: q and k are made unit vectors per head, x / sqrt(sum x^2 + unit_eps), q times q_scale;
// beta = sigmoid(b); g = exp(-exp(A_log_h) softplus(a + dt_bias)), one factor per head and key channel, acting on the
// rows of S. H value heads and G query/key heads (head h reads q/k head h / (H / G)). S lives in the request's state
// slot, float32 [H, dim, vdim], and is read once and written once a step.
//
// The columns of S are independent of one another: column j only ever needs k, q, g, beta and v_j. A wave holds 16
// columns, each spread over four lanes that keep a quarter of its rows each in registers (RPL rows a
// lane; dim is padded to 4 RPL with rows whose k and q are zero), and two shuffles add the four partial dot
// products; a workgroup of four waves shares what it makes of k, q and g for eight tokens at a time in LDS. Tokens of
// a request run one after the other; (request, head, 64 columns) side by side. A step of single tokens is the same
// kernel with one token a workgroup, bound by the memory's bytes: S in and out.
//
// A second kernel divides every head's o by its root mean square, multiplies by a weight over vdim (shared by the
// heads) and by sigmoid or silu of a gate, and rounds to the run's type.
#include "common.h"

#include <math.h>

#define DELTA_TB 8            // tokens made ready at a time
#define DELTA_COLS 64         // value columns a workgroup holds

__device__ __forceinline__ float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <typename T, int RPL>
__global__ __launch_bounds__(256) void gated_delta_kernel(
    const T* __restrict__ qkv, long stride, int q_at, int k_at, int v_at, const float* __restrict__ a, long a_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ b, long b_stride,
    float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts, const int* __restrict__ slots,
    float* __restrict__ out, long out_stride, int H, int G, int dim, int vdim, float q_scale, float unit_eps) {
  constexpr int PAD = RPL == 8 ? 0 : 8;
  constexpr int LD = 4 * (RPL + PAD);             // floats of one staged vector
  __shared__ __attribute__((aligned(16))) float sk[DELTA_TB][LD], sq[DELTA_TB][LD], sg[DELTA_TB][LD];
  __shared__ float sv[DELTA_TB][DELTA_COLS], sbeta[DELTA_TB];
  const int s = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * DELTA_COLS;
  const int tid = threadIdx.x, wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE;
  const int r = lane / 16, col = c0 + wave * 16 + lane % 16;
  const bool col_ok = col < vdim;
  const int t0 = seg_starts[s], t1 = seg_starts[s + 1];
  if (t1 <= t0) return;
  const int gh = h / (H / G);
  float* S = state + (long)slots[s] * state_stride + (long)h * dim * vdim;
  float st[RPL];
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = r * RPL + ii;
    st[ii] = (col_ok && i < dim) ? S[(long)i * vdim + col] : 0.f;
  }
  const float decay_rate = expf(a_log[h]);
  const int dim_pad = 4 * RPL;
  for (int tb = t0; tb < t1; tb += DELTA_TB) {
    const int nt = min(DELTA_TB, t1 - tb);
    __syncthreads();                                // the batch before has been read
    // 32 threads a token: unit vectors, decays
    {
      const int j = tid / 32, l = tid % 32;
      if (j < nt) {
        const long t = tb + j;
        const T* qr = qkv + t * stride + q_at + gh * dim;
        const T* kr = qkv + t * stride + k_at + gh * dim;
        float ssq = 0.f, ssk = 0.f;
        for (int i = l; i < dim; i += 32) {
          const float x = to_f32<T>(qr[i]), y = to_f32<T>(kr[i]);
          ssq += x * x;
          ssk += y * y;
        }
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) {
          ssq += __shfl_xor(ssq, o, LMSF_WAVE);
          ssk += __shfl_xor(ssk, o, LMSF_WAVE);
        }
        const float iq = q_scale / sqrtf(ssq + unit_eps), ik = 1.f / sqrtf(ssk + unit_eps);
        for (int i = l; i < dim_pad; i += 32) {
          const int at = (i / RPL) * (RPL + PAD) + i % RPL;
          float kq = 0.f, kk = 0.f, g = 1.f;
          if (i < dim) {
            kq = to_f32<T>(qr[i]) * iq;
            kk = to_f32<T>(kr[i]) * ik;
            g = expf(-decay_rate * softplus_f32(a[t * a_stride + h * dim + i] + dt_bias[h * dim + i]));
          }
          sq[j][at] = kq;
          sk[j][at] = kk;
          sg[j][at] = g;
        }
        if (l == 0) sbeta[j] = 1.f / (1.f + expf(-b[t * b_stride + h]));
      }
      for (int e = tid; e < nt * DELTA_COLS; e += 256) {
        const int jj = e / DELTA_COLS, c = e % DELTA_COLS;
        sv[jj][c] = c0 + c < vdim ? to_f32<T>(qkv[(long)(tb + jj) * stride + v_at + h * vdim + c0 + c]) : 0.f;
      }
    }
    __syncthreads();
    for (int j = 0; j < nt; ++j) {
      const float* pk = &sk[j][r * (RPL + PAD)];
      const float* pq = &sq[j][r * (RPL + PAD)];
      const float* pg = &sg[j][r * (RPL + PAD)];
      float dot = 0.f;
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) {
        st[ii] *= pg[ii];
        dot = fmaf(pk[ii], st[ii], dot);
      }
      dot += __shfl_xor(dot, 16, LMSF_WAVE);
      dot += __shfl_xor(dot, 32, LMSF_WAVE);
      const float u = sbeta[j] * (sv[j][wave * 16 + lane % 16] - dot);
      float o = 0.f;
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) {
        st[ii] = fmaf(pk[ii], u, st[ii]);
        o = fmaf(pq[ii], st[ii], o);
      }
      o += __shfl_xor(o, 16, LMSF_WAVE);
      o += __shfl_xor(o, 32, LMSF_WAVE);
      if (r == 0 && col_ok) out[(long)(tb + j) * out_stride + h * vdim + col] = o;
    }
  }
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = r * RPL + ii;
    if (col_ok && i < dim) S[(long)i * vdim + col] = st[ii];
  }
}

extern "C" long lmsf_gated_delta_state_floats(int H, int dim, int vdim) { return (long)H * dim * vdim; }

// qkv: the (convolved, activated) q [N, G dim], k [N, G dim], v [N, H vdim] as columns q_at, k_at, v_at of one buffer
// of ``dtype`` with row stride ``stride``; a: float32 [N, H dim] before bias and softplus; dt_bias float32 [H dim];
// a_log float32 [H]; b: float32 [N, >= H] before the sigmoid; state float32 [slots, >= H dim vdim]; out: float32
// [N, H vdim], the heads' read-outs as they are.
extern "C" int lmsf_gated_delta(const void* qkv, int dtype, long stride, int q_at, int k_at, int v_at, const float* a,
                                long a_stride, const float* dt_bias, const float* a_log, const float* b,
                                long b_stride, float* state, long state_stride, const int* seg_starts,
                                const int* slots, float* out, long out_stride, int n_tokens, int n_segments, int H,
                                int G, int dim, int vdim, float q_scale, float unit_eps, hipStream_t stream) {
  LMSF_CHECK(qkv && a && dt_bias && a_log && b && state && seg_starts && slots && out, "gated_delta: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "gated_delta: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && dim <= 256 && vdim > 0,
             "gated_delta: heads %d over %d key heads, keys of %d (at most 256) and values of %d entries", H, G, dim, vdim);
  LMSF_CHECK(H <= 65535 && (vdim + DELTA_COLS - 1) / DELTA_COLS <= 65535, "gated_delta: too many heads or columns");
  LMSF_CHECK(a_stride >= (long)H * dim && b_stride >= H && out_stride >= (long)H * vdim &&
                 state_stride >= (long)H * dim * vdim && q_at >= 0 && k_at >= 0 && v_at >= 0,
             "gated_delta: strides too small");
  if (n_tokens <= 0 || n_segments <= 0) return 0;
  const dim3 grid(n_segments, H, (vdim + DELTA_COLS - 1) / DELTA_COLS);
#define DELTA_LAUNCH(T, R)                                                                                          \
  hipLaunchKernelGGL((gated_delta_kernel<T, R>), grid, dim3(256), 0, stream, (const T*)qkv, stride, q_at, k_at, v_at, \
                     a, a_stride, dt_bias, a_log, b, b_stride, state, state_stride, seg_starts, slots, out,         \
                     out_stride, H, G, dim, vdim, q_scale, unit_eps)
#define DELTA_PICK(T)                         \
  do {                                        \
    if (dim <= 32) DELTA_LAUNCH(T, 8);        \
    else if (dim <= 64) DELTA_LAUNCH(T, 16);  \
    else if (dim <= 128) DELTA_LAUNCH(T, 32); \
    else DELTA_LAUNCH(T, 64);                 \
  } while (0)
  if (dtype == LMSF_F32) DELTA_PICK(float);
  else DELTA_PICK(bf16_t);
#undef DELTA_PICK
#undef DELTA_LAUNCH
  LMSF_LAUNCH_CHECK("gated_delta");
  return 0;
}

// ---------------------------------------------------------------- the heads' norm and gate

// out[n, h, :] = raw[n, h, :] / sqrt(mean(raw[n, h, :]^2) + eps) * w[:] * act(gate[n, h, :]); act: 0 none, 1 sigmoid,
// 2 silu. A wave a (token, head).
template <typename T>
__global__ __launch_bounds__(256) void head_rms_gate_kernel(const float* __restrict__ raw, long raw_stride,
                                                            const float* __restrict__ w, const T* __restrict__ gate,
                                                            long gate_stride, int act, T* __restrict__ out,
                                                            long out_stride, int n_tokens, int H, int vdim, float eps) {
  const long wv = (long)blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE;
  const int lane = threadIdx.x % LMSF_WAVE;
  if (wv >= (long)n_tokens * H) return;
  const int t = (int)(wv / H), h = (int)(wv - (long)t * H);
  const float* x = raw + (long)t * raw_stride + (long)h * vdim;
  float s = 0.f;
  for (int i = lane; i < vdim; i += LMSF_WAVE) s += x[i] * x[i];
  const float inv = 1.f / sqrtf(wave_sum(s) / (float)vdim + eps);
  for (int i = lane; i < vdim; i += LMSF_WAVE) {
    float y = x[i] * inv;
    if (w) y *= w[i];
    if (act) {
      const float g = to_f32<T>(gate[(long)t * gate_stride + (long)h * vdim + i]);
      const float sg = 1.f / (1.f + expf(-g));
      y *= act == 1 ? sg : g * sg;
    }
    out[(long)t * out_stride + (long)h * vdim + i] = from_f32<T>(y);
  }
}

extern "C" int lmsf_head_rms_gate(const float* raw, long raw_stride, const float* w, const void* gate,
                                  long gate_stride, int act, void* out, long out_stride, int dtype, int n_tokens,
                                  int H, int vdim, float eps, hipStream_t stream) {
  LMSF_CHECK(raw && out && (act == 0 || gate), "head_rms_gate: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "head_rms_gate: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && vdim > 0 && act >= 0 && act <= 2 && raw_stride >= (long)H * vdim &&
                 out_stride >= (long)H * vdim && (!gate || gate_stride >= (long)H * vdim), "head_rms_gate: bad sizes");
  if (n_tokens <= 0) return 0;
  const dim3 grid((unsigned)(((long)n_tokens * H + 3) / 4));
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((head_rms_gate_kernel<float>), grid, dim3(256), 0, stream, raw, raw_stride, w,
                       (const float*)gate, gate_stride, act, (float*)out, out_stride, n_tokens, H, vdim, eps);
  else
    hipLaunchKernelGGL((head_rms_gate_kernel<bf16_t>), grid, dim3(256), 0, stream, raw, raw_stride, w,
                       (const bf16_t*)gate, gate_stride, act, (bf16_t*)out, out_stride, n_tokens, H, vdim, eps);
  LMSF_LAUNCH_CHECK("head_rms_gate");
  return 0;
}
