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
// The columns of S are independent of one another: column j only ever needs k, q, g, beta and v_j, and a token's step
// is a chain of dependent operations over the rows of a column, so what bounds a long segment is the time of one
// step, not the chip's rate. Hence two kernels. The first makes k, q, g and beta of every (token, head) ready, side by
// side for all tokens: unit vectors, decays, written as float32 in the order in which the second reads them, a head's
// tokens one behind the other; and the values as float32 in blocks of 16 columns. The second runs the recurrence with
// a column's rows spread over 16 lanes (RPL = rows a lane holds, in registers; the key size is padded to 16 RPL with
// rows whose k and q are zero), four columns a wave and four waves a workgroup: a step is RPL multiplications and
// 3 RPL multiply-adds a lane and two reductions over 16 lanes. What the steps read travels from global memory
// straight into LDS a batch of tokens ahead (two buffers; the operands do not depend on S, so a whole batch of
// steps covers the way from memory; with the operands asked for four tokens ahead into registers a step took 0.66 us,
// nearly all of it waiting). Tokens of a request run one after the other; (request, head, 16 columns) side by side.
// The state lies as [H, ceil(vdim / 4), dim, 4], so that a wave's part of it is one piece of memory; a step of single
// tokens is the same kernels, bound by the memory's bytes: S in and out.
//
// A third kernel divides every head's o by its root mean square, multiplies by a weight over vdim (shared by the
// heads) and by sigmoid or silu of a gate, and rounds to the run's type.
#include "common.h"

#include <math.h>

#define DELTA_R 16            // lanes that share a column
#define DELTA_CPW 4           // columns a wave holds
#define DELTA_WAVES 4         // waves a workgroup
#define DELTA_COLS (DELTA_CPW * DELTA_WAVES)

__device__ __forceinline__ float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

static inline int delta_rows_per_lane(int dim) { return dim <= 16 ? 1 : dim <= 32 ? 2 : dim <= 64 ? 4 : dim <= 128 ? 8 : 16; }
// tokens a batch holds, and the floats of a (token, head)'s operands: k, q, g in the lanes' order, then beta and padding
static inline int delta_batch_tokens(int rpl) { return 2048 / (DELTA_R * rpl); }
static inline int delta_block_floats(int rpl) { return 3 * DELTA_R * rpl + 4; }

// prep [H, N + batch, block] float32: k, q, g of every (token, head), entry p = r * RPL + ii holding row ii * 16 + r,
// then beta; vals [H, ceil(vdim / 16), N + batch, 16]: the values. A wave a (token, head).
template <typename T>
__global__ __launch_bounds__(256) void gated_delta_prepare_kernel(
    const T* __restrict__ qkv, long stride, int q_at, int k_at, int v_at, const float* __restrict__ a, long a_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ b, long b_stride,
    float* __restrict__ prep, float* __restrict__ vals, int n_tokens, long rows, int H, int G, int dim, int vdim,
    int RPL, float q_scale, float unit_eps) {
  const long w = (long)blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE;
  const int lane = threadIdx.x % LMSF_WAVE;
  if (w >= (long)n_tokens * H) return;
  const long t = w / H;
  const int h = (int)(w - t * H), gh = h / (H / G), DP = DELTA_R * RPL, block = 3 * DP + 4;
  const T* qr = qkv + t * stride + q_at + gh * dim;
  const T* kr = qkv + t * stride + k_at + gh * dim;
  float ssq = 0.f, ssk = 0.f;
  for (int i = lane; i < dim; i += LMSF_WAVE) {
    const float x = to_f32<T>(qr[i]), y = to_f32<T>(kr[i]);
    ssq += x * x;
    ssk += y * y;
  }
  const float iq = q_scale / sqrtf(wave_sum(ssq) + unit_eps), ik = 1.f / sqrtf(wave_sum(ssk) + unit_eps);
  const float rate = expf(a_log[h]);
  float* out = prep + ((long)h * rows + t) * block;
  for (int p = lane; p < DP; p += LMSF_WAVE) {
    const int i = (p % RPL) * DELTA_R + p / RPL;
    float kk = 0.f, kq = 0.f, g = 1.f;
    if (i < dim) {
      kk = to_f32<T>(kr[i]) * ik;
      kq = to_f32<T>(qr[i]) * iq;
      g = expf(-rate * softplus_f32(a[t * a_stride + h * dim + i] + dt_bias[h * dim + i]));
    }
    out[p] = kk;
    out[DP + p] = kq;
    out[2 * DP + p] = g;
  }
  if (lane < 4) out[3 * DP + lane] = lane == 0 ? 1.f / (1.f + expf(-b[t * b_stride + h])) : 0.f;
  const int n_cb = (vdim + DELTA_COLS - 1) / DELTA_COLS;
  const T* vr = qkv + t * stride + v_at + h * vdim;
  for (int j = lane; j < n_cb * DELTA_COLS; j += LMSF_WAVE)
    vals[(((long)h * n_cb + j / DELTA_COLS) * rows + t) * DELTA_COLS + j % DELTA_COLS] = j < vdim ? to_f32<T>(vr[j]) : 0.f;
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 is named as clobbered on purpose
// lane i's 16 bytes go from ``src`` to LDS address lds_base_uniform + 16 i (global_load_lds_dwordx4)
__device__ __forceinline__ void delta_global_to_lds_16(const void* src, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base_uniform)
               : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ unsigned delta_lds_address(const void* p) {
  return (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)p;
}

template <int RPL>
__device__ __forceinline__ void delta_load_vec(float* dst, const float* src) {
  if constexpr (RPL >= 4) {
#pragma unroll
    for (int j = 0; j < RPL / 4; ++j) {
      const float4 x = *reinterpret_cast<const float4*>(src + 4 * j);
      dst[4 * j] = x.x; dst[4 * j + 1] = x.y; dst[4 * j + 2] = x.z; dst[4 * j + 3] = x.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < RPL; ++j) dst[j] = src[j];
  }
}

__device__ __forceinline__ float delta_sum16(float v) {
  v += __shfl_xor(v, 8, LMSF_WAVE);
  v += __shfl_xor(v, 4, LMSF_WAVE);
  v += __shfl_xor(v, 2, LMSF_WAVE);
  v += __shfl_xor(v, 1, LMSF_WAVE);
  return v;
}

template <int RPL>
__global__ __launch_bounds__(DELTA_WAVES * LMSF_WAVE) void gated_delta_recurrence_kernel(
    const float* __restrict__ prep, const float* __restrict__ vals, long rows, float* __restrict__ state,
    long state_stride, const int* __restrict__ seg_starts, const int* __restrict__ slots, float* __restrict__ out,
    long out_stride, int H, int dim, int vdim) {
  constexpr int DP = DELTA_R * RPL, BLOCK = 3 * DP + 4, HT = 2048 / DP;
  constexpr int OPS_BYTES = (HT * BLOCK * 4 + 1023) / 1024 * 1024, VAL_BYTES = (HT * DELTA_COLS * 4 + 1023) / 1024 * 1024;
  constexpr int N_OPS = OPS_BYTES / 1024, N_VAL = VAL_BYTES / 1024;     // transfers of 1 KB a batch
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // two buffers of [operands | values]
  const int s = blockIdx.x, h = blockIdx.y, cb = blockIdx.z;
  const int tid = threadIdx.x, wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE, c = lane / DELTA_R, r = lane % DELTA_R;
  const int col = cb * DELTA_COLS + wave * DELTA_CPW + c;
  const bool col_ok = col < vdim;
  const int t0 = seg_starts[s], t1 = seg_starts[s + 1];
  if (t1 <= t0) return;
  const int n_cb4 = (vdim + DELTA_CPW - 1) / DELTA_CPW, n_cb = (vdim + DELTA_COLS - 1) / DELTA_COLS;
  const int cb4 = cb * DELTA_WAVES + wave;
  const bool wave_ok = cb4 < n_cb4;                 // (a wave whose columns all lie beyond vdim keeps no state)
  float* S = state + (long)slots[s] * state_stride + ((long)h * n_cb4 + cb4) * dim * DELTA_CPW;
  float st[RPL];
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = ii * DELTA_R + r;
    st[ii] = (wave_ok && i < dim) ? S[i * DELTA_CPW + c] : 0.f;
  }
  const unsigned char* g_ops = reinterpret_cast<const unsigned char*>(prep + (long)h * rows * BLOCK);
  const unsigned char* g_val = reinterpret_cast<const unsigned char*>(vals + ((long)h * n_cb + cb) * rows * DELTA_COLS);
  const unsigned lds0 = delta_lds_address(lds);
  auto transfer = [&](int tb, int buf) {
    const unsigned base = lds0 + buf * (OPS_BYTES + VAL_BYTES);
    const int first = __builtin_amdgcn_readfirstlane(wave);          // (the same in every lane: the LDS base is a scalar)
    for (int n = first; n < N_OPS; n += DELTA_WAVES)
      delta_global_to_lds_16(g_ops + (long)tb * BLOCK * 4 + n * 1024 + lane * 16,
                             __builtin_amdgcn_readfirstlane(base + n * 1024));
    for (int n = first; n < N_VAL; n += DELTA_WAVES)
      delta_global_to_lds_16(g_val + (long)tb * DELTA_COLS * 4 + n * 1024 + lane * 16,
                             __builtin_amdgcn_readfirstlane(base + OPS_BYTES + n * 1024));
  };
  transfer(t0, 0);
  int buf = 0;
  for (int tb = t0; tb < t1; tb += HT, buf ^= 1) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                   // this batch has landed; everybody is done with the buffer of the one before
    if (tb + HT < t1) transfer(tb + HT, buf ^ 1);
    const float* ops_ = reinterpret_cast<const float*>(lds + buf * (OPS_BYTES + VAL_BYTES));
    const float* val_ = reinterpret_cast<const float*>(lds + buf * (OPS_BYTES + VAL_BYTES) + OPS_BYTES);
    const int nt = min(HT, t1 - tb);
    for (int j = 0; j < nt; ++j) {
      const float* blk = ops_ + j * BLOCK;
      float k[RPL], q[RPL], g[RPL];
      delta_load_vec<RPL>(k, blk + r * RPL);
      delta_load_vec<RPL>(q, blk + DP + r * RPL);
      delta_load_vec<RPL>(g, blk + 2 * DP + r * RPL);
      const float beta = blk[3 * DP], v = val_[j * DELTA_COLS + wave * DELTA_CPW + c];
      float dot = 0.f;
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) {
        st[ii] *= g[ii];
        dot = fmaf(k[ii], st[ii], dot);
      }
      dot = delta_sum16(dot);
      const float u = beta * (v - dot);
      float o = 0.f;
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) {
        st[ii] = fmaf(k[ii], u, st[ii]);
        o = fmaf(q[ii], st[ii], o);
      }
      o = delta_sum16(o);
      if (r == 0 && col_ok) out[(long)(tb + j) * out_stride + h * vdim + col] = o;
    }
  }
  if (wave_ok) {
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) {
      const int i = ii * DELTA_R + r;
      if (i < dim) S[i * DELTA_CPW + c] = st[ii];
    }
  }
}

// floats of a request's memory: [H, ceil(vdim / 4), dim, 4]
extern "C" long lmsf_gated_delta_state_floats(int H, int dim, int vdim) {
  return (long)H * ((vdim + DELTA_CPW - 1) / DELTA_CPW) * dim * DELTA_CPW;
}

// floats of scratch for n_tokens tokens: what the first kernel hands the second (a batch of rows more per head than
// there are tokens, and a transfer's length at the end, so that a batch may be fetched whole wherever it begins)
extern "C" long lmsf_gated_delta_scratch_floats(int n_tokens, int H, int dim, int vdim) {
  const int rpl = delta_rows_per_lane(dim);
  const long rows = (long)n_tokens + delta_batch_tokens(rpl);
  const long n_cb = (vdim + DELTA_COLS - 1) / DELTA_COLS;
  return (long)H * rows * delta_block_floats(rpl) + 256 + (long)H * n_cb * rows * DELTA_COLS + 256;
}

template <int RPL>
static int launch_delta_recurrence(dim3 grid, hipStream_t stream, const float* prep, const float* vals, long rows,
                                   float* state, long state_stride, const int* seg_starts, const int* slots, float* out,
                                   long out_stride, int H, int dim, int vdim) {
  constexpr int DP = DELTA_R * RPL, BLOCK = 3 * DP + 4, HT = 2048 / DP;
  constexpr size_t smem = 2 * ((size_t)(HT * BLOCK * 4 + 1023) / 1024 * 1024 + (size_t)(HT * DELTA_COLS * 4 + 1023) / 1024 * 1024);
  auto kernel = gated_delta_recurrence_kernel<RPL>;
  static bool configured = false;   // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("gated_delta: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(DELTA_WAVES * LMSF_WAVE), smem, stream, prep, vals, rows, state, state_stride,
                     seg_starts, slots, out, out_stride, H, dim, vdim);
  return 0;
}

// qkv: the (convolved, activated) q [N, G dim], k [N, G dim], v [N, H vdim] as columns q_at, k_at, v_at of one buffer
// of ``dtype`` with row stride ``stride``; a: float32 [N, H dim] before bias and softplus; dt_bias float32 [H dim];
// a_log float32 [H]; b: float32 [N, >= H] before the sigmoid; state float32 [slots, >= lmsf_gated_delta_state_floats];
// scratch: lmsf_gated_delta_scratch_floats floats, 16-byte aligned; out: float32 [N, H vdim], the heads' read-outs as
// they are.
extern "C" int lmsf_gated_delta(const void* qkv, int dtype, long stride, int q_at, int k_at, int v_at, const float* a,
                                long a_stride, const float* dt_bias, const float* a_log, const float* b,
                                long b_stride, float* state, long state_stride, const int* seg_starts,
                                const int* slots, float* scratch, float* out, long out_stride, int n_tokens,
                                int n_segments, int H, int G, int dim, int vdim, float q_scale, float unit_eps,
                                hipStream_t stream) {
  LMSF_CHECK(qkv && a && dt_bias && a_log && b && state && seg_starts && slots && out && scratch,
             "gated_delta: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "gated_delta: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && dim <= 256 && vdim > 0,
             "gated_delta: heads %d over %d key heads, keys of %d (at most 256) and values of %d entries", H, G, dim, vdim);
  const int n_cb = (vdim + DELTA_COLS - 1) / DELTA_COLS;
  LMSF_CHECK(H <= 65535 && n_cb <= 65535, "gated_delta: too many heads or columns");
  LMSF_CHECK(a_stride >= (long)H * dim && b_stride >= H && out_stride >= (long)H * vdim &&
                 state_stride >= lmsf_gated_delta_state_floats(H, dim, vdim) && q_at >= 0 && k_at >= 0 && v_at >= 0,
             "gated_delta: strides too small");
  LMSF_CHECK(lmsf_aligned16(scratch), "gated_delta: the scratch must be 16-byte aligned");
  if (n_tokens <= 0 || n_segments <= 0) return 0;
  const int RPL = delta_rows_per_lane(dim);
  const long rows = (long)n_tokens + delta_batch_tokens(RPL);
  float* prep = scratch;
  float* vals = scratch + (long)H * rows * delta_block_floats(RPL) + 256;
  const dim3 g1((unsigned)(((long)n_tokens * H + 3) / 4)), g2(n_segments, H, n_cb);
#define DELTA_PREP(T)                                                                                               \
  hipLaunchKernelGGL((gated_delta_prepare_kernel<T>), g1, dim3(256), 0, stream, (const T*)qkv, stride, q_at, k_at,   \
                     v_at, a, a_stride, dt_bias, a_log, b, b_stride, prep, vals, n_tokens, rows, H, G, dim, vdim, RPL, \
                     q_scale, unit_eps)
  if (dtype == LMSF_F32) DELTA_PREP(float);
  else DELTA_PREP(bf16_t);
#undef DELTA_PREP
#define DELTA_RUN(R)                                                                                              \
  launch_delta_recurrence<R>(g2, stream, prep, vals, rows, state, state_stride, seg_starts, slots, out, out_stride, \
                             H, dim, vdim)
  const int rc = RPL == 1 ? DELTA_RUN(1) : RPL == 2 ? DELTA_RUN(2) : RPL == 4 ? DELTA_RUN(4) : RPL == 8 ? DELTA_RUN(8)
                                                                                                       : DELTA_RUN(16);
#undef DELTA_RUN
  if (rc) return rc;
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
