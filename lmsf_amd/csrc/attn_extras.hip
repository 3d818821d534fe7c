// Queries, keys and values made ready for the paged attention kernels, and the heads made ready for the output
// projection, for attention layers with norms and rotations beyond the plain ones. Every step is optional:
//
// before attention, per token:
//   q <- q / sqrt(mean over all H dim entries of q^2 + eps) * wq   (one norm over the whole projection; wq null: none)
//   k likewise over its G dim entries with wk
//   q, k: the first ``rot`` entries of every head turned by the position (table [max_pos, rot] = [cos | sin])
//   v <- v / sqrt(mean over the head's vdim entries of v^2 + eps)   (``v_norm``; no weight)
//   v: all vdim entries turned by the position (table_v [max_pos, vdim]; null: not)
//   q goes to q_out [N, H D] (zeros behind dim), k and v into their pages (V transposed, zeros behind dim / vdim)
// after attention, per token and head:
//   o: all vdim entries turned back by the position (table_v), times sigmoid(gate[n, h]) (one number a head; null:
//   none), the first vdim of the D entries to out [N, H vdim].
// Pairs are (2m, 2m + 1) if ``interleaved`` else (m, m + rot / 2). A value turned by its own position j and the sum
// turned back by the query's position i leaves every value turned by j - i: a position encoding on the values.
// All arithmetic is float32, the tables are made in float64 on the host; results are rounded once, as stored.
#include "common.h"

#include <math.h>

#define PREP_THREADS 256

// entries (i0, i1) of pair slot ``pi`` of a head of ``dim`` entries of which the first ``rot`` are rotated; *m: the
// pair's index in the table, or -1 for a slot that is not rotated
__device__ __forceinline__ void pair_slot(int pi, int rot, int interleaved, int* i0, int* i1, int* m) {
  if (interleaved) {
    *i0 = 2 * pi;
    *i1 = 2 * pi + 1;
    *m = 2 * pi < rot ? pi : -1;
  } else if (pi < rot / 2) {
    *i0 = pi;
    *i1 = pi + rot / 2;
    *m = pi;
  } else {
    *i0 = rot + 2 * (pi - rot / 2);
    *i1 = *i0 + 1;
    *m = -1;
  }
}

template <typename T>
__global__ __launch_bounds__(PREP_THREADS) void attn_prepare_normed_kernel(
    const T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride, const T* __restrict__ v,
    long v_stride, const float* __restrict__ wq, const float* __restrict__ wk, float eps,
    const int* __restrict__ positions, const float* __restrict__ table, int rot, const float* __restrict__ table_v,
    int max_pos, int interleaved, int v_norm, const int* __restrict__ slots, T* __restrict__ q_out, long qo_stride,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int H, int G, int dim, int vdim, int D, int ps) {
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int p = min(max(positions[t], 0), max_pos - 1);
  const T* qr = q + (long)t * q_stride;
  const T* kr = k + (long)t * k_stride;
  const T* vr = v + (long)t * v_stride;
  float inv_q = 1.f, inv_k = 1.f;
  if (wq) {
    float s = 0.f;
    for (int i = tid; i < H * dim; i += PREP_THREADS) {
      const float x = to_f32<T>(qr[i]);
      s += x * x;
    }
    inv_q = 1.f / sqrtf(block_sum(s, red) / (float)(H * dim) + eps);
  }
  if (wk) {
    float s = 0.f;
    for (int i = tid; i < G * dim; i += PREP_THREADS) {
      const float x = to_f32<T>(kr[i]);
      s += x * x;
    }
    inv_k = 1.f / sqrtf(block_sum(s, red) / (float)(G * dim) + eps);
  }
  const float* cs = table ? table + (long)p * rot : nullptr;
  const int half = dim / 2;
  // queries
  T* qo = q_out + (long)t * qo_stride;
  for (int idx = tid; idx < H * half; idx += PREP_THREADS) {
    const int h = idx / half, pi = idx - h * half;
    int i0, i1, m;
    pair_slot(pi, cs ? rot : 0, interleaved, &i0, &i1, &m);
    float x0 = to_f32<T>(qr[h * dim + i0]) * inv_q, x1 = to_f32<T>(qr[h * dim + i1]) * inv_q;
    if (wq) {
      x0 *= wq[h * dim + i0];
      x1 *= wq[h * dim + i1];
    }
    if (m >= 0) rope_rotate(x0, x1, cs[m], cs[rot / 2 + m], &x0, &x1);
    qo[h * D + i0] = from_f32<T>(x0);
    qo[h * D + i1] = from_f32<T>(x1);
  }
  if (D > dim)
    for (int idx = tid; idx < H * (D - dim); idx += PREP_THREADS) {
      const int h = idx / (D - dim);
      qo[h * D + dim + idx - h * (D - dim)] = from_f32<T>(0.f);
    }
  const int slot = slots ? slots[t] : -1;
  if (slot < 0) return;                      // (uniform over the workgroup: nothing of this token is stored)
  const int page = slot / ps, off = slot - page * ps;
  // keys
  for (int idx = tid; idx < G * half; idx += PREP_THREADS) {
    const int g = idx / half, pi = idx - g * half;
    int i0, i1, m;
    pair_slot(pi, cs ? rot : 0, interleaved, &i0, &i1, &m);
    float x0 = to_f32<T>(kr[g * dim + i0]) * inv_k, x1 = to_f32<T>(kr[g * dim + i1]) * inv_k;
    if (wk) {
      x0 *= wk[g * dim + i0];
      x1 *= wk[g * dim + i1];
    }
    if (m >= 0) rope_rotate(x0, x1, cs[m], cs[rot / 2 + m], &x0, &x1);
    T* kp = k_pages + (((long)page * G + g) * ps + off) * D;
    kp[i0] = from_f32<T>(x0);
    kp[i1] = from_f32<T>(x1);
  }
  if (D > dim)
    for (int idx = tid; idx < G * (D - dim); idx += PREP_THREADS) {
      const int g = idx / (D - dim);
      k_pages[(((long)page * G + g) * ps + off) * D + dim + idx - g * (D - dim)] = from_f32<T>(0.f);
    }
  // values: a wave a head
  const int wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE;
  const float* csv = table_v ? table_v + (long)p * vdim : nullptr;
  for (int g = wave; g < G; g += PREP_THREADS / LMSF_WAVE) {
    float inv = 1.f;
    if (v_norm) {
      float s = 0.f;
      for (int i = lane; i < vdim; i += LMSF_WAVE) {
        const float x = to_f32<T>(vr[g * vdim + i]);
        s += x * x;
      }
      inv = 1.f / sqrtf(wave_sum(s) / (float)vdim + eps);
    }
    T* vp = v_pages + ((long)page * G + g) * D * ps + off;
    for (int pi = lane; pi < vdim / 2; pi += LMSF_WAVE) {
      int i0, i1, m;
      pair_slot(pi, csv ? vdim : 0, interleaved, &i0, &i1, &m);
      float x0 = to_f32<T>(vr[g * vdim + i0]) * inv, x1 = to_f32<T>(vr[g * vdim + i1]) * inv;
      if (m >= 0) rope_rotate(x0, x1, csv[m], csv[vdim / 2 + m], &x0, &x1);
      vp[(long)i0 * ps] = from_f32<T>(x0);
      vp[(long)i1 * ps] = from_f32<T>(x1);
    }
    for (int i = vdim + lane; i < D; i += LMSF_WAVE) vp[(long)i * ps] = from_f32<T>(0.f);
  }
}

extern "C" int lmsf_attn_prepare_normed(const void* q, long q_stride, const void* k, long k_stride, const void* v,
                                        long v_stride, int dtype, const float* wq, const float* wk, float eps,
                                        const int* positions, const float* table, int rot, const float* table_v,
                                        int max_pos, int interleaved, int v_norm, const int* slots, void* q_out,
                                        long qo_stride, void* k_pages, void* v_pages, long num_pages, int n_tokens,
                                        int H, int G, int dim, int vdim, int D, int ps, hipStream_t stream) {
  LMSF_CHECK(q && k && v && positions && q_out && k_pages && v_pages, "attn_prepare_normed: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "attn_prepare_normed: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && G > 0 && H % G == 0 && dim > 0 && vdim > 0 && dim % 2 == 0 && vdim % 2 == 0 && D >= dim &&
                 D >= vdim && ps > 0 && num_pages > 0 && max_pos > 0,
             "attn_prepare_normed: bad sizes (heads %d/%d, dim %d, vdim %d, D %d)", H, G, dim, vdim, D);
  LMSF_CHECK(!table || (rot > 0 && rot % 2 == 0 && rot <= dim), "attn_prepare_normed: %d rotated entries of %d", rot, dim);
  LMSF_CHECK(q_stride >= (long)H * dim && k_stride >= (long)G * dim && v_stride >= (long)G * vdim &&
                 qo_stride >= (long)H * D, "attn_prepare_normed: row strides too small");
  if (n_tokens <= 0) return 0;
#define PREP_LAUNCH(T)                                                                                              \
  hipLaunchKernelGGL((attn_prepare_normed_kernel<T>), dim3(n_tokens), dim3(PREP_THREADS), 0, stream, (const T*)q,   \
                     q_stride, (const T*)k, k_stride, (const T*)v, v_stride, wq, wk, eps, positions, table, rot,    \
                     table_v, max_pos, interleaved, v_norm, slots, (T*)q_out, qo_stride, (T*)k_pages, (T*)v_pages, H, \
                     G, dim, vdim, D, ps)
  if (dtype == LMSF_F32) PREP_LAUNCH(float);
  else PREP_LAUNCH(bf16_t);
#undef PREP_LAUNCH
  LMSF_LAUNCH_CHECK("attn_prepare_normed");
  return 0;
}

// ---------------------------------------------------------------- after attention

template <typename T>
__global__ __launch_bounds__(256) void attn_finish_kernel(const T* __restrict__ a, long a_stride,
                                                          const T* __restrict__ gate, long gate_stride,
                                                          const int* __restrict__ positions,
                                                          const float* __restrict__ table_v, int max_pos,
                                                          int interleaved, T* __restrict__ out, long out_stride,
                                                          int n_tokens, int H, int vdim, int D) {
  const long w = (long)blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE;
  const int lane = threadIdx.x % LMSF_WAVE;
  if (w >= (long)n_tokens * H) return;
  const int t = (int)(w / H), h = (int)(w - (long)t * H);
  const int p = min(max(positions[t], 0), max_pos - 1);
  const float* csv = table_v ? table_v + (long)p * vdim : nullptr;
  float gt = 1.f;
  if (gate) gt = 1.f / (1.f + expf(-to_f32<T>(gate[(long)t * gate_stride + h])));
  const T* ar = a + (long)t * a_stride + (long)h * D;
  T* orow = out + (long)t * out_stride + (long)h * vdim;
  for (int pi = lane; pi < vdim / 2; pi += LMSF_WAVE) {
    int i0, i1, m;
    pair_slot(pi, csv ? vdim : 0, interleaved, &i0, &i1, &m);
    float x0 = to_f32<T>(ar[i0]), x1 = to_f32<T>(ar[i1]);
    if (m >= 0) rope_rotate(x0, x1, csv[m], -csv[vdim / 2 + m], &x0, &x1);
    orow[i0] = from_f32<T>(x0 * gt);
    orow[i1] = from_f32<T>(x1 * gt);
  }
}

// a [N, H D] (the attention's result), gate [N, >= H] (one pre-activation a head; null: none), out [N, H vdim]
extern "C" int lmsf_attn_finish(const void* a, long a_stride, const void* gate, long gate_stride, int dtype,
                                const int* positions, const float* table_v, int max_pos, int interleaved, void* out,
                                long out_stride, int n_tokens, int H, int vdim, int D, hipStream_t stream) {
  LMSF_CHECK(a && positions && out, "attn_finish: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "attn_finish: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && vdim > 0 && vdim % 2 == 0 && D >= vdim && max_pos > 0 && a_stride >= (long)H * D &&
                 out_stride >= (long)H * vdim && (!gate || gate_stride >= H), "attn_finish: bad sizes");
  if (n_tokens <= 0) return 0;
  const dim3 grid((unsigned)(((long)n_tokens * H + 3) / 4));
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((attn_finish_kernel<float>), grid, dim3(256), 0, stream, (const float*)a, a_stride,
                       (const float*)gate, gate_stride, positions, table_v, max_pos, interleaved, (float*)out,
                       out_stride, n_tokens, H, vdim, D);
  else
    hipLaunchKernelGGL((attn_finish_kernel<bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)a, a_stride,
                       (const bf16_t*)gate, gate_stride, positions, table_v, max_pos, interleaved, (bf16_t*)out,
                       out_stride, n_tokens, H, vdim, D);
  LMSF_LAUNCH_CHECK("attn_finish");
  return 0;
}
