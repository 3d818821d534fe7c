// Kernels around attention over a cached latent.
//
// A layer of this kind keeps, per token, one normed latent vector c (R numbers) and one rotated key part r
// (dr numbers) that all heads share; head h's key is [Uk_h c | r] and its value Uv_h c. With the up-projections
// folded into the query and the output,
//     score_h(t, j) = (Uk_h^T qn_h(t)) . c(j) + qr_h(t) . r(j),     out_h(t) = Uv_h (sum_j p_h(t, j) c(j)),
// attention runs over the cache as it is: one key/value head [c | r] of width D >= R + dr (padded with zeros to
// what the attention kernels take), shared by all query heads. The pages hold the row twice, as the attention
// kernels read them: K pages [page, 1, offset, D], V pages [page, 1, D, offset].
//
//   lmsf_latent_cache_write   c = rms_norm(x[:R]) * w, r = rotate(x[R:R+dr]) -> pages at the token's slot; from the
//                             same launch the norm of the query's latent, which lies in the same row of the product
//   lmsf_head_linear          y[n, h, :] = W_h x[n, h, :K] (* sigmoid(gate[n, h]), or with ``gate_wide`` entry by
//                             entry * sigmoid(gate[n, h * O + o])), W [H, O, K]: per-head products
//                             (32 tokens and more in bfloat16: on the matrix cores)
//   lmsf_rope_tail            rotates one part of every head of q into another buffer and zeroes its padding
//
// Norm, rotation, gate and accumulation are float32; storage is float32 or bfloat16.
#include "common.h"

#include <math.h>

#define LAT_THREADS 256

// ---------------------------------------------------------------- latent and shared key part into the cache

template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void latent_cache_write_kernel(
    const T* __restrict__ x, long x_stride, const float* __restrict__ w, float eps, const int* __restrict__ positions,
    const float* __restrict__ table, int rot, int max_pos, const int* __restrict__ slots, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int R, int dr, int D, int ps, const T* __restrict__ qx, const float* __restrict__ qw,
    T* __restrict__ q_out, long q_out_stride, int Q) {
  __shared__ float red[16];
  const int n = blockIdx.x;
  if (qx) {
    // the other latent of the same row of the product: q_out = rms_norm(qx) * qw
    const T* qr = qx + (long)n * x_stride;
    float qs = 0.f;
    for (int i = threadIdx.x; i < Q; i += LAT_THREADS) {
      const float v = to_f32<T>(qr[i]);
      qs += v * v;
    }
    qs = block_sum(qs, red);
    const float qrms = sqrtf(qs / (float)Q + eps);
    for (int i = threadIdx.x; i < Q; i += LAT_THREADS)
      q_out[(long)n * q_out_stride + i] = from_f32<T>(to_f32<T>(qr[i]) / qrms * qw[i]);
  }
  const int slot = slots[n];
  if (slot < 0) return;                     // a padding token stores nothing
  const T* xr = x + (long)n * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += LAT_THREADS) {
    const float v = to_f32<T>(xr[i]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rms = sqrtf(ss / (float)R + eps);
  const long page = slot / ps, off = slot % ps;
  T* kd = k_pages + (page * ps + off) * D;
  T* vd = v_pages + page * D * ps + off;
  const int p = min(max(positions[n], 0), max_pos - 1);
  const float* cs = table + (long)p * rot;
  const int half = rot / 2;
  for (int i = threadIdx.x; i < D; i += LAT_THREADS) {
    float v = 0.f;
    if (i < R) {
      v = to_f32<T>(xr[i]) / rms * w[i];
    } else if (i < R + dr) {
      const int e = i - R;
      if (e < half) {
        float a, b;
        rope_rotate(to_f32<T>(xr[i]), to_f32<T>(xr[i + half]), cs[e], cs[half + e], &a, &b);
        v = a;
      } else if (e < rot) {
        float a, b;
        rope_rotate(to_f32<T>(xr[i - half]), to_f32<T>(xr[i]), cs[e - half], cs[e], &a, &b);
        v = b;
      } else {
        v = to_f32<T>(xr[i]);
      }
    }
    const T s = from_f32<T>(v);
    kd[i] = s;
    vd[(long)i * ps] = s;
  }
}

extern "C" int lmsf_latent_cache_write(const void* x, int dtype, long x_stride, const float* w, float eps,
                                       const int* positions, const float* table, int rot, int max_pos,
                                       const int* slots, void* k_pages, void* v_pages, long num_pages, int n_tokens,
                                       int R, int dr, int D, int ps, const void* qx, const float* qw, void* q_out,
                                       long q_out_stride, int Q, hipStream_t stream) {
  LMSF_CHECK(!qx || (qw && q_out && Q > 0 && q_out_stride >= Q), "latent_cache_write: the second norm needs its weight and output");
  LMSF_CHECK(x && w && positions && table && slots && k_pages && v_pages, "latent_cache_write: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "latent_cache_write: unknown dtype code %d", dtype);
  LMSF_CHECK(R > 0 && dr >= 0 && D >= R + dr && x_stride >= R + dr, "latent_cache_write: sizes %d + %d do not fit %d", R, dr, D);
  LMSF_CHECK(rot >= 0 && rot % 2 == 0 && rot <= dr && max_pos > 0, "latent_cache_write: rotation over %d of %d", rot, dr);
  LMSF_CHECK(ps > 0 && num_pages > 0, "latent_cache_write: bad page geometry");
  if (n_tokens <= 0) return 0;
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((latent_cache_write_kernel<float>), dim3(n_tokens), dim3(LAT_THREADS), 0, stream,
                       (const float*)x, x_stride, w, eps, positions, table, rot, max_pos, slots, (float*)k_pages,
                       (float*)v_pages, R, dr, D, ps, (const float*)qx, qw, (float*)q_out, q_out_stride, Q);
  else
    hipLaunchKernelGGL((latent_cache_write_kernel<bf16_t>), dim3(n_tokens), dim3(LAT_THREADS), 0, stream,
                       (const bf16_t*)x, x_stride, w, eps, positions, table, rot, max_pos, slots, (bf16_t*)k_pages,
                       (bf16_t*)v_pages, R, dr, D, ps, (const bf16_t*)qx, qw, (bf16_t*)q_out, q_out_stride, Q);
  LMSF_LAUNCH_CHECK("latent_cache_write");
  return 0;
}

// ---------------------------------------------------------------- per-head products

// y[n, h * y_head + o] = (sum_k W[h, o, k] x[n, h * x_head + k]) * (gate ? sigmoid(gate[n * gate_stride + h]) : 1)
// A workgroup takes HL_TOKENS tokens of one head: their inputs lie in LDS, a thread owns outputs o, o + 256, ...
// and reads each row of W once for all of them.
#define HL_TOKENS 8

template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void head_linear_kernel(
    const T* __restrict__ x, long x_stride, int x_head, const T* __restrict__ W, T* __restrict__ y, long y_stride,
    int y_head, const T* __restrict__ gate, long gate_stride, int n_tokens, int O, int K, int vec, int gate_wide) {
  extern __shared__ float sx[];   // [HL_TOKENS, K]
  const int h = blockIdx.y, n0 = blockIdx.x * HL_TOKENS;
  const int nt = min(HL_TOKENS, n_tokens - n0);
  for (int i = threadIdx.x; i < HL_TOKENS * K; i += LAT_THREADS) {
    const int t = i / K, k = i - t * K;
    sx[i] = t < nt ? to_f32<T>(x[(long)(n0 + t) * x_stride + (long)h * x_head + k]) : 0.f;
  }
  __syncthreads();
  float g[HL_TOKENS];
#pragma unroll
  for (int t = 0; t < HL_TOKENS; ++t) {
    g[t] = 1.f;
    if (gate && !gate_wide && t < nt) g[t] = 1.f / (1.f + expf(-to_f32<T>(gate[(long)(n0 + t) * gate_stride + h])));
  }
  const T* Wh = W + (long)h * O * K;
  constexpr int V = Vec16<T>::N;
  for (int o = threadIdx.x; o < O; o += LAT_THREADS) {
    float acc[HL_TOKENS];
#pragma unroll
    for (int t = 0; t < HL_TOKENS; ++t) acc[t] = 0.f;
    const T* wr = Wh + (long)o * K;
    if (vec) {
      // 16 bytes of a row of W a load
      for (int k = 0; k < K; k += V) {
        Vec16<T> p;
        p.load(wr + k);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float wv = p.get(e);
#pragma unroll
          for (int t = 0; t < HL_TOKENS; ++t) acc[t] += wv * sx[t * K + k + e];
        }
      }
    } else {
      for (int k = 0; k < K; ++k) {
        const float wv = to_f32<T>(wr[k]);
#pragma unroll
        for (int t = 0; t < HL_TOKENS; ++t) acc[t] += wv * sx[t * K + k];
      }
    }
#pragma unroll
    for (int t = 0; t < HL_TOKENS; ++t)
      if (t < nt) {
        const float gg = gate && gate_wide
            ? 1.f / (1.f + expf(-to_f32<T>(gate[(long)(n0 + t) * gate_stride + (long)h * O + o]))) : g[t];
        y[(long)(n0 + t) * y_stride + (long)h * y_head + o] = from_f32<T>(acc[t] * gg);
      }
  }
}

// The same product on the matrix cores, for many tokens in bfloat16: a workgroup takes 64 tokens of one head against
// 64 outputs, a wave 16 of the outputs (A = 16 rows of W_h x 32 k) and four tiles of 16 tokens (B), operands straight
// from memory. K is a multiple of 32; rows and heads begin at multiples of 16 bytes.
// (MT tiles of 16 tokens a workgroup: 1 for steps of few tokens, 4 else.) With ``tail.positions`` the workgroups of
// the first block of outputs also write the rotated part of their tokens' head behind the products (rope_tail below).
struct RopeTailArgs {
  const int* positions;
  const float* table;
  int rot, max_pos, x_at, y_at, dr;
};

template <typename T>
__device__ __forceinline__ float rope_tail_value(const T* __restrict__ xr, const float* __restrict__ cs, int e, int rot,
                                                 int dr) {
  const int half = rot / 2;
  float a, b;
  if (e < half) {
    rope_rotate(to_f32<T>(xr[e]), to_f32<T>(xr[e + half]), cs[e], cs[half + e], &a, &b);
    return a;
  }
  if (e < rot) {
    rope_rotate(to_f32<T>(xr[e - half]), to_f32<T>(xr[e]), cs[e - half], cs[e], &a, &b);
    return b;
  }
  return e < dr ? to_f32<T>(xr[e]) : 0.f;
}

template <int MT>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(
    const bf16_t* __restrict__ x, long x_stride, int x_head, const bf16_t* __restrict__ W, bf16_t* __restrict__ y,
    long y_stride, int y_head, const bf16_t* __restrict__ gate, long gate_stride, int n_tokens, int O, int K,
    RopeTailArgs tail, int gate_wide) {
  const int h = blockIdx.y, n0 = blockIdx.x * (16 * MT);
  const int wave = threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  const int fr = lane % 16, fg = lane / 16;
  const int o0 = blockIdx.z * 64 + wave * 16;
  if (tail.positions && blockIdx.z == 0) {
    const int span = y_head - tail.y_at;
    for (int i = threadIdx.x; i < 16 * MT * span; i += 256) {
      const int n = n0 + i / span, e = i % span;
      if (n >= n_tokens) break;
      const int p = min(max(tail.positions[n], 0), tail.max_pos - 1);
      y[(long)n * y_stride + (long)h * y_head + tail.y_at + e] = f32_to_bf16(rope_tail_value<bf16_t>(
          x + (long)n * x_stride + (long)h * x_head + tail.x_at, tail.table + (long)p * tail.rot, e, tail.rot, tail.dr));
    }
  }
  if (o0 >= O) return;
  const bf16_t* wa = W + ((long)h * O + min(o0 + fr, O - 1)) * K + fg * 8;
  const bf16_t* xb[MT];
  int tok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    tok[mt] = n0 + mt * 16 + fr;
    xb[mt] = x + (long)min(tok[mt], n_tokens - 1) * x_stride + (long)h * x_head + fg * 8;
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k = 0; k < K; k += 32) {
    const bf16x8_t fa = *reinterpret_cast<const bf16x8_t*>(wa + k);
    bf16x8_t fb[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) fb[mt] = *reinterpret_cast<const bf16x8_t*>(xb[mt] + k);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, fb[mt], acc[mt], 0, 0, 0);
  }
  // lane: token fr of every tile of tokens, outputs o0 + fg * 4 .. + 3
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (tok[mt] >= n_tokens) continue;
    const float g = gate && !gate_wide ? 1.f / (1.f + expf(-bf16_to_f32(gate[(long)tok[mt] * gate_stride + h]))) : 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int o = o0 + fg * 4 + j;
      if (o >= O) continue;
      const float gg = gate && gate_wide
          ? 1.f / (1.f + expf(-bf16_to_f32(gate[(long)tok[mt] * gate_stride + (long)h * O + o]))) : g;
      y[(long)tok[mt] * y_stride + (long)h * y_head + o] = f32_to_bf16(acc[mt][j] * gg);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void rope_tail_kernel(
    const T* __restrict__ x, long x_stride, int x_head, int x_at, T* __restrict__ y, long y_stride, int y_head,
    int y_at, const int* __restrict__ positions, const float* __restrict__ table, int rot, int max_pos, int H,
    int dr);

// ``positions`` (may be null): also y[n, h * y_head + y_at + e] = rotate(x[n, h * x_head + x_at + e]) for e < dr and
// zeros behind them up to the head's end (what lmsf_rope_tail does), from the same launch where the matrix cores run.
extern "C" int lmsf_head_linear(const void* x, int dtype, long x_stride, int x_head, const void* W, void* y,
                                long y_stride, int y_head, const void* gate, long gate_stride, int n_tokens, int H,
                                int O, int K, const int* positions, const float* table, int rot, int max_pos, int x_at,
                                int y_at, int dr, int gate_wide, hipStream_t stream) {
  LMSF_CHECK(x && W && y, "head_linear: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "head_linear: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && H <= 65535 && O > 0 && K > 0, "head_linear: bad sizes");
  LMSF_CHECK(x_head >= K && y_head >= O, "head_linear: heads overlap");
  LMSF_CHECK(x_stride >= (long)(H - 1) * x_head + K && y_stride >= (long)(H - 1) * y_head + O, "head_linear: rows overlap");
  LMSF_CHECK((size_t)HL_TOKENS * K * 4 <= 64 * 1024, "head_linear: %d inputs a head do not fit LDS", K);
  if (positions) {
    LMSF_CHECK(table && dr >= 0 && rot >= 0 && rot % 2 == 0 && rot <= dr && max_pos > 0, "head_linear: bad rotation");
    LMSF_CHECK(x_at >= 0 && x_at + dr <= x_head && y_at >= O && y_at + dr <= y_head, "head_linear: the rotated part leaves its head");
    LMSF_CHECK(x_stride >= (long)H * x_head && y_stride >= (long)H * y_head, "head_linear: rows overlap");
  }
  if (n_tokens <= 0) return 0;
  const int es = lmsf_elem_size(dtype);
  const bool rows16 = lmsf_aligned16(x) && lmsf_aligned16(W) && (x_stride * es) % 16 == 0 && ((long)x_head * es) % 16 == 0;
  if (dtype == LMSF_BF16 && K % 32 == 0 && rows16) {
    const RopeTailArgs tail = {positions, table, rot, max_pos, x_at, y_at, dr};
    // tiles of 16 tokens a workgroup: 4 where that still gives workgroups enough to fill the chip, else 1
    if (n_tokens <= 32 || (long)((n_tokens + 63) / 64) * H * ((O + 63) / 64) < 512)
      hipLaunchKernelGGL(head_linear_mfma_kernel<1>, dim3((n_tokens + 15) / 16, H, (O + 63) / 64), dim3(256), 0, stream,
                         (const bf16_t*)x, x_stride, x_head, (const bf16_t*)W, (bf16_t*)y, y_stride, y_head,
                         (const bf16_t*)gate, gate_stride, n_tokens, O, K, tail, gate_wide);
    else
      hipLaunchKernelGGL(head_linear_mfma_kernel<4>, dim3((n_tokens + 63) / 64, H, (O + 63) / 64), dim3(256), 0, stream,
                         (const bf16_t*)x, x_stride, x_head, (const bf16_t*)W, (bf16_t*)y, y_stride, y_head,
                         (const bf16_t*)gate, gate_stride, n_tokens, O, K, tail, gate_wide);
    LMSF_LAUNCH_CHECK("head_linear (matrix cores)");
    return 0;
  }
  const int vec = lmsf_aligned16(W) && (K * es) % 16 == 0;
  const dim3 grid((n_tokens + HL_TOKENS - 1) / HL_TOKENS, H);
  const size_t smem = (size_t)HL_TOKENS * K * 4;
  if (dtype == LMSF_F32) {
    hipLaunchKernelGGL((head_linear_kernel<float>), grid, dim3(LAT_THREADS), smem, stream, (const float*)x, x_stride,
                       x_head, (const float*)W, (float*)y, y_stride, y_head, (const float*)gate, gate_stride, n_tokens,
                       O, K, vec, gate_wide);
    if (positions)
      hipLaunchKernelGGL((rope_tail_kernel<float>), dim3(n_tokens), dim3(LAT_THREADS), 0, stream, (const float*)x,
                         x_stride, x_head, x_at, (float*)y, y_stride, y_head, y_at, positions, table, rot, max_pos, H, dr);
  } else {
    hipLaunchKernelGGL((head_linear_kernel<bf16_t>), grid, dim3(LAT_THREADS), smem, stream, (const bf16_t*)x, x_stride,
                       x_head, (const bf16_t*)W, (bf16_t*)y, y_stride, y_head, (const bf16_t*)gate, gate_stride,
                       n_tokens, O, K, vec, gate_wide);
    if (positions)
      hipLaunchKernelGGL((rope_tail_kernel<bf16_t>), dim3(n_tokens), dim3(LAT_THREADS), 0, stream, (const bf16_t*)x,
                         x_stride, x_head, x_at, (bf16_t*)y, y_stride, y_head, y_at, positions, table, rot, max_pos, H, dr);
  }
  LMSF_LAUNCH_CHECK("head_linear");
  return 0;
}

// ---------------------------------------------------------------- the rotated part of every head's query

// y[n, h * y_head + y_at + e] = rotate(x[n, h * x_head + x_at + e]) for e < dr (the first ``rot`` of them in pairs
// (e, e + rot/2), the rest as they are), and y[n, h * y_head + y_at + dr ...  y_head) = 0.
template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void rope_tail_kernel(
    const T* __restrict__ x, long x_stride, int x_head, int x_at, T* __restrict__ y, long y_stride, int y_head,
    int y_at, const int* __restrict__ positions, const float* __restrict__ table, int rot, int max_pos, int H,
    int dr) {
  const int n = blockIdx.x;
  const int p = min(max(positions[n], 0), max_pos - 1);
  const float* cs = table + (long)p * rot;
  const int span = y_head - y_at;
  for (int i = threadIdx.x; i < H * span; i += LAT_THREADS) {
    const int h = i / span, e = i - h * span;
    y[(long)n * y_stride + (long)h * y_head + y_at + e] =
        from_f32<T>(rope_tail_value<T>(x + (long)n * x_stride + (long)h * x_head + x_at, cs, e, rot, dr));
  }
}

extern "C" int lmsf_rope_tail(const void* x, int dtype, long x_stride, int x_head, int x_at, void* y, long y_stride,
                              int y_head, int y_at, const int* positions, const float* table, int rot, int max_pos,
                              int n_tokens, int H, int dr, hipStream_t stream) {
  LMSF_CHECK(x && y && positions && table, "rope_tail: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "rope_tail: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && dr >= 0 && rot >= 0 && rot % 2 == 0 && rot <= dr && max_pos > 0, "rope_tail: bad sizes");
  LMSF_CHECK(x_at >= 0 && x_at + dr <= x_head && y_at >= 0 && y_at + dr <= y_head, "rope_tail: the part leaves its head");
  LMSF_CHECK(x_stride >= (long)H * x_head && y_stride >= (long)H * y_head, "rope_tail: rows overlap");
  if (n_tokens <= 0) return 0;
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((rope_tail_kernel<float>), dim3(n_tokens), dim3(LAT_THREADS), 0, stream, (const float*)x,
                       x_stride, x_head, x_at, (float*)y, y_stride, y_head, y_at, positions, table, rot, max_pos, H, dr);
  else
    hipLaunchKernelGGL((rope_tail_kernel<bf16_t>), dim3(n_tokens), dim3(LAT_THREADS), 0, stream, (const bf16_t*)x,
                       x_stride, x_head, x_at, (bf16_t*)y, y_stride, y_head, y_at, positions, table, rot, max_pos, H, dr);
  LMSF_LAUNCH_CHECK("rope_tail");
  return 0;
}
