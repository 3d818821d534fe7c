// Retention: linear attention with a fixed decay per head and no softmax or denominator. Per head, with decay g:
//   S_t = g S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   out_t = o_t / rms(o_t) * silu(gate_t)
// (rms over the head's dv entries, eps inside the root, no weight). q and k are rotated by the token's position
// (pairs (i, i + rot/2) of the first ``rot`` entries, cos and sin from a float32 table) on their way in; k is then
// multiplied by ``kscale``. The state of a slot is S as
// [H, d, dv] float32, all zeros when a request begins. The reference has no such mixer (its only one is attention
// over a paged cache, core/src/model_executor/layers/attention.rs:91-231).
//
// Three forms, as for the other matrix memory of this library (recurrent.hip): a segment's chunks of L tokens one
// after the other in a workgroup; chunks side by side (summaries, a fold, outputs) for long segments; and token by
// token with the state streamed once for steps of single tokens. Over a chunk with first state S_0:
//   P[t][u] = (q_t . k_u) g^(t-u) for u <= t;   O = diag(g^(t+1)) Q S_0 + P V;   S_L = g^L S_0 + K^T diag(g^(L-1-u)) V.
// Powers of g are exp(n log g) in float32. Everything is float32 but the operands as they are stored. The chunked
// forms run their products on the matrix cores in float32 where a head's operands fit LDS (heads of up to 256
// entries), with scalar multiply-adds otherwise.
#include "common.h"
#include "entry_points.h"

#include <math.h>

#define RET_THREADS 1024
#define RET_DVB 32            // value columns a workgroup of the chunked forms takes
#define RET_COLS 64           // and of the token form

// entry dd of a head's rotated vector x (as stored) at a position whose table row is cs = [cos | sin]
template <typename T>
__device__ __forceinline__ float ret_rotated(const T* __restrict__ x, const float* __restrict__ cs, int dd, int rot) {
  const float v = to_f32<T>(x[dd]);
  if (dd >= rot) return v;
  const int half = rot / 2;
  float a, b;
  if (dd < half) {
    rope_rotate(v, to_f32<T>(x[dd + half]), cs[dd], cs[half + dd], &a, &b);
    return a;
  }
  rope_rotate(to_f32<T>(x[dd - half]), v, cs[dd - half], cs[dd], &a, &b);
  return b;
}

__device__ __forceinline__ float ret_pow(float lg, int n) { return n == 0 ? 1.f : expf(lg * (float)n); }

extern "C" long lmsf_retention_state_floats(int H, int d, int dv) { return (long)H * d * dv; }

// MODE 0: a segment's chunks one after the other, the state from the slot and back to it.
// MODE 1: chunk j of segment s leaves U = K^T diag(g^(n-1-u)) V in entry chunk_base[s] + j of the scratch.
// MODE 2: chunk j computes its outputs from its S_0, which the fold kernel has put in U's place.
template <typename T, int MODE>
__global__ __launch_bounds__(RET_THREADS) void retention_chunk_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, long qkv_stride,
    const int* __restrict__ positions, const float* __restrict__ table, int rot, int max_pos,
    const float* __restrict__ log_decay, float* __restrict__ state, long state_stride,
    const int* __restrict__ seg_starts, const int* __restrict__ state_slots, float* __restrict__ o_raw, long o_stride,
    int H, int d, int dv, int L, float kscale, int n_vb, const int* __restrict__ chunk_base, float* __restrict__ sc_U) {
  extern __shared__ float lds[];
  const int dp = d | 1, NCp = RET_DVB | 1, Lp = L | 1;
  float* sq = lds;                  // [L][dp]
  float* sk = sq + L * dp;          // [L][dp]
  float* sv = sk + L * dp;          // [L][NCp]
  float* sP = sv + L * NCp;         // [L][Lp]
  float* sS = sP + L * Lp;          // [d][NCp]
  const int tid = threadIdx.x;
  const int h = blockIdx.x, s = blockIdx.y;
  const int vb = MODE == 0 ? blockIdx.z : blockIdx.z % n_vb, j = MODE == 0 ? 0 : blockIdx.z / n_vb;
  const int e0 = vb * RET_DVB, nb = min(RET_DVB, dv - e0);
  const int seg_start = seg_starts[s], seg_end = seg_starts[s + 1];
  if (MODE != 0 && j * L >= seg_end - seg_start) return;
  const int start = MODE == 0 ? seg_start : seg_start + j * L;
  const int end = MODE == 0 ? seg_end : min(seg_end, start + L);
  const float lg = log_decay[h];
  float* gS = MODE == 0 ? state + (long)state_slots[s] * state_stride + (long)h * d * dv
                        : sc_U + (((long)chunk_base[s] + j) * H + h) * d * dv;
  if (MODE != 1)
    for (int i = tid; i < d * nb; i += RET_THREADS) {
      const int dd = i / nb, c = i % nb;
      sS[dd * NCp + c] = gS[(long)dd * dv + e0 + c];
    }
  for (int t0 = start; t0 < end; t0 += L) {
    const int nt = min(L, end - t0);
    __syncthreads();
    for (int i = tid; i < nt * d; i += RET_THREADS) {
      const int tt = i / d, dd = i % d;
      const long row = (long)(t0 + tt) * qkv_stride + (long)h * d;
      const float* cs = table ? table + (long)min(max(positions[t0 + tt], 0), max_pos - 1) * rot : nullptr;
      if (MODE != 1) sq[tt * dp + dd] = cs ? ret_rotated<T>(q + row, cs, dd, rot) : to_f32<T>(q[row + dd]);
      sk[tt * dp + dd] = (cs ? ret_rotated<T>(k + row, cs, dd, rot) : to_f32<T>(k[row + dd])) * kscale;
    }
    for (int i = tid; i < nt * nb; i += RET_THREADS) {
      const int tt = i / nb, c = i % nb;
      sv[tt * NCp + c] = to_f32<T>(v[(long)(t0 + tt) * qkv_stride + (long)h * dv + e0 + c]);
    }
    __syncthreads();
    if (MODE != 1) {
      for (int i = tid; i < nt * nt; i += RET_THREADS) {
        const int t = i / nt, u = i % nt;
        float acc = 0.f;
        if (u <= t) {
          const float* qr = sq + t * dp;
          const float* kr = sk + u * dp;
#pragma unroll 8
          for (int dd = 0; dd < d; ++dd) acc += qr[dd] * kr[dd];
          acc *= ret_pow(lg, t - u);
        }
        sP[t * Lp + u] = acc;
      }
      __syncthreads();
      for (int i = tid; i < nt * nb; i += RET_THREADS) {
        const int t = i / nb, c = i % nb;
        float acc = 0.f;
        const float* qr = sq + t * dp;
#pragma unroll 8
        for (int dd = 0; dd < d; ++dd) acc += qr[dd] * sS[dd * NCp + c];
        acc *= ret_pow(lg, t + 1);
        const float* pr = sP + t * Lp;
#pragma unroll 4
        for (int u = 0; u <= t; ++u) acc += pr[u] * sv[u * NCp + c];
        o_raw[(long)(t0 + t) * o_stride + (long)h * dv + e0 + c] = acc;
      }
    }
    if (MODE == 0) {
      __syncthreads();
      const float wl = ret_pow(lg, nt);
      for (int i = tid; i < d * nb; i += RET_THREADS) {
        const int dd = i / nb, c = i % nb;
        float r = sS[dd * NCp + c] * wl;
        for (int u = 0; u < nt; ++u) r += sk[u * dp + dd] * ret_pow(lg, nt - 1 - u) * sv[u * NCp + c];
        sS[dd * NCp + c] = r;
      }
    }
    if (MODE == 1)
      for (int i = tid; i < d * nb; i += RET_THREADS) {
        const int dd = i / nb, c = i % nb;
        float r = 0.f;
        for (int u = 0; u < nt; ++u) r += sk[u * dp + dd] * ret_pow(lg, nt - 1 - u) * sv[u * NCp + c];
        gS[(long)dd * dv + e0 + c] = r;
      }
  }
  if (MODE == 0) {
    __syncthreads();
    for (int i = tid; i < d * nb; i += RET_THREADS) {
      const int dd = i / nb, c = i % nb;
      gS[(long)dd * dv + e0 + c] = sS[dd * NCp + c];
    }
  }
}

// The same three forms with the products on the matrix cores in float32 (v_mfma_f32_16x16x4_f32: full float32
// operands and sums). A workgroup of sixteen waves takes a head, a chunk and RM_NB value columns; every size is padded
// with zeros to a multiple of 16 in LDS. A wave computes tiles of 16 x 16: of P = Q K^T (at and below the diagonal,
// masked and decayed as it is stored), of O = diag(g^(t+1)) Q S_0 + P V (the second product as far as the diagonal)
// and of S_L = g^L S_0 + K^T (w V). Rows of operands whose row is the product's inner index lie RM_BS apart, the
// others a multiple of 16 plus 4, so that a wave's 64 operand reads fall into 64 banks.
#define RM_THREADS 1024
#define RM_NB 64
#define RM_BS (RM_NB + 16)

template <typename T, int MODE>
__global__ __launch_bounds__(RM_THREADS) void retention_chunk_mfma_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, long qkv_stride,
    const int* __restrict__ positions, const float* __restrict__ table, int rot, int max_pos,
    const float* __restrict__ log_decay, float* __restrict__ state, long state_stride,
    const int* __restrict__ seg_starts, const int* __restrict__ state_slots, float* __restrict__ o_raw, long o_stride,
    int H, int d, int dv, int L, float kscale, int n_vb, const int* __restrict__ chunk_base, float* __restrict__ sc_U) {
  extern __shared__ float lds[];
  const int d16 = (d + 15) / 16 * 16, dq = d16 + 4, Lq = L + 4;
  float* sq = lds;                  // [L][dq]
  float* sk = sq + L * dq;          // [L][dq]
  float* sv = sk + L * dq;          // [L][RM_BS]
  float* sP = sv + L * RM_BS;       // [L][Lq]
  float* sS = sP + L * Lq;          // [d16][RM_BS]
  float* sw = sS + d16 * RM_BS;     // [L]
  const int tid = threadIdx.x, wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE, fr = lane % 16, fg = lane / 16;
  const int h = blockIdx.x, s = blockIdx.y;
  const int vb = MODE == 0 ? blockIdx.z : blockIdx.z % n_vb, j = MODE == 0 ? 0 : blockIdx.z / n_vb;
  const int e0 = vb * RM_NB, nb = min(RM_NB, dv - e0);
  const int seg_start = seg_starts[s], seg_end = seg_starts[s + 1];
  if (MODE != 0 && j * L >= seg_end - seg_start) return;
  const int start = MODE == 0 ? seg_start : seg_start + j * L;
  const int end = MODE == 0 ? seg_end : min(seg_end, start + L);
  const float lg = log_decay[h];
  const int nRT = L / 16, nCT = (nb + 15) / 16, nDT = d16 / 16;
  float* gS = MODE == 0 ? state + (long)state_slots[s] * state_stride + (long)h * d * dv
                        : sc_U + (((long)chunk_base[s] + j) * H + h) * d * dv;
  if (MODE != 1)
    for (int i = tid; i < d16 * RM_NB; i += RM_THREADS) {
      const int dd = i / RM_NB, c = i % RM_NB;
      sS[dd * RM_BS + c] = dd < d && c < nb ? gS[(long)dd * dv + e0 + c] : 0.f;
    }
  for (int t0 = start; t0 < end; t0 += L) {
    const int nt = min(L, end - t0);
    __syncthreads();
    // a row's units: the rotated pairs (e, e + half), then the entries that pass unchanged and the padding
    const int rotn = table ? rot : 0, half = rotn / 2, per_row = half + (d16 - rotn);
#pragma unroll 2
    for (int i = tid; i < L * per_row; i += RM_THREADS) {
      const int tt = i / per_row, e = i % per_row;
      const bool live = tt < nt;
      const long row = (long)(t0 + min(tt, nt - 1)) * qkv_stride + (long)h * d;
      if (e < half) {
        float qa = 0.f, qb = 0.f, ka = 0.f, kb = 0.f;
        if (live) {
          const float* cs = table + (long)min(max(positions[t0 + tt], 0), max_pos - 1) * rot;
          const float c = cs[e], sn = cs[half + e];
          if (MODE != 1) rope_rotate(to_f32<T>(q[row + e]), to_f32<T>(q[row + e + half]), c, sn, &qa, &qb);
          rope_rotate(to_f32<T>(k[row + e]), to_f32<T>(k[row + e + half]), c, sn, &ka, &kb);
        }
        if (MODE != 1) sq[tt * dq + e] = qa, sq[tt * dq + e + half] = qb;
        sk[tt * dq + e] = ka * kscale, sk[tt * dq + e + half] = kb * kscale;
      } else {
        const int dd = rotn + e - half;
        const bool in = live && dd < d;
        if (MODE != 1) sq[tt * dq + dd] = in ? to_f32<T>(q[row + dd]) : 0.f;
        sk[tt * dq + dd] = in ? to_f32<T>(k[row + dd]) * kscale : 0.f;
      }
    }
#pragma unroll 4
    for (int i = tid; i < L * RM_NB; i += RM_THREADS) {
      const int tt = i / RM_NB, c = i % RM_NB;
      sv[tt * RM_BS + c] =
          tt < nt && c < nb ? to_f32<T>(v[(long)(t0 + tt) * qkv_stride + (long)h * dv + e0 + c]) : 0.f;
    }
    if (MODE != 2)
      for (int i = tid; i < L; i += RM_THREADS) sw[i] = i < nt ? ret_pow(lg, nt - 1 - i) : 0.f;
    __syncthreads();
    if (MODE != 1) {
      for (int tile = wave; tile < nRT * nRT; tile += RM_THREADS / LMSF_WAVE) {
        const int rt = tile / nRT, ct = tile % nRT;
        if (ct > rt) continue;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        const float* ap = sq + (rt * 16 + fr) * dq + fg;
        const float* bp = sk + (ct * 16 + fr) * dq + fg;
#pragma unroll 4
        for (int kk = 0; kk < d16; kk += 4) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[kk], bp[kk], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = rt * 16 + fg * 4 + r, u = ct * 16 + fr;
          sP[t * Lq + u] = u <= t ? acc[r] * ret_pow(lg, t - u) : 0.f;
        }
      }
      __syncthreads();
      for (int tile = wave; tile < nRT * nCT; tile += RM_THREADS / LMSF_WAVE) {
        const int rt = tile / nCT, ct = tile % nCT;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        const float* ap = sq + (rt * 16 + fr) * dq + fg;
        const float* bp = sS + fg * RM_BS + ct * 16 + fr;
#pragma unroll 4
        for (int kk = 0; kk < d16; kk += 4)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[kk], bp[kk * RM_BS], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] *= ret_pow(lg, rt * 16 + fg * 4 + r + 1);
        ap = sP + (rt * 16 + fr) * Lq + fg;
        bp = sv + fg * RM_BS + ct * 16 + fr;
#pragma unroll 4
        for (int kk = 0; kk < (rt + 1) * 16; kk += 4)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[kk], bp[kk * RM_BS], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = rt * 16 + fg * 4 + r, c = ct * 16 + fr;
          if (t < nt && c < nb) o_raw[(long)(t0 + t) * o_stride + (long)h * dv + e0 + c] = acc[r];
        }
      }
    }
    if (MODE != 2) {
      if (MODE == 0) __syncthreads();       // every wave has read the old S
      const float wl = ret_pow(lg, nt);
      for (int tile = wave; tile < nDT * nCT; tile += RM_THREADS / LMSF_WAVE) {
        const int dt = tile / nCT, ct = tile % nCT;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (MODE == 0) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] = sS[(dt * 16 + fg * 4 + r) * RM_BS + ct * 16 + fr] * wl;
        }
        const float* ap = sk + fg * dq + dt * 16 + fr;       // K^T: row dd, inner index u
        const float* bp = sv + fg * RM_BS + ct * 16 + fr;
        const float* wp = sw + fg;
#pragma unroll 4
        for (int kk = 0; kk < L; kk += 4)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ap[kk * dq], bp[kk * RM_BS] * wp[kk], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int dd = dt * 16 + fg * 4 + r, c = ct * 16 + fr;
          if (MODE == 0) sS[dd * RM_BS + c] = acc[r];
          else if (dd < d && c < nb) gS[(long)dd * dv + e0 + c] = acc[r];
        }
      }
    }
  }
  if (MODE == 0) {
    __syncthreads();
    for (int i = tid; i < d * nb; i += RM_THREADS) {
      const int dd = i / nb, c = i % nb;
      gS[(long)dd * dv + e0 + c] = sS[dd * RM_BS + c];
    }
  }
}

static size_t ret_mfma_smem(int d, int L) {
  const int d16 = (d + 15) / 16 * 16;
  return ((size_t)2 * L * (d16 + 4) + (size_t)L * RM_BS + (size_t)L * (L + 4) + (size_t)d16 * RM_BS + L) * sizeof(float);
}

// tokens of a chunk of the matrix-core form at heads of d; 0: its operands do not fit a workgroup's LDS
static int ret_mfma_tokens(int d) {
  for (int L = 64; L >= 16; L /= 2)
    if (ret_mfma_smem(d, L) <= 128 * 1024) return L;
  return 0;
}

// Chunk after chunk of a segment: the chunk's S_0 takes U's place, then S <- g^n S + U (n: the chunk's tokens); at the
// end S goes to the slot. A thread an entry of one head's S.
__global__ __launch_bounds__(256) void retention_fold_kernel(float* __restrict__ state, long state_stride,
                                                             const int* __restrict__ seg_starts,
                                                             const int* __restrict__ state_slots,
                                                             const int* __restrict__ chunk_base,
                                                             float* __restrict__ sc_U,
                                                             const float* __restrict__ log_decay, int H, int d, int dv,
                                                             int L) {
  const int h = blockIdx.x, s = blockIdx.y;
  const long per = (long)d * dv;
  const long i = (long)blockIdx.z * 256 + threadIdx.x;
  if (i >= per) return;
  const int n_tok = seg_starts[s + 1] - seg_starts[s];
  const int n_chunks = (n_tok + L - 1) / L;
  float* st = state + (long)state_slots[s] * state_stride;
  float S = st[(long)h * per + i];
  const float lg = log_decay[h];
  const long base = chunk_base[s];
  for (int j = 0; j < n_chunks; ++j) {
    const long ent = (base + j) * H + h;
    const float U = sc_U[ent * per + i];
    sc_U[ent * per + i] = S;
    S = ret_pow(lg, min(L, n_tok - j * L)) * S + U;
  }
  st[(long)h * per + i] = S;
}

// out[t, h, e] = o[e] / rms_e(o) * silu(g[t, h, e]); a wave a (token, head)
template <typename T>
__global__ __launch_bounds__(256) void retention_head_kernel(const float* __restrict__ o, long o_stride,
                                                             const T* __restrict__ og, long og_stride,
                                                             T* __restrict__ out, long out_stride, int n_tokens, int H,
                                                             int dv, float eps) {
  const long unit = (long)blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE;
  if (unit >= (long)n_tokens * H) return;
  const long t = unit / H;
  const int h = unit % H, lane = threadIdx.x % LMSF_WAVE;
  const float* row = o + t * o_stride + (long)h * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += LMSF_WAVE) ss += row[e] * row[e];
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)dv + eps);
  for (int e = lane; e < dv; e += LMSF_WAVE) {
    const float g = to_f32<T>(og[t * og_stride + (long)h * dv + e]);
    out[t * out_stride + (long)h * dv + e] = from_f32<T>(row[e] * inv * (g / (1.f + expf(-g))));
  }
}

// Steps of single tokens: a workgroup takes one head of one segment and 64 of its value columns; wave w walks the
// rows w, w + 4, ..., a lane a column, eight rows asked for at a time. Segments of several tokens are walked token
// by token.
template <typename T>
__global__ __launch_bounds__(256) void retention_token_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, long qkv_stride,
    const int* __restrict__ positions, const float* __restrict__ table, int rot, int max_pos,
    const float* __restrict__ decay, float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts,
    const int* __restrict__ state_slots, float* __restrict__ o_raw, long o_stride, int H, int d, int dv, float kscale) {
  extern __shared__ float lds[];
  float* sq = lds;               // [d]
  float* sk = sq + d;            // [d]
  float* so = sk + d;            // [4][64]
  const int tid = threadIdx.x, wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE;
  const int h = blockIdx.x, s = blockIdx.y, e0 = blockIdx.z * RET_COLS;
  const bool col_ok = e0 + lane < dv;
  float* gS = state + (long)state_slots[s] * state_stride + (long)h * d * dv;
  const float keep = decay[h];
  for (int t = seg_starts[s]; t < seg_starts[s + 1]; ++t) {
    __syncthreads();
    const long row = (long)t * qkv_stride + (long)h * d;
    const float* cs = table ? table + (long)min(max(positions[t], 0), max_pos - 1) * rot : nullptr;
    for (int i = tid; i < d; i += 256) {
      sq[i] = cs ? ret_rotated<T>(q + row, cs, i, rot) : to_f32<T>(q[row + i]);
      sk[i] = (cs ? ret_rotated<T>(k + row, cs, i, rot) : to_f32<T>(k[row + i])) * kscale;
    }
    const float vv = col_ok ? to_f32<T>(v[(long)t * qkv_stride + (long)h * dv + e0 + lane]) : 0.f;
    __syncthreads();
    float acc = 0.f;
    for (int d0 = wave; d0 < d; d0 += 4 * 8) {
      float r[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int dd = d0 + 4 * j;
        r[j] = (dd < d && col_ok) ? gS[(long)dd * dv + e0 + lane] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int dd = d0 + 4 * j;
        if (dd < d && col_ok) {
          const float x = keep * r[j] + sk[dd] * vv;
          gS[(long)dd * dv + e0 + lane] = x;
          acc += x * sq[dd];
        }
      }
    }
    so[wave * RET_COLS + lane] = acc;
    __syncthreads();
    if (wave == 0 && col_ok)
      o_raw[(long)t * o_stride + (long)h * dv + e0 + lane] =
          so[lane] + so[RET_COLS + lane] + so[2 * RET_COLS + lane] + so[3 * RET_COLS + lane];
  }
}

static size_t ret_chunk_smem(int d, int L) {
  const int dp = d | 1, NCp = RET_DVB | 1;
  return ((size_t)2 * L * dp + (size_t)L * NCp + (size_t)L * (L | 1) + (size_t)d * NCp) * sizeof(float);
}

// tokens of a chunk at heads of d (the most for which a workgroup's operands fit its LDS); 0: none do
extern "C" int lmsf_retention_chunk_tokens(int d) {
  if (ret_mfma_tokens(d) > 0) return ret_mfma_tokens(d);
  for (int L = 64; L >= 4; L /= 2)
    if (ret_chunk_smem(d, L) <= 128 * 1024) return L;
  return 0;
}

// floats of scratch a chunk of the side-by-side form takes
extern "C" long lmsf_retention_chunk_entry_floats(int H, int d, int dv) { return (long)H * d * dv; }

static int ret_check(const void* q, const void* k, const void* v, int dtype, long qkv_stride, const int* positions,
                     const float* table, int rot, int max_pos, const float* decay, const void* og, long og_stride,
                     float* state, long state_stride, const int* seg_starts, const int* state_slots, void* out,
                     long out_stride, float* o_raw, int n_tokens, int n_segments, int H, int d, int dv) {
  LMSF_CHECK(q && k && v && decay && og && state && seg_starts && state_slots && out && o_raw, "retention: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "retention: unknown dtype code %d", dtype);
  LMSF_CHECK(H > 0 && H <= 65535 && d > 0 && d <= 4096 && dv > 0, "retention: bad sizes H=%d d=%d dv=%d", H, d, dv);
  LMSF_CHECK(!table || (positions && rot > 0 && rot % 2 == 0 && rot <= d && max_pos > 0), "retention: bad rotation");
  LMSF_CHECK(qkv_stride >= (long)H * d && og_stride >= (long)H * dv && out_stride >= (long)H * dv &&
                 state_stride >= lmsf_retention_state_floats(H, d, dv),
             "retention: strides too small");
  LMSF_CHECK(n_tokens >= 0 && n_segments >= 0 && n_segments <= 65535, "retention: bad counts");
  return 0;
}

template <typename T>
static void ret_heads(const float* o_raw, const void* og, long og_stride, void* out, long out_stride, int n_tokens,
                      int H, int dv, float eps, hipStream_t stream) {
  const long units = (long)n_tokens * H;
  hipLaunchKernelGGL((retention_head_kernel<T>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, o_raw,
                     (long)H * dv, (const T*)og, og_stride, (T*)out, out_stride, n_tokens, H, dv, eps);
}

// ``decay``: float32 [2 H], every head's decay and then every head's logarithm of it. ``o_raw``: float32 scratch
// [n_tokens, H * dv]. ``chunk_base`` null: every segment's chunks one after the other in a workgroup. Otherwise
// chunk_base[s] is segment s's first entry of ``entries`` (``n_entries`` of them, each
// lmsf_retention_chunk_entry_floats), a segment having ceil(tokens / lmsf_retention_chunk_tokens(d)) chunks and the
// longest ``max_chunks``; the chunks then run side by side.
extern "C" int lmsf_retention_chunked(const void* q, const void* k, const void* v, int dtype, long qkv_stride,
                                      const int* positions, const float* table, int rot, int max_pos,
                                      const float* decay, const void* og, long og_stride, float* state,
                                      long state_stride, const int* seg_starts, const int* state_slots, void* out,
                                      long out_stride, float* o_raw, int n_tokens, int n_segments, int H, int d, int dv,
                                      float kscale, float eps, const int* chunk_base, int max_chunks, long n_entries,
                                      float* entries, hipStream_t stream) {
  if (ret_check(q, k, v, dtype, qkv_stride, positions, table, rot, max_pos, decay, og, og_stride, state, state_stride,
                seg_starts, state_slots, out, out_stride, o_raw, n_tokens, n_segments, H, d, dv))
    return 1;
  LMSF_CHECK(!chunk_base || (entries && max_chunks >= 1 && n_entries >= 1), "retention: chunks without scratch");
  if (n_tokens == 0 || n_segments == 0) return 0;
  const int L = lmsf_retention_chunk_tokens(d);
  LMSF_CHECK(L > 0, "retention: heads of %d entries do not fit a workgroup's LDS", d);
  const bool mfma = ret_mfma_tokens(d) > 0;
  const size_t smem = mfma ? ret_mfma_smem(d, L) : ret_chunk_smem(d, L);
  const int n_vb = mfma ? (dv + RM_NB - 1) / RM_NB : (dv + RET_DVB - 1) / RET_DVB;
  LMSF_CHECK(!chunk_base || (long)n_vb * max_chunks <= 65535, "retention: too many chunks");
  const float* log_decay = decay + H;
#define RET_LAUNCH_OF(KERNEL, THREADS, T, MODE, GRID)                                                                \
  do {                                                                                                               \
    static size_t reserved = 0;                                                                                      \
    if (smem > 64 * 1024 && smem > reserved) {                                                                       \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(KERNEL<T, MODE>),                             \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                     \
      if (e != hipSuccess) {                                                                                         \
        lmsf_set_error("retention: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));                \
        return 2;                                                                                                    \
      }                                                                                                              \
      reserved = smem;                                                                                               \
    }                                                                                                                \
    hipLaunchKernelGGL((KERNEL<T, MODE>), GRID, dim3(THREADS), smem, stream, (const T*)q, (const T*)k, (const T*)v,  \
                       qkv_stride, positions, table, rot, max_pos, log_decay, state, state_stride, seg_starts,       \
                       state_slots, o_raw, (long)H * dv, H, d, dv, L, kscale, n_vb, chunk_base, entries);            \
  } while (0)
#define RET_LAUNCH(T, MODE, GRID)                                                                                    \
  do {                                                                                                               \
    if (mfma) RET_LAUNCH_OF(retention_chunk_mfma_kernel, RM_THREADS, T, MODE, GRID);                                 \
    else RET_LAUNCH_OF(retention_chunk_kernel, RET_THREADS, T, MODE, GRID);                                          \
  } while (0)
  if (!chunk_base) {
    dim3 grid(H, n_segments, n_vb);
    if (dtype == LMSF_F32) RET_LAUNCH(float, 0, grid); else RET_LAUNCH(bf16_t, 0, grid);
    LMSF_LAUNCH_CHECK("retention_chunk");
  } else {
    dim3 grid(H, n_segments, n_vb * max_chunks);
    if (dtype == LMSF_F32) RET_LAUNCH(float, 1, grid); else RET_LAUNCH(bf16_t, 1, grid);
    LMSF_LAUNCH_CHECK("retention_chunk (summaries)");
    const long per = (long)d * dv;
    hipLaunchKernelGGL(retention_fold_kernel, dim3(H, n_segments, (unsigned)((per + 255) / 256)), dim3(256), 0, stream,
                       state, state_stride, seg_starts, state_slots, chunk_base, entries, log_decay, H, d, dv, L);
    LMSF_LAUNCH_CHECK("retention_chunk (fold)");
    if (dtype == LMSF_F32) RET_LAUNCH(float, 2, grid); else RET_LAUNCH(bf16_t, 2, grid);
    LMSF_LAUNCH_CHECK("retention_chunk (outputs)");
  }
#undef RET_LAUNCH
#undef RET_LAUNCH_OF
  if (dtype == LMSF_F32) ret_heads<float>(o_raw, og, og_stride, out, out_stride, n_tokens, H, dv, eps, stream);
  else ret_heads<bf16_t>(o_raw, og, og_stride, out, out_stride, n_tokens, H, dv, eps, stream);
  LMSF_LAUNCH_CHECK("retention_head");
  return 0;
}

// The same function for steps of few tokens a segment (decoding).
extern "C" int lmsf_retention_tokens(const void* q, const void* k, const void* v, int dtype, long qkv_stride,
                                     const int* positions, const float* table, int rot, int max_pos,
                                     const float* decay, const void* og, long og_stride, float* state,
                                     long state_stride, const int* seg_starts, const int* state_slots, void* out,
                                     long out_stride, float* o_raw, int n_tokens, int n_segments, int H, int d, int dv,
                                     float kscale, float eps, hipStream_t stream) {
  if (ret_check(q, k, v, dtype, qkv_stride, positions, table, rot, max_pos, decay, og, og_stride, state, state_stride,
                seg_starts, state_slots, out, out_stride, o_raw, n_tokens, n_segments, H, d, dv))
    return 1;
  LMSF_CHECK((dv + RET_COLS - 1) / RET_COLS <= 65535, "retention: too many value columns");
  if (n_tokens == 0 || n_segments == 0) return 0;
  dim3 grid(H, n_segments, (dv + RET_COLS - 1) / RET_COLS), block(256);
  const size_t smem = (size_t)(2 * d + 4 * RET_COLS) * sizeof(float);
  if (dtype == LMSF_F32) {
    hipLaunchKernelGGL((retention_token_kernel<float>), grid, block, smem, stream, (const float*)q, (const float*)k,
                       (const float*)v, qkv_stride, positions, table, rot, max_pos, decay, state, state_stride,
                       seg_starts, state_slots, o_raw, (long)H * dv, H, d, dv, kscale);
    LMSF_LAUNCH_CHECK("retention_tokens");
    ret_heads<float>(o_raw, og, og_stride, out, out_stride, n_tokens, H, dv, eps, stream);
  } else {
    hipLaunchKernelGGL((retention_token_kernel<bf16_t>), grid, block, smem, stream, (const bf16_t*)q, (const bf16_t*)k,
                       (const bf16_t*)v, qkv_stride, positions, table, rot, max_pos, decay, state, state_stride,
                       seg_starts, state_slots, o_raw, (long)H * dv, H, d, dv, kscale);
    LMSF_LAUNCH_CHECK("retention_tokens");
    ret_heads<bf16_t>(o_raw, og, og_stride, out, out_stride, n_tokens, H, dv, eps, stream);
  }
  LMSF_LAUNCH_CHECK("retention_head");
  return 0;
}
