// The gated delta rule with one decay per head and key channel, a matrix memory S [dim, vdim] per head and request:
//
//   S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
//
// (the read-out sees the token's own write). What enters the recurrence is made here, in float32, from the
// projections' results: q and k are made unit vectors per head, x / sqrt(sum x^2 + unit_eps), q times q_scale;
// beta = sigmoid(b); g = exp(-exp(A_log_h) softplus(a + dt_bias)), one factor per head and key channel, acting on the
// rows of S. H value heads and G query/key heads (head h reads q/k head h / (H / G)). S lives in the request's state
// slot in float32 and is read once and written once a step.
//
// The columns of S are independent of one another: column j only ever needs k, q, g, beta and v_j. Token by token a
// step is a chain of dependent operations (two sums over the rows of a column, one after the other), and what bounds
// a long segment is the time of that chain, not the chip's rate. So the tokens are taken four at a time. With
// G_t the decays' logarithms summed up to token t of the chunk, s_0 the column before the chunk and
//   A[t][m] = sum_i k_t,i k_m,i exp(G_t,i - G_m,i)  (m < t),     B[t][m] = sum_i q_t,i k_m,i exp(G_t,i - G_m,i)  (m <= t)
// the four steps are
//   u_t = beta_t (v_t - (k_t exp G_t) . s_0 - sum_{m<t} A[t][m] u_m),      o_t = (q_t exp G_t) . s_0 + sum_{m<=t} B[t][m] u_m,
//   s_4 = exp(G_4) s_0 + sum_m (k_m exp(G_4 - G_m)) u_m
// (exponents are differences of sums of logarithms and never positive: nothing overflows and nothing is divided). All
// eight sums over the rows are against s_0 and run side by side; the rest is a few multiply-adds per column.
//
// Two kernels. The first makes everything of a chunk ready that does not depend on S, side by side for all chunks: unit
// vectors, decays, the vectors above in the order in which the second kernel's lanes read them, beta, A and B; and the
// values as float32 in blocks of 8 columns. A chunk is four tokens of one request counted from the first token of its
// step's portion (the last chunk of a portion may hold fewer: the missing tokens have beta = 0 and k = q = 0). The
// second runs the recurrence with a column's rows spread over 16 lanes (RPL = rows a lane holds, in registers; the key
// size is padded to 16 RPL), four columns a wave and two waves a workgroup; the sum over a row of 16 lanes is four
// additions through the vector unit's data-parallel path. What the steps read travels from global memory straight
// into LDS a batch of chunks ahead (two buffers). Tokens of a request run one after the other; (request, head, 8
// columns) side by side. Measured at 2,048 tokens, 16 heads of 64 x 128: token by token with the operands asked for
// four tokens ahead into registers 1,360 us (a step waited for memory), through LDS a batch ahead 767 us, with the
// sums through the data-parallel path instead of the lane-permute instruction 376 us, four tokens at a time with one
// store a chunk 293 us: 132 vector, 36 scalar and 23 LDS instructions a chunk and wave with 4 rows a lane (counters), one
// wave a SIMD, issuing in 58 % of its cycles: its own chain of instructions is what bounds it now (sharing the operands
// among 2 or 4 waves changed nothing). The state lies as [H, ceil(vdim / 4), dim, 4], so
// that a wave's part of it is one piece of memory; a step of single tokens is the same kernels with room for one chunk
// in LDS, bound by the memory's bytes: S in and out.
//
// A third kernel divides every head's o by its root mean square, multiplies by a weight over vdim (shared by the
// heads) and by sigmoid or silu of a gate, and rounds to the run's type.
#include "common.h"

#include <math.h>

#define DELTA_R 16            // lanes that share a column
#define DELTA_CPW 4           // columns a wave holds
#define DELTA_WAVES 2         // waves a workgroup (they share the operands in LDS)
#define DELTA_COLS (DELTA_CPW * DELTA_WAVES)
#define DELTA_CHUNK 4         // tokens a chunk

__device__ __forceinline__ float softplus_f32(float x) { return x > 20.f ? x : log1pf(expf(x)); }

static inline int delta_rows_per_lane(int dim) { return dim <= 16 ? 1 : dim <= 32 ? 2 : dim <= 64 ? 4 : dim <= 128 ? 8 : 16; }
// chunks a batch holds, and the floats of a (chunk, head): 13 vectors in the lanes' order (k exp G, q exp G and
// k exp(G_4 - G) of the four tokens, exp G_4), then beta [4], A [6], B [10]
__host__ __device__ constexpr int delta_batch_chunks(int rpl) { return 512 / (DELTA_R * rpl) < 16 ? 512 / (DELTA_R * rpl) : 16; }
__host__ __device__ constexpr int delta_block_floats(int rpl) { return 13 * DELTA_R * rpl + 20; }

// The chunk that begins at token t of segment s (first token t0) lies in row t0 / 4 + s + (t - t0) / 4 of a head's
// rows: rows of different segments never meet, and a segment's rows lie one behind the other.
__device__ __forceinline__ long delta_chunk_row(int t0, int s, int t) { return t0 / DELTA_CHUNK + s + (t - t0) / DELTA_CHUNK; }

// The sum over a row of 16 lanes, in every lane of the row: four additions whose second operand comes through the
// data-parallel path of the vector unit (neighbours within a quad, then the mirror image within 8 and within 16 lanes,
// which by then hold equal sums on either side).
template <int CTRL>
__device__ __forceinline__ float delta_dpp(float v) {
  // (every lane has a source lane under these controls; with bound_ctrl set the compiler folds the move into the addition)
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float delta_sum16(float v) {
  v += delta_dpp<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  v += delta_dpp<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  v += delta_dpp<0x141>(v);     // row_half_mirror
  v += delta_dpp<0x140>(v);     // row_mirror
  return v;
}

// The sum over the wave's 64 lanes, in every lane: the rows' sums, then the four rows' through scalar registers.
__device__ __forceinline__ float delta_sum64(float v) {
  v = delta_sum16(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16)) +
         __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32)) + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
}

// prep [H, chunk_rows, block] float32; vals [H, ceil(vdim / 8), val_rows, 8]: the values. A wave a (token, head);
// the wave of a chunk's first token makes the chunk.
template <typename T>
__global__ __launch_bounds__(256) void gated_delta_prepare_kernel(
    const T* __restrict__ qkv, long stride, int q_at, int k_at, int v_at, const float* __restrict__ a, long a_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ b, long b_stride,
    const int* __restrict__ seg_of, const int* __restrict__ seg_starts, float* __restrict__ prep,
    float* __restrict__ vals, int n_tokens, long chunk_rows, long val_rows, int H, int G, int dim, int vdim, int RPL,
    float q_scale, float unit_eps) {
  const long w = (long)blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE;
  const int lane = threadIdx.x % LMSF_WAVE;
  if (w >= (long)n_tokens * H) return;
  const int t = (int)(w / H), h = (int)(w - (long)t * H);
  const int gh = h / (H / G), DP = DELTA_R * RPL, block = 13 * DP + 20;
  const int n_cb = (vdim + DELTA_COLS - 1) / DELTA_COLS;
  const T* vr = qkv + (long)t * stride + v_at + h * vdim;
  for (int j = lane; j < n_cb * DELTA_COLS; j += LMSF_WAVE)
    vals[(((long)h * n_cb + j / DELTA_COLS) * val_rows + t) * DELTA_COLS + j % DELTA_COLS] = j < vdim ? to_f32<T>(vr[j]) : 0.f;
  const int s = seg_of[t], t0 = seg_starts[s], t1 = seg_starts[s + 1];
  if ((t - t0) % DELTA_CHUNK) return;
  const int nt = min(DELTA_CHUNK, t1 - t);
  float iq[DELTA_CHUNK], ik[DELTA_CHUNK];
#pragma unroll
  for (int m = 0; m < DELTA_CHUNK; ++m) {
    float ssq = 0.f, ssk = 0.f;
    if (m < nt) {
      const T* qr = qkv + (long)(t + m) * stride + q_at + gh * dim;
      const T* kr = qkv + (long)(t + m) * stride + k_at + gh * dim;
      for (int i = lane; i < dim; i += LMSF_WAVE) {
        const float x = to_f32<T>(qr[i]), y = to_f32<T>(kr[i]);
        ssq += x * x;
        ssk += y * y;
      }
    }
    iq[m] = q_scale / sqrtf(delta_sum64(ssq) + unit_eps);
    ik[m] = 1.f / sqrtf(delta_sum64(ssk) + unit_eps);
  }
  const float rate = expf(a_log[h]);
  float* out = prep + ((long)h * chunk_rows + delta_chunk_row(t0, s, t)) * block;
  float A[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, B[10] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int p = lane; p < DP; p += LMSF_WAVE) {
    const int i = (p % RPL) * DELTA_R + p / RPL;
    float k[DELTA_CHUNK], q[DELTA_CHUNK], lg[DELTA_CHUNK];        // lg: the logarithm of the token's decay (<= 0)
#pragma unroll
    for (int m = 0; m < DELTA_CHUNK; ++m) {
      k[m] = q[m] = lg[m] = 0.f;
      if (m < nt && i < dim) {
        k[m] = to_f32<T>(qkv[(long)(t + m) * stride + k_at + gh * dim + i]) * ik[m];
        q[m] = to_f32<T>(qkv[(long)(t + m) * stride + q_at + gh * dim + i]) * iq[m];
        lg[m] = -rate * softplus_f32(a[(long)(t + m) * a_stride + h * dim + i] + dt_bias[h * dim + i]);
      }
    }
    // every exponent is a sum of the logarithms it spans, added up directly (not a difference of running sums)
    float head = 0.f;
#pragma unroll
    for (int m = 0; m < DELTA_CHUNK; ++m) {
      head += lg[m];                                   // G_m
      float tail = 0.f;                                // G_4 - G_m
#pragma unroll
      for (int j = m + 1; j < DELTA_CHUNK; ++j) tail += lg[j];
      const float e = expf(head);
      out[m * DP + p] = k[m] * e;
      out[(4 + m) * DP + p] = q[m] * e;
      out[(8 + m) * DP + p] = k[m] * expf(tail);
      if (m == DELTA_CHUNK - 1) out[12 * DP + p] = e;
    }
    int ia = 0, ib = 0;
#pragma unroll
    for (int x = 0; x < DELTA_CHUNK; ++x)
#pragma unroll
      for (int m = 0; m <= x; ++m) {
        float span = 0.f;                              // G_x - G_m
#pragma unroll
        for (int j = m + 1; j <= x; ++j) span += lg[j];
        const float km = k[m] * expf(span);
        if (m < x) A[ia++] += k[x] * km;
        B[ib++] += q[x] * km;
      }
  }
#pragma unroll
  for (int j = 0; j < 6; ++j) A[j] = delta_sum64(A[j]);
#pragma unroll
  for (int j = 0; j < 10; ++j) B[j] = delta_sum64(B[j]);
  if (lane == 0) {
    float* sc = out + 13 * DP;
#pragma unroll
    for (int m = 0; m < DELTA_CHUNK; ++m) sc[m] = m < nt ? 1.f / (1.f + expf(-b[(long)(t + m) * b_stride + h])) : 0.f;
#pragma unroll
    for (int j = 0; j < 6; ++j) sc[4 + j] = A[j];
#pragma unroll
    for (int j = 0; j < 10; ++j) sc[10 + j] = B[j];
  }
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

// HC: chunks a batch holds (and LDS has room for, twice): delta_batch_chunks(RPL) for portions of prompts; 1 for a step
// whose segments hold no more than a chunk (single tokens), where a workgroup then takes a few KB of LDS instead of
// 59 and many of them share a compute unit.
template <int RPL, int HC>
__global__ __launch_bounds__(DELTA_WAVES * LMSF_WAVE) void gated_delta_recurrence_kernel(
    const float* __restrict__ prep, const float* __restrict__ vals, long chunk_rows, long val_rows,
    float* __restrict__ state, long state_stride, const int* __restrict__ seg_starts, const int* __restrict__ slots,
    float* __restrict__ out, long out_stride, int H, int dim, int vdim) {
  constexpr int DP = DELTA_R * RPL, BLOCK = delta_block_floats(RPL), HT = HC * DELTA_CHUNK;
  constexpr int OPS_BYTES = (HC * BLOCK * 4 + 1023) / 1024 * 1024, VAL_BYTES = (HT * DELTA_COLS * 4 + 1023) / 1024 * 1024;
  constexpr int N_OPS = OPS_BYTES / 1024, N_VAL = VAL_BYTES / 1024;     // transfers of 1 KB a batch
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // two buffers of [chunks | values], two of results
  float* results = reinterpret_cast<float*>(lds + 2 * (OPS_BYTES + VAL_BYTES));          // [2][HT][DELTA_COLS]
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
  const unsigned char* g_ops = reinterpret_cast<const unsigned char*>(
      prep + ((long)h * chunk_rows + delta_chunk_row(t0, s, t0)) * BLOCK);
  const unsigned char* g_val = reinterpret_cast<const unsigned char*>(vals + (((long)h * n_cb + cb) * val_rows + t0) * DELTA_COLS);
  const unsigned lds0 = delta_lds_address(lds);
  const int n_tok = t1 - t0, n_batches = (n_tok + HT - 1) / HT;
  auto transfer = [&](int batch, int buf) {
    // (only what the batch holds)
    const int toks = min(HT, n_tok - batch * HT), chunks = (toks + DELTA_CHUNK - 1) / DELTA_CHUNK;
    const int n_ops = min(N_OPS, (chunks * BLOCK * 4 + 1023) / 1024), n_val = min(N_VAL, (toks * DELTA_COLS * 4 + 1023) / 1024);
    const unsigned base = lds0 + buf * (OPS_BYTES + VAL_BYTES);
    const int first = __builtin_amdgcn_readfirstlane(wave);          // (the same in every lane: the LDS base is a scalar)
    for (int n = first; n < n_ops; n += DELTA_WAVES)
      delta_global_to_lds_16(g_ops + (long)batch * HC * BLOCK * 4 + n * 1024 + lane * 16,
                             __builtin_amdgcn_readfirstlane(base + n * 1024));
    for (int n = first; n < n_val; n += DELTA_WAVES)
      delta_global_to_lds_16(g_val + (long)batch * HT * DELTA_COLS * 4 + n * 1024 + lane * 16,
                             __builtin_amdgcn_readfirstlane(base + OPS_BYTES + n * 1024));
  };
  // A batch's results wait in LDS and go to memory while the next batch is worked on: stored as they come, the wait
  // for the next batch's operands would also wait for the stores just issued, a trip to memory every batch.
  auto flush = [&](int batch) {
    const float* from = results + (batch & 1) * HT * DELTA_COLS;
    const int n = min(HT, n_tok - batch * HT) * DELTA_COLS;
    for (int e = tid; e < n; e += DELTA_WAVES * LMSF_WAVE) {
      const int column = cb * DELTA_COLS + e % DELTA_COLS;
      if (column < vdim) out[((long)t0 + (long)batch * HT + e / DELTA_COLS) * out_stride + h * vdim + column] = from[e];
    }
  };
  transfer(0, 0);
  for (int bt = 0; bt < n_batches; ++bt) {
    const int buf = bt & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                   // this batch has landed; everybody is done with the buffer of the one before
    if (bt + 1 < n_batches) transfer(bt + 1, buf ^ 1);
    if (bt > 0) flush(bt - 1);
    float* res = results + buf * HT * DELTA_COLS;
    const float* ops_ = reinterpret_cast<const float*>(lds + buf * (OPS_BYTES + VAL_BYTES));
    const float* val_ = reinterpret_cast<const float*>(lds + buf * (OPS_BYTES + VAL_BYTES) + OPS_BYTES);
    const int left = n_tok - bt * HT;                              // tokens from this batch's first on
    const int nc = min(HC, (left + DELTA_CHUNK - 1) / DELTA_CHUNK);
    for (int jc = 0; jc < nc; ++jc) {
      const float* blk = ops_ + jc * BLOCK;
      float rs[DELTA_CHUNK], ps[DELTA_CHUNK];
#pragma unroll
      for (int m = 0; m < DELTA_CHUNK; ++m) {
        float kh[RPL], qh[RPL];
        delta_load_vec<RPL>(kh, blk + m * DP + r * RPL);
        delta_load_vec<RPL>(qh, blk + (4 + m) * DP + r * RPL);
        float x = 0.f, y = 0.f;
#pragma unroll
        for (int ii = 0; ii < RPL; ++ii) {
          x = fmaf(kh[ii], st[ii], x);
          y = fmaf(qh[ii], st[ii], y);
        }
        rs[m] = x;
        ps[m] = y;
      }
#pragma unroll
      for (int m = 0; m < DELTA_CHUNK; ++m) {
        rs[m] = delta_sum16(rs[m]);
        ps[m] = delta_sum16(ps[m]);
      }
      float sc[20];                                                // beta [4], A [6], B [10]
      delta_load_vec<20>(sc, blk + 13 * DP);
      float u[DELTA_CHUNK], o[DELTA_CHUNK];
      int ia = 0, ib = 0;
#pragma unroll
      for (int x = 0; x < DELTA_CHUNK; ++x) {
        // (a token beyond the segment's end has beta = 0; its value is whatever lies there and must not be read as one)
        const float v = jc * DELTA_CHUNK + x < left ? val_[(jc * DELTA_CHUNK + x) * DELTA_COLS + wave * DELTA_CPW + c] : 0.f;
        float d = v - rs[x];
#pragma unroll
        for (int m = 0; m < x; ++m) d = fmaf(-sc[4 + ia++], u[m], d);
        u[x] = sc[x] * d;
        float acc = ps[x];
#pragma unroll
        for (int m = 0; m <= x; ++m) acc = fmaf(sc[10 + ib++], u[m], acc);
        o[x] = acc;
      }
      float gl[RPL];
      delta_load_vec<RPL>(gl, blk + 12 * DP + r * RPL);
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) st[ii] *= gl[ii];
#pragma unroll
      for (int m = 0; m < DELTA_CHUNK; ++m) {
        float kl[RPL];
        delta_load_vec<RPL>(kl, blk + (8 + m) * DP + r * RPL);
#pragma unroll
        for (int ii = 0; ii < RPL; ++ii) st[ii] = fmaf(kl[ii], u[m], st[ii]);
      }
      // every lane of a column holds the four results: lane r < 4 of the column stores token r's (one store a chunk)
      const float mine = r == 0 ? o[0] : r == 1 ? o[1] : r == 2 ? o[2] : o[3];
      if (r < DELTA_CHUNK) res[(jc * DELTA_CHUNK + r) * DELTA_COLS + wave * DELTA_CPW + c] = mine;
    }
  }
  __syncthreads();
  flush(n_batches - 1);
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

static inline long delta_chunk_rows(int n_tokens, int n_segments, int rpl) {
  return (long)n_tokens / DELTA_CHUNK + n_segments + 1 + delta_batch_chunks(rpl);
}
static inline long delta_val_rows(int n_tokens, int rpl) { return (long)n_tokens + delta_batch_chunks(rpl) * DELTA_CHUNK; }

// floats of scratch for a step: what the first kernel hands the second (a batch of rows more per head than the step
// needs, and a transfer's length at the end, so that a batch may be fetched whole wherever it begins)
extern "C" long lmsf_gated_delta_scratch_floats(int n_tokens, int n_segments, int H, int dim, int vdim) {
  const int rpl = delta_rows_per_lane(dim);
  const long n_cb = (vdim + DELTA_COLS - 1) / DELTA_COLS;
  return (long)H * delta_chunk_rows(n_tokens, n_segments, rpl) * delta_block_floats(rpl) + 256 +
         (long)H * n_cb * delta_val_rows(n_tokens, rpl) * DELTA_COLS + 256;
}

template <int RPL, int HC>
static int launch_delta_recurrence(dim3 grid, hipStream_t stream, const float* prep, const float* vals, long chunk_rows,
                                   long val_rows, float* state, long state_stride, const int* seg_starts,
                                   const int* slots, float* out, long out_stride, int H, int dim, int vdim) {
  constexpr int BLOCK = delta_block_floats(RPL), HT = HC * DELTA_CHUNK;
  constexpr size_t smem = 2 * ((size_t)(HC * BLOCK * 4 + 1023) / 1024 * 1024 + (size_t)(HT * DELTA_COLS * 4 + 1023) / 1024 * 1024) +
                          2 * (size_t)HT * DELTA_COLS * 4;
  auto kernel = gated_delta_recurrence_kernel<RPL, HC>;
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
  hipLaunchKernelGGL(kernel, grid, dim3(DELTA_WAVES * LMSF_WAVE), smem, stream, prep, vals, chunk_rows, val_rows, state,
                     state_stride, seg_starts, slots, out, out_stride, H, dim, vdim);
  return 0;
}

// qkv: the (convolved, activated) q [N, G dim], k [N, G dim], v [N, H vdim] as columns q_at, k_at, v_at of one buffer
// of ``dtype`` with row stride ``stride``; a: float32 [N, H dim] before bias and softplus; dt_bias float32 [H dim];
// a_log float32 [H]; b: float32 [N, >= H] before the sigmoid; state float32 [slots, >= lmsf_gated_delta_state_floats];
// seg_of [N], seg_starts [S + 1], slots [S]: the step's segments; longest: the most tokens a segment holds, if the caller
// knows (0: not known); scratch: lmsf_gated_delta_scratch_floats floats,
// 16-byte aligned; out: float32 [N, H vdim], the heads' read-outs as they are.
extern "C" int lmsf_gated_delta(const void* qkv, int dtype, long stride, int q_at, int k_at, int v_at, const float* a,
                                long a_stride, const float* dt_bias, const float* a_log, const float* b,
                                long b_stride, float* state, long state_stride, const int* seg_of,
                                const int* seg_starts, const int* slots, float* scratch, float* out, long out_stride,
                                int n_tokens, int n_segments, int longest, int H, int G, int dim, int vdim,
                                float q_scale, float unit_eps, hipStream_t stream) {
  LMSF_CHECK(qkv && a && dt_bias && a_log && b && state && seg_of && seg_starts && slots && out && scratch,
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
  const long chunk_rows = delta_chunk_rows(n_tokens, n_segments, RPL), val_rows = delta_val_rows(n_tokens, RPL);
  float* prep = scratch;
  float* vals = scratch + (long)H * chunk_rows * delta_block_floats(RPL) + 256;
  const dim3 g1((unsigned)(((long)n_tokens * H + 3) / 4)), g2(n_segments, H, n_cb);
#define DELTA_PREP(T)                                                                                               \
  hipLaunchKernelGGL((gated_delta_prepare_kernel<T>), g1, dim3(256), 0, stream, (const T*)qkv, stride, q_at, k_at,   \
                     v_at, a, a_stride, dt_bias, a_log, b, b_stride, seg_of, seg_starts, prep, vals, n_tokens,      \
                     chunk_rows, val_rows, H, G, dim, vdim, RPL, q_scale, unit_eps)
  if (dtype == LMSF_F32) DELTA_PREP(float);
  else DELTA_PREP(bf16_t);
#undef DELTA_PREP
#define DELTA_RUN(R)                                                                                                   \
  (small ? launch_delta_recurrence<R, 1>(g2, stream, prep, vals, chunk_rows, val_rows, state, state_stride, seg_starts, \
                                         slots, out, out_stride, H, dim, vdim)                                         \
         : launch_delta_recurrence<R, delta_batch_chunks(R)>(g2, stream, prep, vals, chunk_rows, val_rows, state,      \
                                                             state_stride, seg_starts, slots, out, out_stride, H, dim, \
                                                             vdim))
  const bool small = longest > 0 && longest <= DELTA_CHUNK;
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
