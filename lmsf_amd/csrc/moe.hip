// Experts chosen by a table: token id t runs the ``top`` experts table[t, 0 .. top-1], each a gated feed-forward
//     y_e(h) = Wd_e (silu(Wg_e h) * (Wu_e h)),
// and the layer's output is base + weight * sum_k y_{table[t, k]}(h) (base: what runs for every token, or nothing).
// The choice is read on the device from the step's token ids, so a step needs nothing from the host and can be
// replayed from a graph. The experts' matrices lie stacked: Wgu [E, 2 F, W] (gate rows, then up rows), Wd [E, W, F].
//
// Few tokens (decoding), and float32 at any number: every (token, choice) streams its expert's rows, a wave per
// output, the token's vector in LDS, 16-byte loads where the rows allow them.
// Many tokens in bfloat16: the (token, choice) pairs are grouped by expert on the device (one small kernel: counts,
// offsets, an order, a list of tiles of up to 128 pairs of one expert), and each tile runs on the matrix cores
// against 128 of its expert's outputs (A = 16 rows of W x 32 k, B = 16 pairs x 32 k; in the gated product the gate
// and the up rows of the same outputs), operands through LDS. The down product leaves float32 rows per pair; a last kernel adds a token's pairs and the shared part. A pair's result
// does not depend on where in its tile it lies, so the order inside an expert's group (atomic counters) is free.
// Accumulation in float32 throughout.
//
// The same kernels serve experts that a router chooses: ``ids`` null makes row n of the table token n's own choice (a
// table [n_tokens, top] that a kernel of the step has just written, lmsf_moe_route below); ``pair_scale`` gives every
// (token, choice) a float32 factor on the expert's *input*, y_e(s h), which the gate and up products take as a factor on
// their results before these are rounded (W (s h) = s (W h)); ``base_scale`` a float32 factor per token on ``base``;
// ``out_scale`` a float32 factor per (token, choice) on what the expert returns. Experts may also be of one matrix in,
// y_e(h) = Wd_e relu(Wu_e h)^2 with Wgu [E, F, W] (lmsf_table_moe_act). A second router (lmsf_moe_route_groups) takes
// softmax scores and chooses within the best groups of neighbouring experts.
#include "common.h"

#include <math.h>

#define MOE_THREADS 256
#define MOE_WAVES (MOE_THREADS / LMSF_WAVE)
#define MOE_OUT_PER_WAVE 4

// NR rows of a matrix against one vector: out[r] = sum_i w[r * ld + i] x[i] over W entries, the lanes of a wave
// together; x in LDS as float32. The loads of all rows are asked for before any is used (rows beyond ``valid`` repeat
// the last valid one).
template <typename T, int NR>
__device__ __forceinline__ void moe_rows_dot(const T* __restrict__ w, long ld, int valid, const float* __restrict__ x,
                                             int W, int lane, bool vec, float* out) {
  float a[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) a[r] = 0.f;
  if (vec) {
    constexpr int V = Vec16<T>::N;
    for (int i = lane * V; i < W; i += LMSF_WAVE * V) {
      Vec16<T> p[NR];
#pragma unroll
      for (int r = 0; r < NR; ++r) p[r].load(w + (long)min(r, valid - 1) * ld + i);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float xv = x[i + e];
#pragma unroll
        for (int r = 0; r < NR; ++r) a[r] += p[r].get(e) * xv;
      }
    }
  } else {
    for (int i = lane; i < W; i += LMSF_WAVE) {
      const float xv = x[i];
#pragma unroll
      for (int r = 0; r < NR; ++r) a[r] += to_f32<T>(w[(long)min(r, valid - 1) * ld + i]) * xv;
    }
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) out[r] = wave_sum(a[r]);
}

// act[(n * top + k), f] = silu(Wg_e[f] . h[n]) * (Wu_e[f] . h[n]),  e = table[ids[n], k]
template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_gate_up_kernel(
    const T* __restrict__ h, long h_stride, const T* __restrict__ Wgu, const int* __restrict__ ids,
    const int* __restrict__ table, int vocab, int top, int E, T* __restrict__ act, int F, int W, int vec,
    const float* __restrict__ pair_scale, int gated) {
  extern __shared__ float sh[];   // [W]
  const int nk = blockIdx.x, n = nk / top, k = nk - n * top;
  const int id = min(max(ids ? ids[n] : n, 0), vocab - 1);
  const int e = min(max(table[(long)id * top + k], 0), E - 1);
  const float ps = pair_scale ? pair_scale[nk] : 1.f;
  for (int i = threadIdx.x; i < W; i += MOE_THREADS) sh[i] = ps * to_f32<T>(h[(long)n * h_stride + i]);
  __syncthreads();
  const int wave = threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  const int f0 = (blockIdx.y * MOE_WAVES + wave) * MOE_OUT_PER_WAVE;
  const T* We = Wgu + (long)e * (gated ? 2 : 1) * F * W;
  if (f0 >= F) return;
  const int valid = min(MOE_OUT_PER_WAVE, F - f0);
  float ag[MOE_OUT_PER_WAVE], au[MOE_OUT_PER_WAVE];
  moe_rows_dot<T, MOE_OUT_PER_WAVE>(We + (long)f0 * W, W, valid, sh, W, lane, vec, ag);
  if (!gated) {
    // one matrix an expert: act = relu(W_up h)^2, the product rounded as a stored activation is
    if (lane < valid) {
      float uu = 0.f;
#pragma unroll
      for (int r = 0; r < MOE_OUT_PER_WAVE; ++r)
        if (r == lane) uu = fmaxf(to_f32<T>(from_f32<T>(ag[r])), 0.f);
      act[(long)nk * F + f0 + lane] = from_f32<T>(uu * uu);
    }
    return;
  }
  moe_rows_dot<T, MOE_OUT_PER_WAVE>(We + (long)(F + f0) * W, W, valid, sh, W, lane, vec, au);
  if (lane < valid) {
    // the two products are rounded as stored activations are, then the activation in float32
    float gg = 0.f, uu = 0.f;
#pragma unroll
    for (int r = 0; r < MOE_OUT_PER_WAVE; ++r)
      if (r == lane) {
        gg = to_f32<T>(from_f32<T>(ag[r]));
        uu = to_f32<T>(from_f32<T>(au[r]));
      }
    act[(long)nk * F + f0 + lane] = from_f32<T>(gg / (1.f + expf(-gg)) * uu);
  }
}

// out[n, o] = base[n, o] + weight * sum_k Wd_{e_k}[o] . act[n * top + k]
template <typename T>
__global__ __launch_bounds__(MOE_THREADS) void moe_down_kernel(
    const T* __restrict__ act, const T* __restrict__ Wd, const int* __restrict__ ids, const int* __restrict__ table,
    int vocab, int top, int E, float weight, const T* __restrict__ base, long base_stride, T* __restrict__ out,
    long out_stride, int F, int W, int vec, const float* __restrict__ base_scale,
    const float* __restrict__ out_scale) {
  extern __shared__ float sa[];   // [top, F]
  const int n = blockIdx.x;
  const int id = min(max(ids ? ids[n] : n, 0), vocab - 1);
  for (int i = threadIdx.x; i < top * F; i += MOE_THREADS) sa[i] = to_f32<T>(act[(long)n * top * F + i]);
  __syncthreads();
  const int wave = threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  const int o0 = (blockIdx.y * MOE_WAVES + wave) * MOE_OUT_PER_WAVE;
  if (o0 >= W) return;
  const int valid = min(MOE_OUT_PER_WAVE, W - o0);
  float total[MOE_OUT_PER_WAVE];
#pragma unroll
  for (int r = 0; r < MOE_OUT_PER_WAVE; ++r) total[r] = 0.f;
  for (int k = 0; k < top; ++k) {
    const int e = min(max(table[(long)id * top + k], 0), E - 1);
    float part[MOE_OUT_PER_WAVE];
    const float os = out_scale ? out_scale[(long)n * top + k] : 1.f;
    moe_rows_dot<T, MOE_OUT_PER_WAVE>(Wd + ((long)e * W + o0) * F, F, valid, sa + k * F, F, lane, vec, part);
#pragma unroll
    for (int r = 0; r < MOE_OUT_PER_WAVE; ++r) total[r] += os * part[r];
  }
  if (lane < valid) {
    float mine = 0.f;
#pragma unroll
    for (int r = 0; r < MOE_OUT_PER_WAVE; ++r)
      if (r == lane) mine = total[r];
    float b = base ? to_f32<T>(base[(long)n * base_stride + o0 + lane]) : 0.f;
    if (base_scale) b *= base_scale[n];
    out[(long)n * out_stride + o0 + lane] = from_f32<T>(b + weight * mine);
  }
}

// ---------------------------------------------------------------- many tokens: grouped by expert, matrix cores

#define MOE_TILE 128         // pairs a tile holds

// Groups the P = N * top pairs by expert. order[i]: the pair at place i of the grouped sequence; tiles: for every
// tile (of up to ``tile_pairs`` pairs) its expert, its first place and its number of pairs; n_tiles[0]: how many
// tiles there are. One workgroup.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ ids, const int* __restrict__ table,
                                                        int vocab, int top, int E, int P, int tile_pairs,
                                                        int* __restrict__ order, int* __restrict__ tiles,
                                                        int* __restrict__ n_tiles) {
  extern __shared__ int sm[];   // [E] counts, [E] first places, [E] fill counters
  int* cnt = sm;
  int* first = sm + E;
  int* fill = sm + 2 * E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = fill[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int id = min(max(ids ? ids[p / top] : p / top, 0), vocab - 1);
    atomicAdd(&cnt[min(max(table[(long)id * top + p % top], 0), E - 1)], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      first[e] = at;
      for (int s = 0; s < cnt[e]; s += tile_pairs) {
        tiles[3 * t] = e;
        tiles[3 * t + 1] = at + s;
        tiles[3 * t + 2] = min(tile_pairs, cnt[e] - s);
        ++t;
      }
      at += cnt[e];
    }
    n_tiles[0] = t;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int id = min(max(ids ? ids[p / top] : p / top, 0), vocab - 1);
    const int e = min(max(table[(long)id * top + p % top], 0), E - 1);
    order[first[e] + atomicAdd(&fill[e], 1)] = p;
  }
}

// One tile of up to 128 pairs against 128 outputs of its expert, operands through LDS. GATED: x = the tokens' vectors
// (row of pair p: p / top), Wm = Wgu, K = W, O = F, y = act [P, F] bfloat16 = silu(gate) * up; else x = act (row of pair
// p: p), Wm = Wd, K = F, O = W, y = float32 rows [P, W]. A step of 32 k: the workgroup copies the rows of W (128, or 128 gate + 128 up) and the 128 pairs' rows, 64 bytes of each, into
// LDS with 16-byte loads (the next step's while this step is multiplied: two buffers, one barrier a step), and every
// wave of the 2 x 2 reads the fragments of its 64 pairs and 64 outputs from there (rows of 64 bytes back to back: a
// fragment's 64 lanes read 1 KB in a row, no bank conflicts). A first form whose waves fetched their fragments
// themselves, straight from memory in tiles of 64 pairs, did 2.7 times fewer multiplications per byte fetched and lost
// at every number of pairs: 2,048 tokens (256 pairs an expert) 319 against 194 us for the four kernels, 512 tokens 230
// against 98, 64 tokens (8 pairs an expert, every tile mostly empty) 101 against 83.

// KIND 0: the down product; 1: gate and up with silu(gate) * up; 2: one matrix an expert (Wm [E, O, K]) with relu(.)^2.
template <int KIND>
__global__ __launch_bounds__(256) void moe_tile_lds_kernel(const bf16_t* __restrict__ x, long x_stride, int top,
                                                           const bf16_t* __restrict__ Wm, const int* __restrict__ order,
                                                           const int* __restrict__ tiles, const int* __restrict__ n_tiles,
                                                           void* __restrict__ y, int O, int K,
                                                           const float* __restrict__ pair_scale) {
  constexpr bool GATED = KIND == 1, UP = KIND != 0;
  constexpr int AR = GATED ? 256 : 128;            // rows of W a step
  constexpr int NLA = AR * 4 / 256;                // 16-byte pieces of W a thread copies a step
  constexpr int NLB = MOE_TILE * 4 / 256;      // and of the pairs' rows
  constexpr int NA = GATED ? 8 : 4;                // fragments of W a wave
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(16))) unsigned char lds[2][(AR + MOE_TILE) * 64];
  const int t = blockIdx.x;
  if (t >= n_tiles[0]) return;
  const int e = tiles[3 * t], place = tiles[3 * t + 1], count = tiles[3 * t + 2];
  const int tid = threadIdx.x, wave = tid / LMSF_WAVE, lane = tid % LMSF_WAVE;
  const int fr = lane % 16, fg = lane / 16;
  const int wr = wave / 2, wc = wave % 2;          // the wave's 64 pairs and 64 outputs
  const int o_base = blockIdx.y * 128;
  // what this thread copies: piece (tid % 4) of rows tid / 4, + 64, ...
  const bf16_t* ga[NLA];
  const bf16_t* gb[NLB];
#pragma unroll
  for (int i = 0; i < NLA; ++i) {
    const int r = tid / 4 + i * 64;                // 0 .. AR-1; gated: rows 128 .. 255 are the up rows
    const int o = min(o_base + (r & 127), O - 1);
    ga[i] = Wm + ((long)e * (GATED ? 2 : 1) * O + (GATED && r >= 128 ? O : 0) + o) * K + (tid % 4) * 8;
  }
#pragma unroll
  for (int i = 0; i < NLB; ++i) {
    const int p = order[place + min(tid / 4 + i * 64, count - 1)];
    gb[i] = x + (long)(UP ? p / top : p) * x_stride + (tid % 4) * 8;
  }
  f32x4_t acc[NA][4];
#pragma unroll
  for (int a = 0; a < NA; ++a)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[a][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  u32x4 ra[NLA], rb[NLB];
#pragma unroll
  for (int i = 0; i < NLA; ++i) ra[i] = *reinterpret_cast<const u32x4*>(ga[i]);
#pragma unroll
  for (int i = 0; i < NLB; ++i) rb[i] = *reinterpret_cast<const u32x4*>(gb[i]);
#pragma unroll
  for (int i = 0; i < NLA; ++i) *reinterpret_cast<u32x4*>(lds[0] + (tid / 4 + i * 64) * 64 + (tid % 4) * 16) = ra[i];
#pragma unroll
  for (int i = 0; i < NLB; ++i) *reinterpret_cast<u32x4*>(lds[0] + (AR + tid / 4 + i * 64) * 64 + (tid % 4) * 16) = rb[i];
  __syncthreads();
  int cur = 0;
  for (int k = 0; k < K; k += 32) {
    const bool more = k + 32 < K;
    if (more) {
#pragma unroll
      for (int i = 0; i < NLA; ++i) ra[i] = *reinterpret_cast<const u32x4*>(ga[i] + k + 32);
#pragma unroll
      for (int i = 0; i < NLB; ++i) rb[i] = *reinterpret_cast<const u32x4*>(gb[i] + k + 32);
    }
    const unsigned char* buf = lds[cur];
    bf16x8_t fa[NA], fb[4];
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      // fragment a: outputs wc * 64 + (a % 4) * 16 ..; gated: a >= 4 are the up rows of the same outputs
      const int row = (GATED && a >= 4 ? 128 : 0) + wc * 64 + (a & 3) * 16 + fr;
      fa[a] = *reinterpret_cast<const bf16x8_t*>(buf + row * 64 + fg * 16);
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
      fb[mt] = *reinterpret_cast<const bf16x8_t*>(buf + (AR + wr * 64 + mt * 16 + fr) * 64 + fg * 16);
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[a][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[a], fb[mt], acc[a][mt], 0, 0, 0);
    if (more) {
      unsigned char* nxt = lds[cur ^ 1];
#pragma unroll
      for (int i = 0; i < NLA; ++i) *reinterpret_cast<u32x4*>(nxt + (tid / 4 + i * 64) * 64 + (tid % 4) * 16) = ra[i];
#pragma unroll
      for (int i = 0; i < NLB; ++i) *reinterpret_cast<u32x4*>(nxt + (AR + tid / 4 + i * 64) * 64 + (tid % 4) * 16) = rb[i];
    }
    __syncthreads();
    cur ^= 1;
  }
  // lane: pair wr * 64 + mt * 16 + fr, outputs o_base + wc * 64 + a * 16 + fg * 4 .. + 3
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int slot = wr * 64 + mt * 16 + fr;
    if (slot >= count) continue;
    const int p = order[place + slot];
    const float ps = UP && pair_scale ? pair_scale[p] : 1.f;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int o = o_base + wc * 64 + a * 16 + fg * 4 + j;
        if (o >= O) continue;
        if (GATED) {
          const float g = bf16_to_f32(f32_to_bf16(ps * acc[a][mt][j])), u = bf16_to_f32(f32_to_bf16(ps * acc[NA - 4 + a][mt][j]));
          reinterpret_cast<bf16_t*>(y)[(long)p * O + o] = f32_to_bf16(g / (1.f + expf(-g)) * u);
        } else if (UP) {
          const float u = fmaxf(bf16_to_f32(f32_to_bf16(ps * acc[a][mt][j])), 0.f);
          reinterpret_cast<bf16_t*>(y)[(long)p * O + o] = f32_to_bf16(u * u);
        } else {
          reinterpret_cast<float*>(y)[(long)p * O + o] = acc[a][mt][j];
        }
      }
  }
}

// out[n, o] = base[n, o] + weight * sum_k rows[n * top + k, o]
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ rows, int top, float weight,
                                                          const bf16_t* __restrict__ base, long base_stride,
                                                          bf16_t* __restrict__ out, long out_stride, int W,
                                                          const float* __restrict__ base_scale,
                                                          const float* __restrict__ out_scale) {
  const int n = blockIdx.x;
  const float bs = base_scale ? base_scale[n] : 1.f;
  for (int o = threadIdx.x; o < W; o += 256) {
    float s = 0.f;
    for (int k = 0; k < top; ++k)
      s += (out_scale ? out_scale[(long)n * top + k] : 1.f) * rows[((long)n * top + k) * W + o];
    const float b = base ? bs * bf16_to_f32(base[(long)n * base_stride + o]) : 0.f;
    out[(long)n * out_stride + o] = f32_to_bf16(b + weight * s);
  }
}

// ints and floats of scratch that the grouped form needs for n_tokens tokens
extern "C" long lmsf_table_moe_scratch_ints(int n_tokens, int top, int E) {
  const long P = (long)n_tokens * top;
  return P + 3 * (P / MOE_TILE + E + 1) + 4;
}

// whether lmsf_table_moe takes the grouped form for these sizes (then it needs the scratch: ints as above,
// floats n_tokens * top * W)
extern "C" int lmsf_table_moe_grouped(int dtype, int n_tokens, int top, int E, int F, int W, long h_stride) {
  return dtype == LMSF_BF16 && (long)n_tokens * top >= 32 && W % 32 == 0 && F % 32 == 0 && h_stride % 8 == 0 &&
         E <= 4096;
}

// ``act_kind`` 0: gated experts, Wgu [E, 2 F, W]; 1: experts of one matrix, Wgu [E, F, W], y_e(h) = Wd_e relu(Wu_e h)^2.
// ``out_scale``: a float32 factor per (token, choice) on what the expert returns (null: none).
extern "C" int lmsf_table_moe_act(const void* h, int dtype, long h_stride, const void* Wgu, const void* Wd,
                                  const int* ids, const int* table, int vocab, int top, int E, float weight,
                                  const void* base, long base_stride, const float* pair_scale,
                                  const float* base_scale, const float* out_scale, int act_kind, void* act, void* out,
                                  long out_stride, int n_tokens, int F, int W, int* scratch_ints,
                                  float* scratch_rows, hipStream_t stream) {
  LMSF_CHECK(act_kind == 0 || act_kind == 1, "table_moe: unknown kind of expert %d", act_kind);
  const int gated = act_kind == 0;
  LMSF_CHECK(h && Wgu && Wd && table && act && out, "table_moe: null pointer");
  LMSF_CHECK(ids || vocab >= n_tokens, "table_moe: without token ids the table has a row per token");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "table_moe: unknown dtype code %d", dtype);
  LMSF_CHECK(vocab > 0 && top > 0 && E > 0 && F > 0 && W > 0, "table_moe: bad sizes");
  LMSF_CHECK(h_stride >= W && out_stride >= W && (!base || base_stride >= W), "table_moe: rows overlap");
  LMSF_CHECK((size_t)W * 4 <= 64 * 1024 && (size_t)top * F * 4 <= 64 * 1024, "table_moe: a row does not fit LDS");
  LMSF_CHECK((long)n_tokens * top < 2147483647L, "table_moe: too many rows");
  if (n_tokens <= 0) return 0;
  if (lmsf_table_moe_grouped(dtype, n_tokens, top, E, F, W, h_stride) && scratch_ints && scratch_rows &&
      lmsf_aligned16(h) && lmsf_aligned16(Wgu) && lmsf_aligned16(Wd) && lmsf_aligned16(act)) {
    const int P = n_tokens * top, max_tiles = P / MOE_TILE + E;
    int* order = scratch_ints;
    int* tiles = order + P;
    int* n_tiles = tiles + 3 * (max_tiles + 1);
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), (size_t)3 * E * 4, stream, ids, table, vocab, top, E, P,
                       MOE_TILE, order, tiles, n_tiles);
    if (gated)
      hipLaunchKernelGGL((moe_tile_lds_kernel<1>), dim3(max_tiles, (F + 127) / 128), dim3(256), 0, stream,
                         (const bf16_t*)h, h_stride, top, (const bf16_t*)Wgu, order, tiles, n_tiles, act, F, W, pair_scale);
    else
      hipLaunchKernelGGL((moe_tile_lds_kernel<2>), dim3(max_tiles, (F + 127) / 128), dim3(256), 0, stream,
                         (const bf16_t*)h, h_stride, top, (const bf16_t*)Wgu, order, tiles, n_tiles, act, F, W, pair_scale);
    hipLaunchKernelGGL((moe_tile_lds_kernel<0>), dim3(max_tiles, (W + 127) / 128), dim3(256), 0, stream,
                       (const bf16_t*)act, (long)F, top, (const bf16_t*)Wd, order, tiles, n_tiles, (void*)scratch_rows, W,
                       F, (const float*)nullptr);
    hipLaunchKernelGGL(moe_combine_kernel, dim3(n_tokens), dim3(256), 0, stream, scratch_rows, top, weight,
                       (const bf16_t*)base, base_stride, (bf16_t*)out, out_stride, W, base_scale, out_scale);
    LMSF_LAUNCH_CHECK("table_moe (grouped)");
    return 0;
  }
  const int per_block = MOE_WAVES * MOE_OUT_PER_WAVE;
  const dim3 g1(n_tokens * top, (F + per_block - 1) / per_block), g2(n_tokens, (W + per_block - 1) / per_block);
  const int es = lmsf_elem_size(dtype), vn = 16 / es;
  const int vec1 = W % vn == 0 && lmsf_aligned16(Wgu), vec2 = F % vn == 0 && lmsf_aligned16(Wd);
  if (dtype == LMSF_F32) {
    hipLaunchKernelGGL((moe_gate_up_kernel<float>), g1, dim3(MOE_THREADS), (size_t)W * 4, stream, (const float*)h,
                       h_stride, (const float*)Wgu, ids, table, vocab, top, E, (float*)act, F, W, vec1, pair_scale, gated);
    hipLaunchKernelGGL((moe_down_kernel<float>), g2, dim3(MOE_THREADS), (size_t)top * F * 4, stream, (const float*)act,
                       (const float*)Wd, ids, table, vocab, top, E, weight, (const float*)base, base_stride,
                       (float*)out, out_stride, F, W, vec2, base_scale, out_scale);
  } else {
    hipLaunchKernelGGL((moe_gate_up_kernel<bf16_t>), g1, dim3(MOE_THREADS), (size_t)W * 4, stream, (const bf16_t*)h,
                       h_stride, (const bf16_t*)Wgu, ids, table, vocab, top, E, (bf16_t*)act, F, W, vec1, pair_scale, gated);
    hipLaunchKernelGGL((moe_down_kernel<bf16_t>), g2, dim3(MOE_THREADS), (size_t)top * F * 4, stream,
                       (const bf16_t*)act, (const bf16_t*)Wd, ids, table, vocab, top, E, weight, (const bf16_t*)base,
                       base_stride, (bf16_t*)out, out_stride, F, W, vec2, base_scale, out_scale);
  }
  LMSF_LAUNCH_CHECK("table_moe");
  return 0;
}

extern "C" int lmsf_table_moe(const void* h, int dtype, long h_stride, const void* Wgu, const void* Wd, const int* ids,
                              const int* table, int vocab, int top, int E, float weight, const void* base,
                              long base_stride, const float* pair_scale, const float* base_scale, void* act, void* out,
                              long out_stride, int n_tokens, int F, int W, int* scratch_ints, float* scratch_rows,
                              hipStream_t stream) {
  return lmsf_table_moe_act(h, dtype, h_stride, Wgu, Wd, ids, table, vocab, top, E, weight, base, base_stride,
                            pair_scale, base_scale, nullptr, 0, act, out, out_stride, n_tokens, F, W, scratch_ints,
                            scratch_rows, stream);
}

// ---------------------------------------------------------------- a router's choice
// From float32 router logits z [n_tokens, >= E]: scores s = sigmoid(z); choice[n, 0 .. top-1] the experts with the
// largest scores (the largest first; of equal scores the lower index), weight[n, k] their scores, divided by their sum
// if ``renorm``. ``extra`` >= 0: also gate[n] = sigmoid(z[n, extra]) (a column beside the experts': the gate of a
// shared expert). A wave a token; top times a pass over the E scores.
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, long z_stride, int n_tokens, int E,
                                                        int top, int renorm, int extra, int* __restrict__ choice,
                                                        float* __restrict__ weight, float* __restrict__ gate) {
  const int n = blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  if (n >= n_tokens) return;
  const float* row = z + (long)n * z_stride;
  float last = INFINITY, total = 0.f, mine = 0.f;
  int last_e = -1, mine_e = 0;
  for (int k = 0; k < top; ++k) {
    // the largest (score, -index) below the one taken before
    float best = -INFINITY;
    int best_e = E;
    for (int e = lane; e < E; e += LMSF_WAVE) {
      const float sc = row[e];
      const bool below = sc < last || (sc == last && e > last_e);
      if (below && (sc > best || (sc == best && e < best_e))) {
        best = sc;
        best_e = e;
      }
    }
#pragma unroll
    for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, LMSF_WAVE);
      const int oe = __shfl_xor(best_e, o, LMSF_WAVE);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
    last = best;
    last_e = best_e;
    const float sg = 1.f / (1.f + expf(-best));
    total += sg;
    if (lane == k) {      // lane k keeps the k-th choice
      mine = sg;
      mine_e = min(best_e, E - 1);
    }
  }
  if (lane < top) {
    choice[(long)n * top + lane] = mine_e;
    weight[(long)n * top + lane] = renorm ? mine / total : mine;
  }
  if (extra >= 0 && lane == 0) gate[n] = 1.f / (1.f + expf(-row[extra]));
}

extern "C" int lmsf_moe_route(const float* z, long z_stride, int n_tokens, int E, int top, int renorm, int extra,
                              int* choice, float* weight, float* gate, hipStream_t stream) {
  LMSF_CHECK(z && choice && weight && (extra < 0 || gate), "moe_route: null pointer");
  LMSF_CHECK(E > 0 && top > 0 && top <= E && top <= LMSF_WAVE && z_stride >= E && extra < z_stride, "moe_route: bad sizes");
  if (n_tokens <= 0) return 0;
  hipLaunchKernelGGL(moe_route_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, stream, z, z_stride, n_tokens, E, top,
                     renorm, extra, choice, weight, gate);
  LMSF_LAUNCH_CHECK("moe_route");
  return 0;
}

// The same with the scores a softmax over all experts (``softmax`` 1; 0: sigmoid) and a limit on where the choice may
// fall: the experts form ``groups`` equal groups of neighbours, a group's score is its best expert's, and only experts
// of the ``keep`` best groups can be chosen (groups = keep = 1: no limit). weight[n, k]: the chosen experts' scores
// (over their sum with ``renorm``). A wave a token; a lane keeps the best score and the "kept" flag of the groups
// lane, lane + 64, ... (at most 256 groups).
__global__ __launch_bounds__(256) void moe_route_groups_kernel(const float* __restrict__ z, long z_stride, int n_tokens,
                                                               int E, int top, int softmax, int groups, int keep,
                                                               int renorm, int* __restrict__ choice,
                                                               float* __restrict__ weight) {
  const int n = blockIdx.x * (256 / LMSF_WAVE) + threadIdx.x / LMSF_WAVE, lane = threadIdx.x % LMSF_WAVE;
  if (n >= n_tokens) return;
  const float* row = z + (long)n * z_stride;
  float mx = -INFINITY, sum = 0.f;
  if (softmax) {
    for (int e = lane; e < E; e += LMSF_WAVE) mx = fmaxf(mx, row[e]);
    mx = wave_max(mx);
    for (int e = lane; e < E; e += LMSF_WAVE) sum += expf(row[e] - mx);
    sum = wave_sum(sum);
  }
  const int per = E / groups;
  float gbest[4];
  unsigned kept = 0;           // bit i: group lane + 64 i is kept
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int g = lane + LMSF_WAVE * i;
    gbest[i] = -INFINITY;
    if (g < groups)
      for (int e = g * per; e < (g + 1) * per; ++e) gbest[i] = fmaxf(gbest[i], row[e]);
  }
  if (keep >= groups) kept = 0xFu;
  else
    for (int k = 0; k < keep; ++k) {
      float best = -INFINITY;
      int best_g = groups;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int g = lane + LMSF_WAVE * i;
        if (g < groups && !((kept >> i) & 1u) && (gbest[i] > best || (gbest[i] == best && g < best_g))) {
          best = gbest[i];
          best_g = g;
        }
      }
#pragma unroll
      for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, LMSF_WAVE);
        const int og = __shfl_xor(best_g, o, LMSF_WAVE);
        if (ob > best || (ob == best && og < best_g)) {
          best = ob;
          best_g = og;
        }
      }
      if (best_g < groups && (best_g % LMSF_WAVE) == lane) kept |= 1u << (best_g / LMSF_WAVE);
    }
  float last = INFINITY, total = 0.f, mine = 0.f;
  int last_e = -1, mine_e = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_e = E;
    for (int e0 = 0; e0 < E; e0 += LMSF_WAVE) {      // (every lane takes part in the shuffle)
      const int e = e0 + lane;
      const int g = min(e, E - 1) / per;
      const unsigned flags = __shfl(kept, g % LMSF_WAVE, LMSF_WAVE);
      if (e >= E || !((flags >> (g / LMSF_WAVE)) & 1u)) continue;
      const float sc = row[e];
      const bool below = sc < last || (sc == last && e > last_e);
      if (below && (sc > best || (sc == best && e < best_e))) {
        best = sc;
        best_e = e;
      }
    }
#pragma unroll
    for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, LMSF_WAVE);
      const int oe = __shfl_xor(best_e, o, LMSF_WAVE);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
    last = best;
    last_e = best_e;
    const float sc = softmax ? expf(best - mx) / sum : 1.f / (1.f + expf(-best));
    total += sc;
    if (lane == k) {
      mine = sc;
      mine_e = min(best_e, E - 1);
    }
  }
  if (lane < top) {
    choice[(long)n * top + lane] = mine_e;
    weight[(long)n * top + lane] = renorm ? mine / total : mine;
  }
}

extern "C" int lmsf_moe_route_groups(const float* z, long z_stride, int n_tokens, int E, int top, int softmax,
                                     int groups, int keep, int renorm, int* choice, float* weight,
                                     hipStream_t stream) {
  LMSF_CHECK(z && choice && weight, "moe_route_groups: null pointer");
  LMSF_CHECK(E > 0 && top > 0 && top <= E && top <= LMSF_WAVE && z_stride >= E, "moe_route_groups: bad sizes");
  LMSF_CHECK(groups > 0 && groups <= 256 && E % groups == 0 && keep > 0 && keep <= groups &&
                 (long)keep * (E / groups) >= top,
             "moe_route_groups: %d of %d groups of %d experts cannot hold %d choices", keep, groups, E, top);
  if (n_tokens <= 0) return 0;
  hipLaunchKernelGGL(moe_route_groups_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, stream, z, z_stride, n_tokens, E,
                     top, softmax, groups, keep, renorm, choice, weight);
  LMSF_LAUNCH_CHECK("moe_route_groups");
  return 0;
}
