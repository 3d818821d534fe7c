// What a token brings to the stream beside its embedding row, and small elementwise kernels around it.
//
// - An embedding with a hashed pair table: x = table[id] + pairs[row], row = (previous id * mul_prev + id * mul_cur)
//   mod buckets, the last row (number ``buckets``) for a request's first token. The previous id of a segment's
//   first token is the last id of the request's step before, kept per state slot in ``prev_state`` (a second tiny
//   kernel brings it up to date, so that nothing is written that another workgroup of the first still reads).
// - Two float32 rows laid side by side as one row of the run's type (the operand of a product over both).
// - act(z) * table[id, at .. at + dim): a gate times a slice of a per-token table, act the tanh form of GELU.
// - relu(z)^2, elementwise.
// All arithmetic is float32; results are rounded once, as they are stored.
#include "common.h"

#include <math.h>

template <typename T>
__global__ __launch_bounds__(256) void hashed_pair_embedding_kernel(
    const int* __restrict__ ids, const int* __restrict__ pos, const int* __restrict__ seg_of,
    const int* __restrict__ seg_starts, const int* __restrict__ state_slots, const int* __restrict__ prev_state,
    const T* __restrict__ table, const T* __restrict__ pairs, float* __restrict__ out, float* __restrict__ keep,
    int V, int W, int buckets, long mul_prev, long mul_cur) {
  const int t = blockIdx.x;
  const int id = min(max(ids[t], 0), V - 1);
  const int s = seg_of[t];
  int row = buckets;
  if (pos[t] > 0) {
    const int prev = (t == seg_starts[s]) ? prev_state[state_slots[s]] : ids[t - 1];
    const long hsh = ((long)min(max(prev, 0), V - 1) * mul_prev + (long)id * mul_cur) % (long)buckets;
    row = (int)(hsh < 0 ? hsh + buckets : hsh);
  }
  const T* a = table + (long)id * W;
  const T* b = pairs + (long)row * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float x = to_f32<T>(a[i]) + to_f32<T>(b[i]);
    out[(long)t * W + i] = x;
    if (keep) keep[(long)t * W + i] = x;
  }
}

__global__ void last_token_kernel(const int* __restrict__ ids, const int* __restrict__ seg_starts,
                                  const int* __restrict__ state_slots, int* __restrict__ prev_state, int S) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S) return;
  const int end = seg_starts[s + 1];
  if (end > seg_starts[s]) prev_state[state_slots[s]] = ids[end - 1];
}

// out, keep: float32 [n_tokens, W] (keep may be null: a second copy of the result, for a part that needs the
// embedding's output after the stream has moved on). table [V, W], pairs [buckets + 1, W] of ``dtype``.
// prev_state: int32, one entry per state slot (and the spare one).
extern "C" int lmsf_hashed_pair_embedding(const int* ids, const int* pos, const int* seg_of, const int* seg_starts,
                                          const int* state_slots, int* prev_state, const void* table,
                                          const void* pairs, int dtype, float* out, float* keep, int n_tokens,
                                          int n_segments, int V, int W, int buckets, long mul_prev, long mul_cur,
                                          hipStream_t stream) {
  LMSF_CHECK(ids && pos && seg_of && seg_starts && state_slots && prev_state && table && pairs && out,
             "hashed_pair_embedding: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "hashed_pair_embedding: unknown dtype code %d", dtype);
  LMSF_CHECK(V > 0 && W > 0 && buckets > 0 && n_segments >= 0, "hashed_pair_embedding: bad sizes");
  if (n_tokens <= 0) return 0;
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((hashed_pair_embedding_kernel<float>), dim3(n_tokens), dim3(256), 0, stream, ids, pos, seg_of,
                       seg_starts, state_slots, prev_state, (const float*)table, (const float*)pairs, out, keep, V, W,
                       buckets, mul_prev, mul_cur);
  else
    hipLaunchKernelGGL((hashed_pair_embedding_kernel<bf16_t>), dim3(n_tokens), dim3(256), 0, stream, ids, pos, seg_of,
                       seg_starts, state_slots, prev_state, (const bf16_t*)table, (const bf16_t*)pairs, out, keep, V,
                       W, buckets, mul_prev, mul_cur);
  hipLaunchKernelGGL(last_token_kernel, dim3((n_segments + 63) / 64), dim3(64), 0, stream, ids, seg_starts,
                     state_slots, prev_state, n_segments);
  LMSF_LAUNCH_CHECK("hashed_pair_embedding");
  return 0;
}

// ---------------------------------------------------------------- two rows side by side

template <typename T>
__global__ __launch_bounds__(256) void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          T* __restrict__ out, int Wa, int Wb) {
  const long n = blockIdx.x;
  for (int i = threadIdx.x; i < Wa + Wb; i += 256)
    out[n * (Wa + Wb) + i] = from_f32<T>(i < Wa ? a[n * Wa + i] : b[n * Wb + i - Wa]);
}

// out [n, Wa + Wb] of ``dtype`` = [a | b], a float32 [n, Wa], b float32 [n, Wb], all contiguous.
extern "C" int lmsf_concat_rows(const float* a, const float* b, void* out, int dtype, int n, int Wa, int Wb,
                                hipStream_t stream) {
  LMSF_CHECK(a && b && out && Wa > 0 && Wb > 0, "concat_rows: bad arguments");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "concat_rows: unknown dtype code %d", dtype);
  if (n <= 0) return 0;
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((concat_rows_kernel<float>), dim3(n), dim3(256), 0, stream, a, b, (float*)out, Wa, Wb);
  else
    hipLaunchKernelGGL((concat_rows_kernel<bf16_t>), dim3(n), dim3(256), 0, stream, a, b, (bf16_t*)out, Wa, Wb);
  LMSF_LAUNCH_CHECK("concat_rows");
  return 0;
}

// ---------------------------------------------------------------- a gate times a slice of a per-token table

template <typename T>
__global__ __launch_bounds__(256) void gate_table_kernel(const T* __restrict__ z, long z_stride,
                                                         const int* __restrict__ ids, const T* __restrict__ table,
                                                         long table_stride, int at, int V, T* __restrict__ out,
                                                         int n, int dim) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)n * dim) return;
  const int t = (int)(i / dim), j = (int)(i - (long)t * dim);
  const int id = min(max(ids[t], 0), V - 1);
  const float g = gated_product_activation<5>(to_f32<T>(z[(long)t * z_stride + j]));
  out[i] = from_f32<T>(g * to_f32<T>(table[(long)id * table_stride + at + j]));
}

// out [n, dim] (contiguous) = gelu_tanh(z [n, dim]) * table[ids[n], at .. at + dim)
extern "C" int lmsf_gate_table(const void* z, long z_stride, const int* ids, const void* table, long table_stride,
                               int at, int V, void* out, int dtype, int n, int dim, hipStream_t stream) {
  LMSF_CHECK(z && ids && table && out, "gate_table: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "gate_table: unknown dtype code %d", dtype);
  LMSF_CHECK(dim > 0 && at >= 0 && at + dim <= table_stride && z_stride >= dim && V > 0, "gate_table: bad sizes");
  if (n <= 0) return 0;
  const dim3 grid((unsigned)(((long)n * dim + 255) / 256));
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((gate_table_kernel<float>), grid, dim3(256), 0, stream, (const float*)z, z_stride, ids,
                       (const float*)table, table_stride, at, V, (float*)out, n, dim);
  else
    hipLaunchKernelGGL((gate_table_kernel<bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)z, z_stride, ids,
                       (const bf16_t*)table, table_stride, at, V, (bf16_t*)out, n, dim);
  LMSF_LAUNCH_CHECK("gate_table");
  return 0;
}

// ---------------------------------------------------------------- relu(z)^2

template <typename T>
__global__ __launch_bounds__(256) void relu_squared_kernel(const T* __restrict__ z, long z_stride,
                                                           T* __restrict__ out, int n, int F) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)n * F) return;
  const int t = (int)(i / F), j = (int)(i - (long)t * F);
  const float v = fmaxf(to_f32<T>(z[(long)t * z_stride + j]), 0.f);
  out[i] = from_f32<T>(v * v);
}

extern "C" int lmsf_relu_squared(const void* z, long z_stride, void* out, int dtype, int n, int F,
                                 hipStream_t stream) {
  LMSF_CHECK(z && out && F > 0 && z_stride >= F, "relu_squared: bad arguments");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "relu_squared: unknown dtype code %d", dtype);
  if (n <= 0) return 0;
  const dim3 grid((unsigned)(((long)n * F + 255) / 256));
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((relu_squared_kernel<float>), grid, dim3(256), 0, stream, (const float*)z, z_stride,
                       (float*)out, n, F);
  else
    hipLaunchKernelGGL((relu_squared_kernel<bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)z, z_stride,
                       (bf16_t*)out, n, F);
  LMSF_LAUNCH_CHECK("relu_squared");
  return 0;
}
