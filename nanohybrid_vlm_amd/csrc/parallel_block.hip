// Kernels of layers whose mixer and feed-forward read two norms of the same stream, and of an embedding that adds a
// row chosen by a hash of (previous token, token):
//   nhv_embed_pair_hash   rows of two tables added in float; the previous token of a request is kept per state slot
//   nhv_layernorm_pair    x (+ a + b) -> one or two layer norms (weight and bias) of it; x is the float stream
//   nhv_add_streams       x += a (+ b)
// Rows are float or bfloat16; the stream, statistics and sums are float.
#include "nhv_common.h"
#include <math.h>

// ---------------------------------------------------------------- embedding with a hashed pair row
// out[t] = table[id_t] + pair_table[row_t], row_t = (prev_t * mul_prev + id_t * mul_cur) mod buckets, and row
// ``buckets`` (the last) for the token at position 0. prev_t is the token before t: the one before it in this step, or
// for the first token of a request's portion what ``prev_state`` holds at the request's slot. The block of a request's
// first token of the step then writes the request's last token of the step there (the same thread reads, then writes).
template <typename T>
__global__ void embed_pair_hash_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                       const T* __restrict__ pair_table, float* __restrict__ out,
                                       const int* __restrict__ positions, const int* __restrict__ cu_seqlens,
                                       const int* __restrict__ token_req, const int* __restrict__ state_slots,
                                       int* __restrict__ prev_state, int W, int V, int buckets, int mul_prev, int mul_cur) {
  const int t = blockIdx.x;
  __shared__ int row_s;
  if (threadIdx.x == 0) {
    const int req = token_req[t];
    const int first = cu_seqlens[req];
    const int pos = positions[t];
    int prev = -1;
    if (t > first) prev = ids[t - 1];
    else prev = prev_state[state_slots[req]];
    if (t == first) prev_state[state_slots[req]] = ids[cu_seqlens[req + 1] - 1];
    int row = buckets;
    if (pos > 0 && prev >= 0) {
      const long long hsh = (long long)prev * mul_prev + (long long)ids[t] * mul_cur;
      row = (int)(((hsh % buckets) + buckets) % buckets);
    }
    row_s = row;
  }
  __syncthreads();
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;      // the host checks ids; an id out of range gives the pair row alone
  const T* a = table + (size_t)(ok ? id : 0) * W;
  const T* b = pair_table + (size_t)row_s * W;
  float* dst = out + (size_t)t * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) dst[i] = (ok ? to_f32(a[i]) : 0.f) + to_f32(b[i]);
}

extern "C" int nhv_embed_pair_hash(const void* ids, const void* table, const void* pair_table, void* out,
                                   const void* positions, const void* cu_seqlens, const void* token_req,
                                   const void* state_slots, void* prev_state, int T, int W, int V, int buckets,
                                   int mul_prev, int mul_cur, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && V > 0 && buckets > 0, "embed_pair_hash: bad sizes T=%d W=%d V=%d buckets=%d", T, W, V, buckets);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(embed_pair_hash_kernel<float>, dim3(T), dim3(256), 0, s, (const int*)ids, (const float*)table,
                       (const float*)pair_table, (float*)out, (const int*)positions, (const int*)cu_seqlens,
                       (const int*)token_req, (const int*)state_slots, (int*)prev_state, W, V, buckets, mul_prev, mul_cur);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(embed_pair_hash_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const int*)ids, (const bf16_t*)table,
                       (const bf16_t*)pair_table, (float*)out, (const int*)positions, (const int*)cu_seqlens,
                       (const int*)token_req, (const int*)state_slots, (int*)prev_state, W, V, buckets, mul_prev, mul_cur);
  else
    return nhv_fail("embed_pair_hash: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("embed_pair_hash");
  return 0;
}

// ---------------------------------------------------------------- two layer norms of one stream
// s = x (+ a) (+ b), written back to x where something was added; mean and variance (mean of squared deviations) of s
// once; y1 = (s - mean) r w1 + b1, y2 = (s - mean) r w2 + b2, r = 1 / sqrt(variance + eps). y2 may be absent.
template <typename T>
__global__ void layernorm_pair_kernel(float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
                                      const float* __restrict__ w1, const float* __restrict__ b1, T* __restrict__ y1,
                                      const float* __restrict__ w2, const float* __restrict__ b2, T* __restrict__ y2,
                                      int W, float eps) {
  extern __shared__ float row[];          // W floats + 16
  float* scratch = row + W;
  const size_t base = (size_t)blockIdx.x * W;
  float sum = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = x[base + i];
    if (a != nullptr) v += to_f32(a[base + i]);
    if (b != nullptr) v += to_f32(b[base + i]);
    if (a != nullptr || b != nullptr) x[base + i] = v;
    row[i] = v;
    sum += v;
  }
  const float mean = block_sum(sum, scratch) / (float)W;
  float sq = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float d = row[i] - mean;
    sq += d * d;
  }
  const float r = 1.0f / sqrtf(block_sum(sq, scratch) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float n = (row[i] - mean) * r;
    if (y1 != nullptr) y1[base + i] = from_f32<T>(n * w1[i] + b1[i]);
    if (y2 != nullptr) y2[base + i] = from_f32<T>(n * w2[i] + b2[i]);
  }
}

extern "C" int nhv_layernorm_pair(void* x, const void* a, const void* b, const void* w1, const void* b1, void* y1,
                                  const void* w2, const void* b2, void* y2, int T, int W, float eps, int dtype,
                                  void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && W <= 16368, "layernorm_pair: bad sizes T=%d W=%d (widths up to 16368)", T, W);
  NHV_REQUIRE(y1 != nullptr || y2 != nullptr || a != nullptr || b != nullptr, "layernorm_pair: nothing to do");
  const size_t lds = ((size_t)W + 16) * sizeof(float);
  const int threads = W >= 2048 ? 512 : 256;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(layernorm_pair_kernel<float>, dim3(T), dim3(threads), lds, s, (float*)x, (const float*)a,
                       (const float*)b, (const float*)w1, (const float*)b1, (float*)y1, (const float*)w2, (const float*)b2,
                       (float*)y2, W, eps);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(layernorm_pair_kernel<bf16_t>, dim3(T), dim3(threads), lds, s, (float*)x, (const bf16_t*)a,
                       (const bf16_t*)b, (const float*)w1, (const float*)b1, (bf16_t*)y1, (const float*)w2,
                       (const float*)b2, (bf16_t*)y2, W, eps);
  else
    return nhv_fail("layernorm_pair: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("layernorm_pair");
  return 0;
}

// ---------------------------------------------------------------- x += a (+ b)
template <typename T>
__global__ void add_streams_kernel(float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float v = x[i] + to_f32(a[i]);
    if (b != nullptr) v += to_f32(b[i]);
    x[i] = v;
  }
}

extern "C" int nhv_add_streams(void* x, const void* a, const void* b, size_t n, int dtype, void* stream) {
  NHV_REQUIRE(n > 0 && a != nullptr, "add_streams: nothing to add");
  const int blocks = (int)((n + 255) / 256 > 65535 * 4 ? 65535 * 4 : (n + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(add_streams_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)x, (const float*)a, (const float*)b, n);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(add_streams_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (float*)x, (const bf16_t*)a, (const bf16_t*)b, n);
  else
    return nhv_fail("add_streams: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("add_streams");
  return 0;
}
