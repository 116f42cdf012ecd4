// A feed-forward made of many small gated feed-forwards of which every token uses a few.
//   nhv_route_topk        float router logits of a row, a score per expert (sigmoid), the ``top`` largest: their numbers
//                         and scores
//   nhv_experts_gate_up   for every (token, chosen expert): act(s G_e h) * (s U_e h), s the score: the expert's input is
//                         s h, and a product is linear in its rows, so the score multiplies the finished float sums
//   nhv_experts_down      out[t] = sum over the token's experts of D_e u[t, j]
// One wave per output: a sum runs over its inner index in an order that depends on the sizes only, so a row's result
// does not depend on its batch. Weights of all experts lie in one tensor, [experts, 2 ff, width] (gate rows, then up
// rows) and [experts, width, ff].
#include "nhv_common.h"
#include <math.h>

template <typename T>
__global__ __launch_bounds__(256) void route_topk_kernel(const T* __restrict__ h, const float* __restrict__ router,
                                                         int* __restrict__ ids, float* __restrict__ scores, int W, int E,
                                                         int top) {
  extern __shared__ float z[];               // E logits
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* x = h + (size_t)t * W;
  for (int e = wave; e < E; e += 4) {
    const float* w = router + (size_t)e * W;
    float s = 0.f;
    for (int k = lane; k < W; k += NHV_WAVE) s = fmaf(w[k], to_f32(x[k]), s);
    s = wave_sum(s);
    if (lane == 0) z[e] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  // the largest first; among equal logits the lower number. A chosen expert's logit becomes -inf.
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += NHV_WAVE) {
      const float v = z[e];
      if (v > best) { best = v; at = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, NHV_WAVE);
      const int oa = __shfl_xor(at, o, NHV_WAVE);
      if (ov > best || (ov == best && oa < at)) { best = ov; at = oa; }
    }
    if (lane == 0) {
      ids[(size_t)t * top + j] = at;
      scores[(size_t)t * top + j] = 1.0f / (1.0f + expf(-best));
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
}

extern "C" int nhv_route_topk(const void* h, const void* router, void* ids, void* scores, int T, int W, int E, int top,
                              int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && E > 0 && top > 0 && top <= E && E <= 8192, "route_topk: bad sizes T=%d W=%d E=%d top=%d", T, W, E, top);
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)E * sizeof(float);
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(route_topk_kernel<float>, dim3(T), dim3(256), lds, s, (const float*)h, (const float*)router,
                       (int*)ids, (float*)scores, W, E, top);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(route_topk_kernel<bf16_t>, dim3(T), dim3(256), lds, s, (const bf16_t*)h, (const float*)router,
                       (int*)ids, (float*)scores, W, E, top);
  else
    return nhv_fail("route_topk: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("route_topk");
  return 0;
}

__device__ __forceinline__ float nhv_expert_act(float z, int act) {
  if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z / (1.0f + expf(-z));
}

// u[t * top + j, f] for the pair (t, j): one wave per f.
template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ h, const int* __restrict__ ids,
                                                              const float* __restrict__ scores,
                                                              const T* __restrict__ gate_up, T* __restrict__ u, int W,
                                                              int F, int top, int E, int act) {
  const int pair = blockIdx.x;
  const int f = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (f >= F) return;
  const int e = ids[pair];
  if (e < 0 || e >= E) return;
  const T* x = h + (size_t)(pair / top) * W;
  const T* g = gate_up + ((size_t)e * 2 * F + f) * W;
  const T* p = g + (size_t)F * W;
  float sg = 0.f, su = 0.f;
  for (int k = lane; k < W; k += NHV_WAVE) {
    const float xv = to_f32(x[k]);
    sg = fmaf(to_f32(g[k]), xv, sg);
    su = fmaf(to_f32(p[k]), xv, su);
  }
  sg = wave_sum(sg);
  su = wave_sum(su);
  if (lane == 0) {
    const float s = scores[pair];
    u[(size_t)pair * F + f] = from_f32<T>(nhv_expert_act(s * sg, act) * (s * su));
  }
}

extern "C" int nhv_experts_gate_up(const void* h, const void* ids, const void* scores, const void* gate_up, void* u,
                                   int T, int W, int F, int top, int E, int act, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && F > 0 && top > 0 && E > 0, "experts_gate_up: bad sizes T=%d W=%d F=%d top=%d E=%d", T, W, F, top, E);
  NHV_REQUIRE((long long)T * top < (1ll << 31) && (F + 3) / 4 <= 65535, "experts_gate_up: T=%d top=%d F=%d are beyond this kernel's grid", T, top, F);
  const dim3 grid(T * top, (F + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(experts_gate_up_kernel<float>, grid, dim3(256), 0, s, (const float*)h, (const int*)ids,
                       (const float*)scores, (const float*)gate_up, (float*)u, W, F, top, E, act);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(experts_gate_up_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)h, (const int*)ids,
                       (const float*)scores, (const bf16_t*)gate_up, (bf16_t*)u, W, F, top, E, act);
  else
    return nhv_fail("experts_gate_up: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("experts_gate_up");
  return 0;
}

// out[t, n] = sum over j < top (rising), each a sum over f: one wave per n.
template <typename T>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ u, const int* __restrict__ ids,
                                                           const T* __restrict__ down, T* __restrict__ out, int W, int F,
                                                           int top, int E) {
  const int t = blockIdx.x;
  const int n = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (n >= W) return;
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[(size_t)t * top + j];
    if (e < 0 || e >= E) continue;
    const T* d = down + ((size_t)e * W + n) * F;
    const T* x = u + ((size_t)t * top + j) * F;
    float s = 0.f;
    for (int f = lane; f < F; f += NHV_WAVE) s = fmaf(to_f32(d[f]), to_f32(x[f]), s);
    total += wave_sum(s);
  }
  if (lane == 0) out[(size_t)t * W + n] = from_f32<T>(total);
}

extern "C" int nhv_experts_down(const void* u, const void* ids, const void* down, void* out, int T, int W, int F, int top,
                                int E, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && W > 0 && F > 0 && top > 0 && E > 0, "experts_down: bad sizes T=%d W=%d F=%d top=%d E=%d", T, W, F, top, E);
  NHV_REQUIRE((W + 3) / 4 <= 65535, "experts_down: width %d is beyond this kernel's grid", W);
  const dim3 grid(T, (W + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(experts_down_kernel<float>, grid, dim3(256), 0, s, (const float*)u, (const int*)ids,
                       (const float*)down, (float*)out, W, F, top, E);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(experts_down_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)u, (const int*)ids,
                       (const bf16_t*)down, (bf16_t*)out, W, F, top, E);
  else
    return nhv_fail("experts_down: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("experts_down");
  return 0;
}
