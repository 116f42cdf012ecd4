// The gated delta rule: a recurrent mixer whose state is one matrix S[D, E] per head and request,
//   S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t,
// with a decay g_t per key channel, preceded by short causal convolutions over time on q, k and v.
// Four kernels, the same for prompt portions and for single decoded tokens:
//  - nhv_delta_prepare: per token, the convolutions (earlier inputs come from the step's own rows or from the
//    request's kept inputs), SiLU, unit length per head for q and k, the decays from their linear part, beta;
//  - nhv_conv_state_update: per request, the last taps - 1 inputs are kept for the next step;
//  - nhv_delta_rule: per (request, head, tile of value columns), the recurrence over the step's tokens in order,
//    from the request's state (zero for a request that starts at position 0) and back into it;
//  - nhv_gated_head_norm: per (token, head), o over its root mean square, times a weight, times sigmoid(gate).
// Everything here is float: the state, the decays, the unit vectors, the sums. A column of S (one value channel)
// never meets another column, so a block owns a tile of columns, a column belongs to R adjacent lanes that hold D / R
// entries each, and the two sums over D per token are taken with lane shuffles; the next token's vectors are asked
// for before this token's are used. A request without tokens in the step is left alone.
#include "nhv_common.h"
#include <math.h>

#define NHV_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------- per token: what enters the recurrence
// proj[T, ld]: q (G D) | k (G D) | v (H E) | beta (H) as the projection left them. taps[C, n], C = 2 G D + H E, last
// column for the token itself. kept[slots, C, n - 1]: the inputs at the n - 1 positions before the request's first
// token of this step. a_lin[T, H D]: the decays' linear part on entry, the decays on return.
template <typename TI>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const TI* __restrict__ proj, int ld, const float* __restrict__ taps, int n_taps, const float* __restrict__ kept,
    float* __restrict__ a_lin, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ token_req, const int* __restrict__ positions, const int* __restrict__ cu,
    const int* __restrict__ state_slots, float* __restrict__ q_out, float* __restrict__ k_out, float* __restrict__ v_out,
    float* __restrict__ beta_out, int H, int G, int D, int E) {
  extern __shared__ float conv[];            // C floats
  const int t = blockIdx.x;
  const int req = token_req[t];
  const int first = cu[req];
  const int i_in_step = t - first;           // tokens of this request before this one in the step
  const int pos = positions[t];
  const int C = 2 * G * D + H * E;
  const float* mine = kept + (size_t)state_slots[req] * C * (n_taps - 1);
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float sum = 0.f;
    for (int j = 0; j < n_taps; ++j) {       // the input j positions back meets the tap n - 1 - j
      if (pos - j < 0) break;
      float x;
      if (j <= i_in_step) x = to_f32(proj[(size_t)(t - j) * ld + c]);
      else x = mine[(size_t)c * (n_taps - 1) + (n_taps - 1) + i_in_step - j];
      sum = fmaf(taps[(size_t)c * n_taps + n_taps - 1 - j], x, sum);
    }
    conv[c] = silu_f(sum);
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
  // q and k heads: unit length (the sum of squares plus 1e-6 under the root); q also times D^(-1/2)
  const float q_scale = 1.0f / sqrtf((float)D);
  for (int head = wave; head < 2 * G; head += n_waves) {
    const float* src = conv + head * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += NHV_WAVE) ss = fmaf(src[d], src[d], ss);
    ss = wave_sum(ss);
    const float r = (head < G ? q_scale : 1.0f) / sqrtf(ss + 1e-6f);
    float* dst = head < G ? q_out + ((size_t)t * G + head) * D : k_out + ((size_t)t * G + head - G) * D;
    for (int d = lane; d < D; d += NHV_WAVE) dst[d] = src[d] * r;
  }
  for (int c = threadIdx.x; c < H * E; c += blockDim.x) v_out[(size_t)t * H * E + c] = conv[2 * G * D + c];
  for (int c = threadIdx.x; c < H * D; c += blockDim.x) {
    const float step = softplus_f(a_lin[(size_t)t * H * D + c] + dt_bias[c]);
    a_lin[(size_t)t * H * D + c] = expf(-expf(a_log[c / D]) * step);
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x)
    beta_out[(size_t)t * H + h] = sigmoid_f(to_f32(proj[(size_t)t * ld + C + h]));
}

extern "C" int nhv_delta_prepare(const void* proj, int proj_dtype, const void* taps, int n_taps, const void* kept,
                                 void* a_lin, const void* dt_bias, const void* a_log, const void* token_req,
                                 const void* positions, const void* cu, const void* state_slots, void* q_out, void* k_out,
                                 void* v_out, void* beta_out, int T, int H, int G, int D, int E, void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && G > 0 && D > 0 && E > 0 && H % G == 0, "delta_prepare: bad sizes T=%d H=%d G=%d D=%d E=%d", T, H, G, D, E);
  NHV_REQUIRE(n_taps >= 1 && n_taps <= NHV_MAX_TAPS, "delta_prepare: %d taps (1 to %d are taken)", n_taps, NHV_MAX_TAPS);
  const int C = 2 * G * D + H * E;
  const size_t lds = (size_t)C * sizeof(float);
  NHV_REQUIRE(lds <= 160 * 1024, "delta_prepare: %d channels do not fit a block's scratch memory", C);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TI)                                                                                                    \
  do {                                                                                                                \
    if (lds > 64 * 1024)                                                                                              \
      (void)hipFuncSetAttribute((const void*)delta_prepare_kernel<TI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
    hipLaunchKernelGGL(delta_prepare_kernel<TI>, dim3(T), dim3(256), lds, s, (const TI*)proj, C + H, (const float*)taps, \
                       n_taps, (const float*)kept, (float*)a_lin, (const float*)dt_bias, (const float*)a_log,         \
                       (const int*)token_req, (const int*)positions, (const int*)cu, (const int*)state_slots,         \
                       (float*)q_out, (float*)k_out, (float*)v_out, (float*)beta_out, H, G, D, E);                    \
  } while (0)
  if (proj_dtype == NHV_F32) LAUNCH(float);
  else if (proj_dtype == NHV_BF16) LAUNCH(bf16_t);
  else return nhv_fail("delta_prepare: unknown dtype %d", proj_dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("delta_prepare");
  return 0;
}

// ---------------------------------------------------------------- per request: the inputs kept for the next step
// After a step that brought a request n tokens from position ``start`` on, kept[., c, s] is the input at position
// start + n - (taps - 1) + s: one of the step's rows, or what was kept before (nothing, i.e. zero, before position 0).
// A thread owns one channel of one request, reads all it needs and then writes.
template <typename TI>
__global__ void conv_state_update_kernel(const TI* __restrict__ proj, int ld, float* __restrict__ kept, int n_taps,
                                         const int* __restrict__ positions, const int* __restrict__ cu,
                                         const int* __restrict__ state_slots, int C) {
  const int req = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int first = cu[req], n = cu[req + 1] - first;
  if (n <= 0 || c >= C) return;
  const int start = positions[first];
  float* mine = kept + ((size_t)state_slots[req] * C + c) * (n_taps - 1);
  float next[NHV_MAX_TAPS];
  for (int s = 0; s < n_taps - 1; ++s) {
    const int rel = n - (n_taps - 1) + s;     // which of the step's tokens, if not negative
    if (rel >= 0) next[s] = to_f32(proj[(size_t)(first + rel) * ld + c]);
    else next[s] = start + rel >= 0 ? mine[n + s] : 0.f;
  }
  for (int s = 0; s < n_taps - 1; ++s) mine[s] = next[s];
}

extern "C" int nhv_conv_state_update(const void* proj, int proj_dtype, int ld, void* kept, int n_taps, const void* positions,
                                     const void* cu, const void* state_slots, int B, int C, void* stream) {
  NHV_REQUIRE(B > 0 && C > 0 && ld >= C && B <= 65535, "conv_state_update: bad sizes B=%d C=%d ld=%d", B, C, ld);
  NHV_REQUIRE(n_taps >= 1 && n_taps <= NHV_MAX_TAPS, "conv_state_update: %d taps (1 to %d are taken)", n_taps, NHV_MAX_TAPS);
  if (n_taps == 1) return 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((C + 255) / 256, B);
  if (proj_dtype == NHV_F32)
    hipLaunchKernelGGL(conv_state_update_kernel<float>, grid, dim3(256), 0, s, (const float*)proj, ld, (float*)kept, n_taps,
                       (const int*)positions, (const int*)cu, (const int*)state_slots, C);
  else if (proj_dtype == NHV_BF16)
    hipLaunchKernelGGL(conv_state_update_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)proj, ld, (float*)kept, n_taps,
                       (const int*)positions, (const int*)cu, (const int*)state_slots, C);
  else return nhv_fail("conv_state_update: unknown dtype %d", proj_dtype);
  NHV_LAUNCH_CHECK("conv_state_update");
  return 0;
}

// ---------------------------------------------------------------- the recurrence
// state[slots, H, E, D]: a column of S lies contiguous. Thread (column e, part r) of a block holds S[r DR .. r DR + DR, e];
// the R parts of a column are adjacent lanes (R a power of two, at most 64). Entries beyond D (where D is no multiple
// of R DR) are zeros that change nothing.
template <int DR>
__global__ __launch_bounds__(256) void delta_rule_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ decay,
    const float* __restrict__ beta, float* __restrict__ state, float* __restrict__ out, const int* __restrict__ positions,
    const int* __restrict__ cu, const int* __restrict__ state_slots, int H, int G, int D, int E, int R, int cols) {
  const int req = blockIdx.z, h = blockIdx.y;
  const int first = cu[req], end = cu[req + 1];
  if (end <= first) return;                  // (the same for the whole block)
  const int e = blockIdx.x * cols + threadIdx.x / R;
  const int r = threadIdx.x % R;
  const int d0 = r * DR;
  const bool column = e < E;
  const int g = h / (H / G);
  float S[DR];
  float* mine = state + (((size_t)state_slots[req] * H + h) * E + (column ? e : 0)) * D;
  const bool fresh = positions[first] == 0;
#pragma unroll
  for (int i = 0; i < DR; ++i) S[i] = (!fresh && column && d0 + i < D) ? mine[d0 + i] : 0.f;

  float nq[DR], nk[DR], ng[DR], nv, nb;
  auto fetch = [&](int t) {
    const float* qr = q + ((size_t)t * G + g) * D;
    const float* kr = k + ((size_t)t * G + g) * D;
    const float* gr = decay + ((size_t)t * H + h) * D;
#pragma unroll
    for (int i = 0; i < DR; ++i) {
      const bool ok = d0 + i < D;
      nq[i] = ok ? qr[d0 + i] : 0.f;
      nk[i] = ok ? kr[d0 + i] : 0.f;
      ng[i] = ok ? gr[d0 + i] : 0.f;
    }
    nv = column ? v[((size_t)t * H + h) * E + e] : 0.f;
    nb = beta[(size_t)t * H + h];
  };
  fetch(first);
  for (int t = first; t < end; ++t) {
    float cq[DR], ck[DR];
    const float cv = nv, cb = nb;
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < DR; ++i) {
      cq[i] = nq[i];
      ck[i] = nk[i];
      S[i] *= ng[i];
      dot = fmaf(ck[i], S[i], dot);
    }
    if (t + 1 < end) fetch(t + 1);
    for (int o = 1; o < R; o <<= 1) dot += __shfl_xor(dot, o, NHV_WAVE);
    const float u = cb * (cv - dot);
    float read = 0.f;
#pragma unroll
    for (int i = 0; i < DR; ++i) {
      S[i] = fmaf(ck[i], u, S[i]);
      read = fmaf(cq[i], S[i], read);
    }
    for (int o = 1; o < R; o <<= 1) read += __shfl_xor(read, o, NHV_WAVE);
    if (r == 0 && column) out[((size_t)t * H + h) * E + e] = read;
  }
  if (column) {
#pragma unroll
    for (int i = 0; i < DR; ++i)
      if (d0 + i < D) mine[d0 + i] = S[i];
  }
}

extern "C" int nhv_delta_rule(const void* q, const void* k, const void* v, const void* decay, const void* beta, void* state,
                              void* out, const void* positions, const void* cu, const void* state_slots, int B, int H, int G,
                              int D, int E, void* stream) {
  NHV_REQUIRE(B > 0 && H > 0 && G > 0 && D > 0 && E > 0 && H % G == 0, "delta_rule: bad sizes B=%d H=%d G=%d D=%d E=%d", B, H, G, D, E);
  NHV_REQUIRE(D <= 1024 && B <= 65535 && H <= 65535, "delta_rule: D=%d (up to 1024), B=%d, H=%d (up to 65535)", D, B, H);
  // entries a lane: 8 from a key size of 64 on, 4 below, 16 where 8 would need more than 64 lanes a column
  const int dr = D > 512 ? 16 : (D >= 64 ? 8 : 4);
  int R = 1;
  while (R * dr < D) R <<= 1;
  int cols = 256 / R;
  if (cols < 1) cols = 1;
  if (cols > E) cols = E;
  const dim3 grid((E + cols - 1) / cols, H, B), block(cols * R);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(DRV)                                                                                                   \
  hipLaunchKernelGGL(delta_rule_kernel<DRV>, grid, block, 0, s, (const float*)q, (const float*)k, (const float*)v,    \
                     (const float*)decay, (const float*)beta, (float*)state, (float*)out, (const int*)positions,      \
                     (const int*)cu, (const int*)state_slots, H, G, D, E, R, cols)
  if (dr == 16) LAUNCH(16);
  else if (dr == 8) LAUNCH(8);
  else LAUNCH(4);
#undef LAUNCH
  NHV_LAUNCH_CHECK("delta_rule");
  return 0;
}

// ---------------------------------------------------------------- the read-out's norm and gate
// y[t, h, e] = o[t, h, e] / sqrt(mean over e of o^2 + eps) * w[e] * sigmoid(gate[t, h, e]); one wave per (t, h).
template <typename TO>
__global__ void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ gate, const float* __restrict__ w,
                                       TO* __restrict__ y, int E, float eps, int n_items) {
  const int item = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= n_items) return;
  const int lane = threadIdx.x & 63;
  const float* src = o + (size_t)item * E;
  float ss = 0.f;
  for (int e = lane; e < E; e += NHV_WAVE) ss = fmaf(src[e], src[e], ss);
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)E + eps);
  for (int e = lane; e < E; e += NHV_WAVE)
    y[(size_t)item * E + e] = from_f32<TO>(src[e] * r * w[e] * sigmoid_f(gate[(size_t)item * E + e]));
}

extern "C" int nhv_gated_head_norm(const void* o, const void* gate, const void* w, void* y, int T, int H, int E, float eps,
                                   int y_dtype, void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && E > 0 && (long long)T * H < (1ll << 31), "gated_head_norm: bad sizes T=%d H=%d E=%d", T, H, E);
  const int n_items = T * H;
  const unsigned blocks = (unsigned)((n_items + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (y_dtype == NHV_F32)
    hipLaunchKernelGGL(gated_head_norm_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)o, (const float*)gate,
                       (const float*)w, (float*)y, E, eps, n_items);
  else if (y_dtype == NHV_BF16)
    hipLaunchKernelGGL(gated_head_norm_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const float*)o, (const float*)gate,
                       (const float*)w, (bf16_t*)y, E, eps, n_items);
  else return nhv_fail("gated_head_norm: unknown dtype %d", y_dtype);
  NHV_LAUNCH_CHECK("gated_head_norm");
  return 0;
}
