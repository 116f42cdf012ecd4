// Kernels of attention over a cached latent: every token stores one row [c | r], c the normed low-rank latent that
// keys and values of all heads are made of, r a rotated key part shared by all heads (it may be absent).
//   nhv_latent_prepare      the packed down projections of a step's rows -> the normed query latent, and the row
//                           [RMS-normed c | rotated r] stored at the step's slots
//   nhv_head_gemm           y[t, h, :] = M_h x[t, h, :] for a matrix per head (strides say which way M_h lies), with an
//                           optional sigmoid gate per (token, head) on the result
//   nhv_head_gemm_fewrows   the same for up to 16 rows, with the turning of the queries' rotated part in the same launch
//   nhv_rotate_interleaved  the rotated part of every query head, turned by position and copied beside the rest
// Pairs (2i, 2i + 1) turn by angle = position * freqs[i]; cosine and sine are multiplied by ``gain``. The frequencies
// come as doubles and the product with the position is taken and brought into [-pi, pi] in double (a float product
// of a position in the thousands is off by 1e-4 of a turn), then sine and cosine in float. Norm statistics and sums
// are float; rows are float or bfloat16.
#include "nhv_common.h"
#include <math.h>

__device__ __forceinline__ void nhv_turn_angle(int pos, double f, float gain, float* sn, float* cs) {
  const double a = (double)pos * f;
  const double turns = rint(a * 0.15915494309189535);
  sincosf((float)(a - turns * 6.283185307179586), sn, cs);
  *sn *= gain;
  *cs *= gain;
}

// a: [T, A] float. Query latent: columns q_off .. q_off + q_rank, normed with wq into cq [T, q_rank]. Latent:
// columns c_off .. c_off + kv_rank normed with wc, then ``rot`` columns turned; both stored at slot_mapping[t] in
// ``cache`` (rows of ``row`` entries; entries beyond kv_rank + rot are left alone). kv_rank 0: nothing is stored.
template <typename T>
__global__ void latent_prepare_kernel(const float* __restrict__ a, int A, int q_off, int q_rank, int c_off, int kv_rank,
                                      int rot, const float* __restrict__ wq, const float* __restrict__ wc, float eps,
                                      const double* __restrict__ freqs, float gain, const int* __restrict__ positions,
                                      const int* __restrict__ slot_mapping, T* __restrict__ cache, int row,
                                      T* __restrict__ cq) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* src = a + (size_t)t * A;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = src[q_off + i];
    ss += v * v;
  }
  const float rq = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
    cq[(size_t)t * q_rank + i] = from_f32<T>(src[q_off + i] * rq * wq[i]);
  if (kv_rank == 0 || slot_mapping == nullptr) return;
  const int slot = slot_mapping[t];          // the same for the whole block
  if (slot < 0) return;
  ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = src[c_off + i];
    ss += v * v;
  }
  const float rc = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
  T* dst = cache + (size_t)slot * row;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) dst[i] = from_f32<T>(src[c_off + i] * rc * wc[i]);
  const int pos = positions[t];
  for (int i = threadIdx.x; i < rot / 2; i += blockDim.x) {
    float sn, cs;
    nhv_turn_angle(pos, freqs[i], gain, &sn, &cs);
    const float u = src[c_off + kv_rank + 2 * i], v = src[c_off + kv_rank + 2 * i + 1];
    dst[kv_rank + 2 * i] = from_f32<T>(u * cs - v * sn);
    dst[kv_rank + 2 * i + 1] = from_f32<T>(v * cs + u * sn);
  }
}

extern "C" int nhv_latent_prepare(const void* a, int A, int q_off, int q_rank, int c_off, int kv_rank, int rot,
                                  const void* wq, const void* wc, float eps, const void* freqs, float gain,
                                  const void* positions, const void* slot_mapping, void* cache, int row, void* cq, int T,
                                  int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && A > 0 && q_rank > 0 && kv_rank >= 0 && rot >= 0 && rot % 2 == 0,
              "latent_prepare: bad sizes T=%d A=%d q_rank=%d kv_rank=%d rot=%d", T, A, q_rank, kv_rank, rot);
  NHV_REQUIRE(q_off >= 0 && q_off + q_rank <= A && (kv_rank == 0 || (c_off >= 0 && c_off + kv_rank + rot <= A)),
              "latent_prepare: columns %d+%d and %d+%d+%d of %d", q_off, q_rank, c_off, kv_rank, rot, A);
  NHV_REQUIRE(kv_rank == 0 || slot_mapping == nullptr || (cache != nullptr && row >= kv_rank + rot),
              "latent_prepare: cache rows of %d entries for %d + %d", row, kv_rank, rot);
  NHV_REQUIRE(rot == 0 || kv_rank == 0 || freqs != nullptr, "latent_prepare: a rotated part without frequencies");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(T), dim3(256), 0, s, (const float*)a, A, q_off, q_rank, c_off,
                       kv_rank, rot, (const float*)wq, (const float*)wc, eps, (const double*)freqs, gain,
                       (const int*)positions, (const int*)slot_mapping, (float*)cache, row, (float*)cq);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const float*)a, A, q_off, q_rank, c_off,
                       kv_rank, rot, (const float*)wq, (const float*)wc, eps, (const double*)freqs, gain,
                       (const int*)positions, (const int*)slot_mapping, (bf16_t*)cache, row, (bf16_t*)cq);
  else
    return nhv_fail("latent_prepare: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("latent_prepare");
  return 0;
}

// ---------------------------------------------------------------- a matrix per head
// y[t * ys_t + h * ys_h + n] = sum over k of x[t * xs_t + h * xs_h + k] * w[h * ws_h + n * ws_n + k * ws_k], k rising,
// one thread per output, so a row's result does not depend on its batch. A block owns 32 rows x 64 outputs of one head
// and walks over k in pieces of 16 through LDS. gate: y *= sigmoid(gate[t * gs_t + h]).
#define HG_TM 32
#define HG_TN 64
#define HG_TK 16
template <typename T>
__global__ __launch_bounds__(256) void head_gemm_kernel(const T* __restrict__ x, long long xs_t, long long xs_h,
                                                        const T* __restrict__ w, long long ws_h, long long ws_n,
                                                        long long ws_k, T* __restrict__ y, long long ys_t, long long ys_h,
                                                        const float* __restrict__ gate, long long gs_t, int rows, int N,
                                                        int K) {
  __shared__ float xs[HG_TM][HG_TK];
  __shared__ float wt[HG_TN][HG_TK + 1];
  const int h = blockIdx.z;
  const int m0 = blockIdx.x * HG_TM, n0 = blockIdx.y * HG_TN;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  float acc[HG_TM / 4];
#pragma unroll
  for (int i = 0; i < HG_TM / 4; ++i) acc[i] = 0.f;
  const T* xh = x + (size_t)h * xs_h;
  const T* wh = w + (size_t)h * ws_h;
  for (int k0 = 0; k0 < K; k0 += HG_TK) {
    for (int idx = threadIdx.x; idx < HG_TM * HG_TK; idx += 256) {
      const int m = idx / HG_TK, kk = idx % HG_TK;
      xs[m][kk] = (m0 + m < rows && k0 + kk < K) ? to_f32(xh[(size_t)(m0 + m) * xs_t + k0 + kk]) : 0.f;
    }
    for (int idx = threadIdx.x; idx < HG_TN * HG_TK; idx += 256) {
      int n, kk;
      if (ws_k == 1) { n = idx / HG_TK; kk = idx % HG_TK; }
      else { n = idx % HG_TN; kk = idx / HG_TN; }
      wt[n][kk] = (n0 + n < N && k0 + kk < K) ? to_f32(wh[(size_t)(n0 + n) * ws_n + (size_t)(k0 + kk) * ws_k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HG_TK; ++kk) {
      const float wv = wt[tx][kk];
#pragma unroll
      for (int i = 0; i < HG_TM / 4; ++i) acc[i] = fmaf(xs[ty * (HG_TM / 4) + i][kk], wv, acc[i]);
    }
    __syncthreads();
  }
  const int n = n0 + tx;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < HG_TM / 4; ++i) {
    const int m = m0 + ty * (HG_TM / 4) + i;
    if (m >= rows) continue;
    float v = acc[i];
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(size_t)m * gs_t + h]));
    y[(size_t)m * ys_t + (size_t)h * ys_h + n] = from_f32<T>(v);
  }
}

extern "C" int nhv_head_gemm(const void* x, long long xs_t, long long xs_h, const void* w, long long ws_h, long long ws_n,
                             long long ws_k, void* y, long long ys_t, long long ys_h, const void* gate, long long gs_t,
                             int rows, int H, int N, int K, int dtype, void* stream) {
  NHV_REQUIRE(rows > 0 && H > 0 && N > 0 && K > 0 && H <= 65535, "head_gemm: bad sizes rows=%d H=%d N=%d K=%d", rows, H, N, K);
  const dim3 grid((rows + HG_TM - 1) / HG_TM, (N + HG_TN - 1) / HG_TN, H);
  NHV_REQUIRE(grid.y <= 65535, "head_gemm: %d outputs a head are too many", N);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(head_gemm_kernel<float>, grid, dim3(256), 0, s, (const float*)x, xs_t, xs_h, (const float*)w, ws_h,
                       ws_n, ws_k, (float*)y, ys_t, ys_h, (const float*)gate, gs_t, rows, N, K);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(head_gemm_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)x, xs_t, xs_h, (const bf16_t*)w,
                       ws_h, ws_n, ws_k, (bf16_t*)y, ys_t, ys_h, (const float*)gate, gs_t, rows, N, K);
  else
    return nhv_fail("head_gemm: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("head_gemm");
  return 0;
}

// The same for up to 16 rows (a decoding step): a block owns 64 outputs of one head. It first brings the head's rows
// of x (as floats) and its 64 x K piece of the matrix into LDS, every thread asking for all its share at once (a
// thread that walked over k with loads from memory waited for memory at every step); then lane = output, wave = four
// of the rows, k rising as above, so the sums are the same bits. One more block a head may turn the rotated part of x
// and copy it beside the outputs (``rot`` entries from x_rot_off to y_rot_off), which saves the launch of
// nhv_rotate_interleaved.
template <typename V>
__device__ __forceinline__ void hg_load8f(const V* p, float* out);
template <>
__device__ __forceinline__ void hg_load8f<bf16_t>(const bf16_t* p, float* out) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 v8;
  const v8 v = *reinterpret_cast<const v8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
}
template <>
__device__ __forceinline__ void hg_load8f<float>(const float* p, float* out) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w; out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}

// VEC: K and N are multiples of 8 and every row of x and of the matrix starts at a multiple of 8 entries from an
// address that is a multiple of 32 bytes (the host checks), so eight entries can be asked for at once.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void head_gemm_fewrows_kernel(const T* __restrict__ x, long long xs_t, long long xs_h,
                                                                const T* __restrict__ w, long long ws_h, long long ws_n,
                                                                long long ws_k, T* __restrict__ y, long long ys_t,
                                                                long long ys_h, const float* __restrict__ gate,
                                                                long long gs_t, int rows, int N, int K, int n_chunks, int rot,
                                                                int x_rot_off, int y_rot_off, const double* __restrict__ freqs,
                                                                float gain, const int* __restrict__ positions) {
  extern __shared__ float xs[];              // 16 x K floats, then the block's piece of the matrix
  const int h = blockIdx.y;
  if ((int)blockIdx.x == n_chunks) {         // the rotated part
    for (int i = threadIdx.x; i < rows * (rot / 2); i += blockDim.x) {
      const int t = i / (rot / 2), p = i % (rot / 2);
      float sn, cs;
      nhv_turn_angle(positions[t], freqs[p], gain, &sn, &cs);
      const T* s = x + (size_t)t * xs_t + (size_t)h * xs_h + x_rot_off + 2 * p;
      T* d = y + (size_t)t * ys_t + (size_t)h * ys_h + y_rot_off + 2 * p;
      const float u = to_f32(s[0]), v = to_f32(s[1]);
      d[0] = from_f32<T>(u * cs - v * sn);
      d[1] = from_f32<T>(v * cs + u * sn);
    }
    return;
  }
  // [K][LDW]: rows a little longer than 64 outputs: pieces of 16 bytes stay aligned, and threads that walk along k (a
  // matrix that is contiguous in k) do not all store into one bank
  constexpr int LDW = 64 + 16 / (int)sizeof(T);
  T* wl = reinterpret_cast<T*>(xs + 16 * K);
  const int n0 = blockIdx.x * 64;
  const T* wh = w + (size_t)h * ws_h;
  const T* xh = x + (size_t)h * xs_h;
  if (VEC) {
    // eight entries a load, and all of a thread's loads asked for before the first is stored (the matrix comes from
    // memory: a thread that stored each piece before it asked for the next waited once a piece)
    const int w_chunks = 8 * K;              // 64 x K / 8
    for (int c0 = 0; c0 < w_chunks; c0 += 256 * 8) {
      float v[8][8];
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const int c = c0 + b * 256 + (int)threadIdx.x;
        if (c >= w_chunks) continue;
        int n, k;
        if (ws_k == 1) { n = c / (K / 8); k = (c % (K / 8)) * 8; }
        else { k = c / 8; n = (c % 8) * 8; }
        const bool ok = ws_k == 1 ? n0 + n < N : n0 + n + 7 < N;
        if (ok) hg_load8f(wh + (size_t)(n0 + n) * ws_n + (size_t)k * ws_k, v[b]);
        else {
#pragma unroll
          for (int i = 0; i < 8; ++i) v[b][i] = (ws_k != 1 && n0 + n + i < N) ? to_f32(wh[(size_t)(n0 + n + i) + (size_t)k * ws_k]) : 0.f;
        }
      }
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const int c = c0 + b * 256 + (int)threadIdx.x;
        if (c >= w_chunks) continue;
        if (ws_k == 1) {
          const int n = c / (K / 8), k = (c % (K / 8)) * 8;
#pragma unroll
          for (int i = 0; i < 8; ++i) wl[(k + i) * LDW + n] = from_f32<T>(v[b][i]);
        } else {
          const int k = c / 8, n = (c % 8) * 8;
#pragma unroll
          for (int i = 0; i < 8; ++i) wl[k * LDW + n + i] = from_f32<T>(v[b][i]);
        }
      }
    }
    const int x_chunks = 2 * K;              // 16 x K / 8
    for (int c = threadIdx.x; c < x_chunks; c += blockDim.x) {
      const int t = c / (K / 8), k = (c % (K / 8)) * 8;
      float v[8];
      if (t < rows) hg_load8f(xh + (size_t)t * xs_t + k, v);
#pragma unroll
      for (int i = 0; i < 8; ++i) xs[t * K + k + i] = t < rows ? v[i] : 0.f;
    }
  } else {
    if (ws_k == 1) {                         // a row of the matrix is contiguous in k: threads walk along k
      for (int i = threadIdx.x; i < 64 * K; i += blockDim.x) {
        const int n = i / K, k = i % K;
        wl[k * LDW + n] = n0 + n < N ? wh[(size_t)(n0 + n) * ws_n + k] : from_f32<T>(0.f);
      }
    } else {                                 // contiguous in n
      for (int i = threadIdx.x; i < 64 * K; i += blockDim.x) {
        const int k = i / 64, n = i % 64;
        wl[k * LDW + n] = n0 + n < N ? wh[(size_t)(n0 + n) * ws_n + (size_t)k * ws_k] : from_f32<T>(0.f);
      }
    }
    for (int i = threadIdx.x; i < 16 * K; i += blockDim.x) {
      const int t = i / K, k = i % K;
      xs[i] = t < rows ? to_f32(xh[(size_t)t * xs_t + k]) : 0.f;
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, t0 = (threadIdx.x >> 6) * 4;
  const int n = n0 + lane;
  if (n >= N || t0 >= rows) return;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const float* x0 = xs + t0 * K;
  for (int k = 0; k < K; ++k) {
    const float wv = to_f32(wl[k * LDW + lane]);
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[t] = fmaf(x0[t * K + k], wv, acc[t]);
  }
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if (t0 + t >= rows) break;
    float v = acc[t];
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(size_t)(t0 + t) * gs_t + h]));
    y[(size_t)(t0 + t) * ys_t + (size_t)h * ys_h + n] = from_f32<T>(v);
  }
}

extern "C" int nhv_head_gemm_fewrows(const void* x, long long xs_t, long long xs_h, const void* w, long long ws_h,
                                     long long ws_n, long long ws_k, void* y, long long ys_t, long long ys_h, const void* gate,
                                     long long gs_t, int rows, int H, int N, int K, int rot, int x_rot_off, int y_rot_off,
                                     const void* freqs, float gain, const void* positions, int dtype, void* stream) {
  const size_t item = dtype == NHV_F32 ? 4 : 2;
  const size_t lds = 16 * (size_t)K * sizeof(float) + (64 + 16 / item) * (size_t)K * item;
  NHV_REQUIRE(rows > 0 && rows <= 16 && H > 0 && H <= 65535 && N > 0 && K > 0 && lds <= 96 * 1024,
              "head_gemm_fewrows: bad sizes rows=%d (up to 16) H=%d N=%d K=%d (LDS of %zu bytes, up to 98304)", rows, H, N, K, lds);
  NHV_REQUIRE(rot >= 0 && rot % 2 == 0 && (rot == 0 || (freqs != nullptr && positions != nullptr)),
              "head_gemm_fewrows: a rotated part of %d entries needs frequencies and positions", rot);
  const int n_chunks = (N + 63) / 64;
  const dim3 grid(n_chunks + (rot > 0 ? 1 : 0), H);
  hipStream_t s = (hipStream_t)stream;
  const long long strides[] = {xs_t, xs_h, ws_h, ws_n == 1 ? ws_k : ws_n};
  bool vec = K % 8 == 0 && N % 8 == 0 && (uintptr_t)x % 32 == 0 && (uintptr_t)w % 32 == 0 && (ws_n == 1 || ws_k == 1);
  for (long long st : strides) vec = vec && st % 8 == 0;
#define NHV_HG_LAUNCH(TYPE, VEC)                                                                                          \
  do {                                                                                                                    \
    if (lds > 64 * 1024)                                                                                                  \
      (void)hipFuncSetAttribute((const void*)head_gemm_fewrows_kernel<TYPE, VEC>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
    hipLaunchKernelGGL((head_gemm_fewrows_kernel<TYPE, VEC>), grid, dim3(256), lds, s, (const TYPE*)x, xs_t, xs_h,          \
                       (const TYPE*)w, ws_h, ws_n, ws_k, (TYPE*)y, ys_t, ys_h, (const float*)gate, gs_t, rows, N, K, n_chunks, \
                       rot, x_rot_off, y_rot_off, (const double*)freqs, gain, (const int*)positions);                      \
  } while (0)
  if (dtype == NHV_F32) {
    if (vec) NHV_HG_LAUNCH(float, true); else NHV_HG_LAUNCH(float, false);
  } else if (dtype == NHV_BF16) {
    if (vec) NHV_HG_LAUNCH(bf16_t, true); else NHV_HG_LAUNCH(bf16_t, false);
  } else {
    return nhv_fail("head_gemm_fewrows: unknown dtype %d", dtype);
  }
#undef NHV_HG_LAUNCH
  NHV_LAUNCH_CHECK("head_gemm_fewrows");
  return 0;
}

// ---------------------------------------------------------------- the gate alone
// y[t, h, :] *= sigmoid(gate[t * gs_t + h]) for rows that a library product has made
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ y, const float* __restrict__ gate, long long gs_t, int H, int N, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t th = i / N;
    const float g = gate[(th / H) * gs_t + th % H];
    y[i] = from_f32<T>(to_f32(y[i]) * (1.0f / (1.0f + expf(-g))));
  }
}

extern "C" int nhv_head_gate(void* y, const void* gate, long long gs_t, int rows, int H, int N, int dtype, void* stream) {
  NHV_REQUIRE(rows > 0 && H > 0 && N > 0 && gate != nullptr, "head_gate: bad sizes rows=%d H=%d N=%d", rows, H, N);
  const size_t total = (size_t)rows * H * N;
  const int blocks = (int)((total + 255) / 256 > 65535 * 4 ? 65535 * 4 : (total + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(head_gate_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)y, (const float*)gate, gs_t, H, N, total);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (bf16_t*)y, (const float*)gate, gs_t, H, N, total);
  else
    return nhv_fail("head_gate: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("head_gate");
  return 0;
}

// ---------------------------------------------------------------- the rotated part of the queries
// dst[t, h, d_off + j] = turned src[t, h, s_off + j], j < rot; src rows of ``s_row`` entries a head, dst of ``d_row``.
template <typename T>
__global__ void rotate_interleaved_kernel(const T* __restrict__ src, int s_row, int s_off, T* __restrict__ dst, int d_row,
                                          int d_off, int rot, const double* __restrict__ freqs, float gain,
                                          const int* __restrict__ positions, int H, size_t total) {
  const int half = rot / 2;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const int p = (int)(i % half);
    const size_t th = i / half;
    const int t = (int)(th / H);
    float sn, cs;
    nhv_turn_angle(positions[t], freqs[p], gain, &sn, &cs);
    const T* s = src + th * s_row + s_off + 2 * p;
    T* d = dst + th * d_row + d_off + 2 * p;
    const float u = to_f32(s[0]), v = to_f32(s[1]);
    d[0] = from_f32<T>(u * cs - v * sn);
    d[1] = from_f32<T>(v * cs + u * sn);
  }
}

extern "C" int nhv_rotate_interleaved(const void* src, int s_row, int s_off, void* dst, int d_row, int d_off, int rot,
                                      const void* freqs, float gain, const void* positions, int T, int H, int dtype,
                                      void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && rot > 0 && rot % 2 == 0, "rotate_interleaved: bad sizes T=%d H=%d rot=%d", T, H, rot);
  NHV_REQUIRE(s_off >= 0 && s_off + rot <= s_row && d_off >= 0 && d_off + rot <= d_row,
              "rotate_interleaved: %d entries at %d of %d into %d of %d", rot, s_off, s_row, d_off, d_row);
  const size_t total = (size_t)T * H * (rot / 2);
  const int blocks = (int)((total + 255) / 256 > 65535 * 4 ? 65535 * 4 : (total + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(rotate_interleaved_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)src, s_row, s_off,
                       (float*)dst, d_row, d_off, rot, (const double*)freqs, gain, (const int*)positions, H, total);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(rotate_interleaved_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)src, s_row, s_off,
                       (bf16_t*)dst, d_row, d_off, rot, (const double*)freqs, gain, (const int*)positions, H, total);
  else
    return nhv_fail("rotate_interleaved: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("rotate_interleaved");
  return 0;
}
