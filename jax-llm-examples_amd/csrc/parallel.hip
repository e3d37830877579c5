// The norm of a layer whose branches run in parallel: both branches read the same residual stream, each through
// a norm with weights of its own, so one kernel adds what is pending, forms the row's statistics once and writes
// the two normed rows:
//     x += (a + b)            the two branch outputs of the layer before (run dtype, summed in float32; b optional)
//     x += rows + vec         what a looped stretch of layers injects where a pass begins (float32; both optional)
//     h1 = x / sqrt(mean(x^2) + eps) * w1,   h2 = ... * w2
// One block per row, the row in registers (THREADS * EPT elements; wider rows are read again).  The sum of squares
// is formed in an order that depends on the width only, so a token's rows do not depend on what else is in the step.
#include "common.h"
#include "rows.h"

using namespace jle;

namespace {

template <typename DT>
struct PairArgs {
  float* x;          // [N, D] residual, updated in place
  const DT* a;       // [N, D] or null
  const DT* b;       // [N, D] or null
  const float* rows; // [N, D] or null
  const float* vec;  // [D] or null
  const float* w1;   // [D] or null (no weight)
  const float* w2;
  DT* h1;            // [N, D] or null (no norm wanted)
  DT* h2;            // [N, D] or null
  float eps;
  int D;
};

template <typename DT>
__device__ __forceinline__ float updated(const PairArgs<DT>& p, size_t base, int d) {
  float v = p.x[base + d];
  if (p.a != nullptr) {
    float t = Num<DT>::load(p.a + base + d);
    if (p.b != nullptr) t += Num<DT>::load(p.b + base + d);
    v += t;
  }
  if (p.rows != nullptr) v += p.rows[base + d];
  if (p.vec != nullptr) v += p.vec[d];
  return v;
}

template <typename DT, int THREADS, int EPT>
__global__ __launch_bounds__(THREADS) void add_norm_pair_kernel(PairArgs<DT> p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  const bool writes = p.a != nullptr || p.rows != nullptr || p.vec != nullptr;
  float v[EPT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    v[i] = d < D ? updated(p, base, d) : 0.f;
  }
  if (writes) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int d = threadIdx.x + THREADS * i;
      if (d < D) p.x[base + d] = v[i];
    }
  }
  if (p.h1 == nullptr) return;  // (the sums only)
#pragma unroll
  for (int i = 0; i < EPT; ++i) ss = __builtin_fmaf(v[i], v[i], ss);
  const float inv = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)D + p.eps);
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    if (d < D) {
      const float h = v[i] * inv;
      Num<DT>::store(p.h1 + base + d, p.w1 != nullptr ? h * p.w1[d] : h);
      if (p.h2 != nullptr) Num<DT>::store(p.h2 + base + d, p.w2 != nullptr ? h * p.w2[d] : h);
    }
  }
}

// Rows whose width is a multiple of 4, all arrays 16-byte aligned: a thread takes CPT pieces of 4 neighbouring
// elements (piece = thread, thread + THREADS, ...), every load of the row before its first store.
template <typename DT, int THREADS, int CPT>
__global__ __launch_bounds__(THREADS) void add_norm_pair_vec_kernel(PairArgs<DT> p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f}, one = {1.f, 1.f, 1.f, 1.f};
  f32x4_t v[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int d = (threadIdx.x + THREADS * i) * 4;
    v[i] = d < D ? load4<float>(p.x + base + d) : zero;
  }
  if (p.a != nullptr) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      if (d < D) {
        f32x4_t t = load4<DT>(p.a + base + d);
        if (p.b != nullptr) t += load4<DT>(p.b + base + d);
        v[i] += t;
      }
    }
  }
  if (p.rows != nullptr) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      if (d < D) v[i] += load4<float>(p.rows + base + d);
    }
  }
  if (p.vec != nullptr) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      if (d < D) v[i] += load4<float>(p.vec + d);
    }
  }
  if (p.a != nullptr || p.rows != nullptr || p.vec != nullptr) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      if (d < D) store4<float>(p.x + base + d, v[i]);
    }
  }
  if (p.h1 == nullptr) return;  // (the sums only)
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < CPT; ++i) ss = add_squares4(ss, v[i]);
  const float inv = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)D + p.eps);
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int d = (threadIdx.x + THREADS * i) * 4;
    if (d < D) {
      const f32x4_t h = v[i] * inv;
      store4<DT>(p.h1 + base + d, p.w1 != nullptr ? h * load4<float>(p.w1 + d) : h * one);
      if (p.h2 != nullptr) store4<DT>(p.h2 + base + d, p.w2 != nullptr ? h * load4<float>(p.w2 + d) : h * one);
    }
  }
}

// Rows wider than the registers hold: the sums are stored, the row read again for the statistics' use.
template <typename DT, int THREADS>
__global__ __launch_bounds__(THREADS) void add_norm_pair_wide_kernel(PairArgs<DT> p) {
  __shared__ float red[THREADS / 64];
  const size_t base = (size_t)blockIdx.x * p.D;
  const int D = p.D;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += THREADS) {
    const float v = updated(p, base, d);
    p.x[base + d] = v;
    ss = __builtin_fmaf(v, v, ss);
  }
  if (p.h1 == nullptr) return;
  const float inv = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)D + p.eps);
  for (int d = threadIdx.x; d < D; d += THREADS) {
    const float h = p.x[base + d] * inv;  // (this thread's own store)
    Num<DT>::store(p.h1 + base + d, p.w1 != nullptr ? h * p.w1[d] : h);
    if (p.h2 != nullptr) Num<DT>::store(p.h2 + base + d, p.w2 != nullptr ? h * p.w2[d] : h);
  }
}

template <typename DT>
int launch_pair(const PairArgs<DT>& p, int N, hipStream_t s) {
  const int D = p.D;
  // (which kernel: by the width and the arrays' alignment alone, never by the step's size)
  const uintptr_t all = (uintptr_t)p.x | (uintptr_t)p.a | (uintptr_t)p.b | (uintptr_t)p.rows | (uintptr_t)p.vec |
                        (uintptr_t)p.w1 | (uintptr_t)p.w2 | (uintptr_t)p.h1 | (uintptr_t)p.h2;
  if (D % 4 == 0 && all % 16 == 0 && D >= 1024 && D <= 8192) {
    if (D <= 2048)
      hipLaunchKernelGGL((add_norm_pair_vec_kernel<DT, 256, 2>), dim3(N), dim3(256), 0, s, p);
    else if (D <= 4096)
      hipLaunchKernelGGL((add_norm_pair_vec_kernel<DT, 256, 4>), dim3(N), dim3(256), 0, s, p);
    else
      hipLaunchKernelGGL((add_norm_pair_vec_kernel<DT, 512, 4>), dim3(N), dim3(512), 0, s, p);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
  }
  if (D <= 256)
    hipLaunchKernelGGL((add_norm_pair_kernel<DT, 64, 4>), dim3(N), dim3(64), 0, s, p);
  else if (D <= 1024)
    hipLaunchKernelGGL((add_norm_pair_kernel<DT, 256, 4>), dim3(N), dim3(256), 0, s, p);
  else if (D <= 4096)
    hipLaunchKernelGGL((add_norm_pair_kernel<DT, 256, 16>), dim3(N), dim3(256), 0, s, p);
  else if (D <= 8192)
    hipLaunchKernelGGL((add_norm_pair_kernel<DT, 512, 16>), dim3(N), dim3(512), 0, s, p);
  else
    hipLaunchKernelGGL((add_norm_pair_wide_kernel<DT, 512>), dim3(N), dim3(512), 0, s, p);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

}  // namespace

// a, b, h1, h2 in the run dtype (is_bf16); x, rows, vec, w1, w2 float32.  Any of a, b, rows, vec, w1, w2, h2 may be
// null; h1 null: the sums only (then h2 must be null too).  b needs a.
JLE_API int jle_add_norm_pair(float* x, const void* a, const void* b, const float* rows, const float* vec,
                              const float* w1, const float* w2, float eps, void* h1, void* h2, int is_bf16, int N,
                              int D, hipStream_t s) {
  if (N <= 0) return 0;
  if (D <= 0 || x == nullptr || (b != nullptr && a == nullptr) || (h1 == nullptr && h2 != nullptr)) return JLE_BAD_ARG;
  if (is_bf16) {
    PairArgs<bf16_t> p{x, (const bf16_t*)a, (const bf16_t*)b, rows, vec, w1, w2, (bf16_t*)h1, (bf16_t*)h2, eps, D};
    return launch_pair(p, N, s);
  }
  PairArgs<float> p{x, (const float*)a, (const float*)b, rows, vec, w1, w2, (float*)h1, (float*)h2, eps, D};
  return launch_pair(p, N, s);
}
