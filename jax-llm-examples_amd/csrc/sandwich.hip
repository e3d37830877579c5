// Kernels of the sandwich arrangement (a norm before and behind every branch, a sigmoid gate on the branch's
// output, a token shift before the mixer) and of the polynomial activation.
//
// add_norm_shift: per row
//     t  = (y + y_bias) * sigmoid(g + g_bias)                       the gated branch output (or a plain delta, or none)
//     x' = x + t / sqrt(mean(t^2) + eps_b) * w_b                    the residual sum, float32, into a NEW array
//     h  = x' / sqrt(mean(x'^2) + eps) * w                          the next branch's input
//     hs = h + (h_prev - h) * shift                                 h_prev: the float32 h of the token before
// h_prev of a segment's first row comes from the request's state (zeros at position 0); the h of a segment's last
// row goes into the state's other half.  A block takes `rows_per_block` consecutive rows one after the other and
// keeps the last h in registers; if its first row is not a segment's first, it forms the h of the row before
// anew (which is why the sum is not written in place).  Every row's arithmetic is the same whatever block it
// is in, so a token's result does not depend on how its request was cut into steps or batched.
#include "common.h"
#include "rows.h"

using namespace jle;

namespace {

constexpr int kThreads = 256;

template <typename T, int VEC>
__device__ __forceinline__ void load_piece(const T* p, float (&o)[VEC]) {
  if constexpr (VEC == 4) {
    const f32x4_t r = load4<T>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = r[e];
  } else {
    o[0] = Num<T>::load(p);
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void store_piece(T* p, const float (&o)[VEC]) {
  if constexpr (VEC == 4) {
    store4<T>(p, f32x4_t{o[0], o[1], o[2], o[3]});
  } else {
    Num<T>::store(p, o[0]);
  }
}

struct SandwichArgs {
  const float* x;        // [N, D]
  float* x_out;          // [N, D] or null (no delta: the residual stays as it is)
  int delta_kind;        // 0 none, 1 plain [N, D], 2 gated
  const void* y;         // [N, D]
  const float* y_bias;   // [D] or null
  const void* g;         // [N, D]
  const float* g_bias;   // [D] or null
  const float* post_w;   // [D] or null
  float post_eps;
  int do_norm;
  const float* w;        // [D] or null
  float eps;
  void* h_out;           // [N, D] or null
  const float* shift_w;  // [D] or null: no shift
  void* hs_out;          // [N, D]
  float* state;          // [slots, 2, D]
  const int* positions;
  const int* token_segment;
  const int* cu_seqlens;
  const int* state_slots;
  const int* state_phase;
  int N, D, rows_per_block;
};

template <typename T, int CPT, int VEC>
__global__ __launch_bounds__(kThreads) void add_norm_shift_kernel(SandwichArgs a) {
  __shared__ float red[kThreads / 64];
  const int D = a.D;
  const int r0 = blockIdx.x * a.rows_per_block;
  const int r1 = min(a.N, r0 + a.rows_per_block);
  const bool shift = a.shift_w != nullptr;
  float hprev[CPT][VEC];
#pragma unroll
  for (int i = 0; i < CPT; ++i)
#pragma unroll
    for (int e = 0; e < VEC; ++e) hprev[i][e] = 0.f;
  int r = r0;
  if (shift && r0 > 0 && a.cu_seqlens[a.token_segment[r0]] != r0) r = r0 - 1;  // the row before, formed anew
  for (; r < r1; ++r) {
    const bool write = r >= r0;
    const size_t base = (size_t)r * D;
    float v[CPT][VEC];
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + kThreads * i) * VEC;
      if (d < D) {
        load_piece<float, VEC>(a.x + base + d, v[i]);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[i][e] = 0.f;
      }
    }
    if (a.delta_kind == 1) {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const int d = (threadIdx.x + kThreads * i) * VEC;
        if (d < D) {
          float t[VEC];
          load_piece<T, VEC>((const T*)a.y + base + d, t);
#pragma unroll
          for (int e = 0; e < VEC; ++e) v[i][e] += t[e];
        }
      }
    } else if (a.delta_kind == 2) {
      float t[CPT][VEC];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const int d = (threadIdx.x + kThreads * i) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) t[i][e] = 0.f;
        if (d < D) {
          float yy[VEC], gg[VEC];
          load_piece<T, VEC>((const T*)a.y + base + d, yy);
          load_piece<T, VEC>((const T*)a.g + base + d, gg);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            const float yb = a.y_bias != nullptr ? yy[e] + a.y_bias[d + e] : yy[e];
            const float gb = a.g_bias != nullptr ? gg[e] + a.g_bias[d + e] : gg[e];
            t[i][e] = yb * (1.0f / (1.0f + expf(-gb)));
            ss = __builtin_fmaf(t[i][e], t[i][e], ss);
          }
        }
      }
      const float tot = block_sum<kThreads>(ss, red);
      const float inv = 1.0f / sqrtf(tot / (float)D + a.post_eps);
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const int d = (threadIdx.x + kThreads * i) * VEC;
        if (d < D) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            float u = t[i][e] * inv;
            if (a.post_w != nullptr) u *= a.post_w[d + e];
            v[i][e] += u;
          }
        }
      }
    }
    if (write && a.x_out != nullptr) {
#pragma unroll
      for (int i = 0; i < CPT; ++i) {
        const int d = (threadIdx.x + kThreads * i) * VEC;
        if (d < D) store_piece<float, VEC>(a.x_out + base + d, v[i]);
      }
    }
    if (!a.do_norm) continue;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < CPT; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) ss = __builtin_fmaf(v[i][e], v[i][e], ss);
    const float tot = block_sum<kThreads>(ss, red);
    const float inv = 1.0f / sqrtf(tot / (float)D + a.eps);
    int seg = 0, first = 0, last = 0, slot = 0, phase = 0, pos = 0;
    if (shift && write) {
      seg = a.token_segment[r];
      first = a.cu_seqlens[seg];
      last = a.cu_seqlens[seg + 1] - 1;
      slot = a.state_slots[seg];
      phase = a.state_phase[seg];
      pos = a.positions[r];
    }
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + kThreads * i) * VEC;
      if (d < D) {
        float h[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          h[e] = v[i][e] * inv;
          if (a.w != nullptr) h[e] *= a.w[d + e];
        }
        if (write) {
          if (a.h_out != nullptr) store_piece<T, VEC>((T*)a.h_out + base + d, h);
          if (shift) {
            if (r == first) {
              if (pos == 0) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) hprev[i][e] = 0.f;
              } else {
                load_piece<float, VEC>(a.state + ((size_t)slot * 2 + phase) * D + d, hprev[i]);
              }
            }
            float hs[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) hs[e] = h[e] + (hprev[i][e] - h[e]) * a.shift_w[d + e];
            store_piece<T, VEC>((T*)a.hs_out + base + d, hs);
            if (r == last) store_piece<float, VEC>(a.state + ((size_t)slot * 2 + (1 - phase)) * D + d, h);
          }
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) hprev[i][e] = h[e];
      }
    }
  }
}

template <typename T, int VEC>
int launch_sandwich(const SandwichArgs& a, hipStream_t s) {
  const int pieces = (a.D + VEC - 1) / VEC;
  const int cpt = (pieces + kThreads - 1) / kThreads;
  dim3 g((unsigned)((a.N + a.rows_per_block - 1) / a.rows_per_block)), b(kThreads);
#define JLE_SANDWICH_CASE(C)                                                                   \
  if (cpt <= C) {                                                                              \
    hipLaunchKernelGGL((add_norm_shift_kernel<T, C, VEC>), g, b, 0, s, a);                     \
    return 0;                                                                                  \
  }
  JLE_SANDWICH_CASE(1)
  JLE_SANDWICH_CASE(2)
  JLE_SANDWICH_CASE(4)
  JLE_SANDWICH_CASE(8)
  if (VEC == 1) {
    JLE_SANDWICH_CASE(16)
    JLE_SANDWICH_CASE(32)
  }
#undef JLE_SANDWICH_CASE
  return JLE_BAD_ARG;
}

// ------------------------------------------------------------------ polynomial activation
// out = c0 N(u) + c1 N(u^2) + c2 N(u^3) + c3,  u = z + bias,  N(v) = v / sqrt(mean(v^2) + eps) over the row.
// PIECES > 0: the row (up to kThreads * VEC * PIECES wide) stays in registers between the sums and the polynomial;
// PIECES == 0: any width, the row is read twice.
template <typename T, int VEC, int PIECES>
__global__ __launch_bounds__(kThreads) void polynorm_kernel(const T* __restrict__ z, int ldz,
                                                            const float* __restrict__ bias,
                                                            const float* __restrict__ coef, float eps,
                                                            T* __restrict__ out, int F) {
  __shared__ float red[kThreads / 64];
  const size_t row = blockIdx.x;
  const T* zr = z + row * ldz;
  T* o = out + row * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  auto sums = [&](const float (&u)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float u2 = u[e] * u[e], u3 = u2 * u[e];
      s1 = __builtin_fmaf(u[e], u[e], s1);
      s2 = __builtin_fmaf(u2, u2, s2);
      s3 = __builtin_fmaf(u3, u3, s3);
    }
  };
  auto fetch = [&](int d, float (&u)[VEC]) {
    load_piece<T, VEC>(zr + d, u);
    if (bias != nullptr) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) u[e] += bias[d + e];
    }
  };
  constexpr int P = PIECES > 0 ? PIECES : 1;
  float kept[P][VEC];
  if constexpr (PIECES > 0) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int d = (threadIdx.x + kThreads * i) * VEC;
#pragma unroll
      for (int e = 0; e < VEC; ++e) kept[i][e] = 0.f;
      if (d < F) fetch(d, kept[i]);
    }
#pragma unroll
    for (int i = 0; i < PIECES; ++i) sums(kept[i]);  // (zeros beyond the row's end add nothing)
  } else {
    for (int d = threadIdx.x * VEC; d < F; d += kThreads * VEC) {
      float u[VEC];
      fetch(d, u);
      sums(u);
    }
  }
  const float t1 = block_sum<kThreads>(s1, red);
  const float t2 = block_sum<kThreads>(s2, red);
  const float t3 = block_sum<kThreads>(s3, red);
  const float i1 = coef[0] / sqrtf(t1 / (float)F + eps);
  const float i2 = coef[1] / sqrtf(t2 / (float)F + eps);
  const float i3 = coef[2] / sqrtf(t3 / (float)F + eps);
  const float c3 = coef[3];
  auto poly = [&](const float (&u)[VEC], float (&v)[VEC]) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float u2 = u[e] * u[e];
      v[e] = u[e] * i1 + u2 * i2 + u2 * u[e] * i3 + c3;
    }
  };
  if constexpr (PIECES > 0) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int d = (threadIdx.x + kThreads * i) * VEC;
      if (d < F) {
        float v[VEC];
        poly(kept[i], v);
        store_piece<T, VEC>(o + d, v);
      }
    }
  } else {
    for (int d = threadIdx.x * VEC; d < F; d += kThreads * VEC) {
      float u[VEC], v[VEC];
      fetch(d, u);
      poly(u, v);
      store_piece<T, VEC>(o + d, v);
    }
  }
}

template <typename T>
void launch_polynorm(const T* z, int ldz, const float* bias, const float* coef, float eps, T* out, int N, int F,
                     bool vec, hipStream_t s) {
  // (which form runs depends on the width and on where the arrays lie, not on the step; the sums of a row are
  // formed in the same order in the forms that keep the row and in the one that reads it twice)
  dim3 g(N), b(kThreads);
  if (vec && F <= kThreads * 4 * 4)
    hipLaunchKernelGGL((polynorm_kernel<T, 4, 4>), g, b, 0, s, z, ldz, bias, coef, eps, out, F);
  else if (vec && F <= kThreads * 4 * 16)
    hipLaunchKernelGGL((polynorm_kernel<T, 4, 16>), g, b, 0, s, z, ldz, bias, coef, eps, out, F);
  else if (vec)
    hipLaunchKernelGGL((polynorm_kernel<T, 4, 0>), g, b, 0, s, z, ldz, bias, coef, eps, out, F);
  else
    hipLaunchKernelGGL((polynorm_kernel<T, 1, 0>), g, b, 0, s, z, ldz, bias, coef, eps, out, F);
}

}  // namespace

JLE_API int jle_add_norm_shift(const float* x, float* x_out, int delta_kind, const void* y, const float* y_bias,
                               const void* g, const float* g_bias, const float* post_w, float post_eps, int do_norm,
                               const float* w, float eps, void* h_out, const float* shift_w, void* hs_out,
                               float* state, const int* positions, const int* token_segment, const int* cu_seqlens,
                               const int* state_slots, const int* state_phase, int is_bf16, int N, int D,
                               int rows_per_block, hipStream_t s) {
  if (N <= 0) return 0;
  if (D <= 0 || rows_per_block < 1 || delta_kind < 0 || delta_kind > 2) return JLE_BAD_ARG;
  if (delta_kind != 0 && (y == nullptr || x_out == nullptr)) return JLE_BAD_ARG;
  if (delta_kind == 2 && g == nullptr) return JLE_BAD_ARG;
  if (shift_w != nullptr && (!do_norm || hs_out == nullptr || state == nullptr || positions == nullptr ||
                             token_segment == nullptr || cu_seqlens == nullptr || state_slots == nullptr ||
                             state_phase == nullptr))
    return JLE_BAD_ARG;
  SandwichArgs a{x, x_out, delta_kind, y, y_bias, g, g_bias, post_w, post_eps, do_norm, w, eps, h_out, shift_w,
                 hs_out, state, positions, token_segment, cu_seqlens, state_slots, state_phase, N, D,
                 shift_w != nullptr ? rows_per_block : 1};
  auto aligned = [](const void* p) { return p == nullptr || ((uintptr_t)p % 16) == 0; };
  const bool vec = D % 4 == 0 && aligned(x) && aligned(x_out) && aligned(y) && aligned(g) && aligned(h_out) &&
                   aligned(hs_out) && aligned(state) && D <= kThreads * 8 * 4;
  int rc;
  if (is_bf16)
    rc = vec ? launch_sandwich<bf16_t, 4>(a, s) : launch_sandwich<bf16_t, 1>(a, s);
  else
    rc = vec ? launch_sandwich<float, 4>(a, s) : launch_sandwich<float, 1>(a, s);
  if (rc != 0) return rc;
  JLE_LAUNCH_CHECK();
  return 0;
}

JLE_API int jle_polynorm(const void* z, int ldz, const float* bias, const float* coef, float eps, void* out,
                         int is_bf16, int N, int F, hipStream_t s) {
  if (N <= 0) return 0;
  if (F <= 0 || ldz < F || coef == nullptr) return JLE_BAD_ARG;
  const bool vec = F % 4 == 0 && ldz % 4 == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)out % 16 == 0;
  if (is_bf16)
    launch_polynorm<bf16_t>((const bf16_t*)z, ldz, bias, coef, eps, (bf16_t*)out, N, F, vec, s);
  else
    launch_polynorm<float>((const float*)z, ldz, bias, coef, eps, (float*)out, N, F, vec, s);
  JLE_LAUNCH_CHECK();
  return 0;
}
