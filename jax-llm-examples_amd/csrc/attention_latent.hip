// Attention over a cached latent: every token leaves a normed latent c (kv_rank numbers) and one rotated key
// part k_r (rope numbers) in pages; all heads share them.  For a token and a head
//     score_j = (q_lat . c_j + q_r . k_r_j) * scale      over the visible j (a window, or all earlier tokens)
//     out     = sum_j softmax(score)_j c_j
// where q_lat is the head's unrotated query taken into the latent's space by the caller and q_r its rotated part.
// Float32 arithmetic on float32 or bfloat16 storage.
//
//   latent_prepare: rotates the q_r of every head in place, norms the latent, rotates the shared key part and
//                   writes both into their pages (one block per token).
//   latent_attention: one wavefront per (token, head[, key range]); keys in tiles of 64 absolute positions, so
//                   which tiles a query visits depends on its own position and window only.  Scores: a key per
//                   lane; values: latent elements lane, lane + 64, ... per lane, probabilities by shuffle.  With
//                   few tokens a query's tiles are shared between wavefronts and merged in their order.
#include "common.h"

using namespace jle;

namespace {

template <typename T>
struct Vec16L;
template <>
struct Vec16L<float> {
  static constexpr int kN = 4;
  float4 v;
  __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
  __device__ __forceinline__ float get(int i) const { return (&v.x)[i]; }
};
template <>
struct Vec16L<bf16_t> {
  static constexpr int kN = 8;
  uint4 v;
  __device__ __forceinline__ void load(const bf16_t* p) { v = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = (&v.x)[i >> 1];
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
};

// pairing: 0 adjacent (x[2j], x[2j+1]), 1 half-split (x[j], x[j + rd/2]); rd leading elements turn
__device__ __forceinline__ void pair_index(int pairing, int rd, int j, int& a, int& b) {
  if (pairing == 0) {
    a = 2 * j;
    b = 2 * j + 1;
  } else {
    a = j;
    b = j + rd / 2;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(T* __restrict__ rows, int ld, int H, int dn, int dr,
                                                             int R, const int* __restrict__ positions,
                                                             const float* __restrict__ inv_freq, int pairing, int rd,
                                                             const float* __restrict__ norm_w, float eps,
                                                             T* __restrict__ latent_pages, T* __restrict__ rope_pages,
                                                             const int* __restrict__ slot_mapping, int writes) {
  __shared__ float red[4];
  const size_t n = blockIdx.x;
  T* row = rows + n * ld;
  const float pos = (float)positions[n];
  const int half = rd / 2;
  // the heads' rotated query parts, in place (a thread owns both elements of its pairs)
  for (int idx = threadIdx.x; idx < H * half; idx += 256) {
    const int h = idx / half, j = idx - h * half;
    int ia, ib;
    pair_index(pairing, rd, j, ia, ib);
    T* q = row + (size_t)h * (dn + dr) + dn;
    float sn, cs;
    sincosf(pos * inv_freq[j], &sn, &cs);
    const float u = Num<T>::load(q + ia), v = Num<T>::load(q + ib);
    Num<T>::store(q + ia, u * cs - v * sn);
    Num<T>::store(q + ib, v * cs + u * sn);
  }
  if (!writes) return;
  const T* c = row + (size_t)H * (dn + dr);
  const T* kr = c + R;
  float ss = 0.f;
  for (int d = threadIdx.x; d < R; d += 256) {
    const float v = Num<T>::load(c + d);
    ss = __builtin_fmaf(v, v, ss);
  }
  const float tot = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)R + eps);
  const size_t slot = (size_t)slot_mapping[n];
  T* lp = latent_pages + slot * R;
  for (int d = threadIdx.x; d < R; d += 256) {
    float v = Num<T>::load(c + d) * inv;
    if (norm_w != nullptr) v *= norm_w[d];
    Num<T>::store(lp + d, v);
  }
  T* rp = rope_pages + slot * dr;
  for (int j = threadIdx.x; j < half; j += 256) {
    int ia, ib;
    pair_index(pairing, rd, j, ia, ib);
    float sn, cs;
    sincosf(pos * inv_freq[j], &sn, &cs);
    const float u = Num<T>::load(kr + ia), v = Num<T>::load(kr + ib);
    Num<T>::store(rp + ia, u * cs - v * sn);
    Num<T>::store(rp + ib, v * cs + u * sn);
  }
  for (int d = rd + threadIdx.x; d < dr; d += 256) rp[d] = kr[d];  // what does not turn
}

constexpr int kMaxAcc = 8;  // latent elements per lane: kv_rank up to 512

template <typename T>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    const T* __restrict__ q_lat /* [H, N, R] */, const T* __restrict__ q /* rows of q_ld: [H, dn + dr] first */,
    int q_ld, int dn, int dr,
    const T* __restrict__ latent_pages, const T* __restrict__ rope_pages, T* __restrict__ out /* [N, H, R] */,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, int window, float scale, int N, int H, int R, int ps, int splits, int tiles_per_split,
    float* __restrict__ ws_ml, float* __restrict__ ws_o, int vec /* rows may be read 16 bytes at a time */) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= N * H * splits) return;  // whole wavefront leaves; no block-wide barrier below
  const int sp = item % splits, nh = item / splits;
  const int n = nh / H, h = nh - n * H;
  const int pos = positions[n];
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_table + (size_t)token_segment[n] * table_width;
  const T* ql = q_lat + ((size_t)h * N + n) * R;
  const T* qr = q + (size_t)n * q_ld + (size_t)h * (dn + dr) + dn;

  float m = -INFINITY, l = 0.f;
  float acc[kMaxAcc];
#pragma unroll
  for (int i = 0; i < kMaxAcc; ++i) acc[i] = 0.f;
  bool bad = false;

  int t_lo = (first / 64) * 64, t_hi = pos;
  if (splits > 1) {
    t_lo += sp * tiles_per_split * 64;
    t_hi = min(pos, t_lo + tiles_per_split * 64 - 1);
  }
  for (int t0 = t_lo; t0 <= t_hi; t0 += 64) {
    const int key = t0 + lane;
    const bool valid = key >= first && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = table[key / ps];
      if (page < 0) {
        bad = true;
      } else {
        const size_t slot = (size_t)page * ps + key % ps;
        const T* crow = latent_pages + slot * R;
        const T* krow = rope_pages + slot * dr;
        float dot = 0.f;
        int c = 0;
        for (; vec && c + Vec16L<T>::kN <= R; c += Vec16L<T>::kN) {
          Vec16L<T> a, b;
          a.load(ql + c);
          b.load(crow + c);
#pragma unroll
          for (int i = 0; i < Vec16L<T>::kN; ++i) dot = __builtin_fmaf(a.get(i), b.get(i), dot);
        }
        for (; c < R; ++c) dot = __builtin_fmaf(Num<T>::load(ql + c), Num<T>::load(crow + c), dot);
        for (c = 0; c < dr; ++c) dot = __builtin_fmaf(Num<T>::load(qr + c), Num<T>::load(krow + c), dot);
        s = dot * scale;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    if (m_new == -INFINITY) continue;  // (a tile whose keys are all missing: flagged)
    const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < kMaxAcc; ++i) acc[i] *= corr;
    const int cnt = (pos - t0 + 1) < 64 ? (pos - t0 + 1) : 64;
    const int lo = first > t0 ? first - t0 : 0;
    for (int kk = lo; kk < cnt; ++kk) {
      const float pk = __shfl(p, kk, 64);
      const int page = table[(t0 + kk) / ps];  // the same for the whole wavefront
      if (page < 0) continue;                   // flagged above
      const T* crow = latent_pages + ((size_t)page * ps + (t0 + kk) % ps) * R;
#pragma unroll
      for (int i = 0; i < kMaxAcc; ++i) {
        const int d = lane + 64 * i;
        if (d < R) acc[i] = __builtin_fmaf(pk, Num<T>::load(crow + d), acc[i]);
      }
    }
  }
  bad = __any(bad);
  if (splits > 1) {
    const size_t slot = (size_t)nh * splits + sp;
    if (lane == 0) {
      ws_ml[slot * 2] = bad ? __builtin_nanf("") : m;
      ws_ml[slot * 2 + 1] = l;
    }
#pragma unroll
    for (int i = 0; i < kMaxAcc; ++i) {
      const int d = lane + 64 * i;
      if (d < R) ws_o[slot * R + d] = acc[i];
    }
    return;
  }
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
  T* o = out + (size_t)nh * R;
#pragma unroll
  for (int i = 0; i < kMaxAcc; ++i) {
    const int d = lane + 64 * i;
    if (d < R) Num<T>::store(o + d, acc[i] * inv);
  }
}

// Merges the key ranges of a (token, head): one wavefront each, the ranges in their order.
template <typename T>
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(const float* __restrict__ ws_ml,
                                                                     const float* __restrict__ ws_o,
                                                                     T* __restrict__ out, int NH, int R, int splits) {
  const int lane = threadIdx.x & 63;
  const int nh = blockIdx.x * 4 + wave_index();
  if (nh >= NH) return;
  const float* ml = ws_ml + (size_t)nh * splits * 2;
  float mx = -INFINITY;
  bool bad = false;
  for (int s0 = 0; s0 < splits; s0 += 64) {
    const float ms = s0 + lane < splits ? ml[(s0 + lane) * 2] : -INFINITY;
    bad |= ms != ms;
    mx = fmaxf(mx, ms);
  }
  bad = __any(bad);
  mx = wave_max(mx);
  float l = 0.f;
  float acc[kMaxAcc];
#pragma unroll
  for (int i = 0; i < kMaxAcc; ++i) acc[i] = 0.f;
  for (int sp = 0; sp < splits; ++sp) {
    const float ms = ml[sp * 2], ls = ml[sp * 2 + 1];
    if (ms == -INFINITY || ms != ms) continue;  // a range without keys
    const float wgt = expf(ms - mx);
    l += ls * wgt;
    const float* row = ws_o + ((size_t)nh * splits + sp) * R;
#pragma unroll
    for (int i = 0; i < kMaxAcc; ++i) {
      const int d = lane + 64 * i;
      if (d < R) acc[i] = __builtin_fmaf(row[d], wgt, acc[i]);
    }
  }
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
#pragma unroll
  for (int i = 0; i < kMaxAcc; ++i) {
    const int d = lane + 64 * i;
    if (d < R) Num<T>::store(out + (size_t)nh * R + d, acc[i] * inv);
  }
}

}  // namespace

JLE_API int jle_latent_prepare(void* rows, int ld, int H, int dn, int dr, int R, const int* positions,
                               const float* inv_freq, int pairing, int rd, const float* norm_w, float eps,
                               void* latent_pages, void* rope_pages, const int* slot_mapping, int writes,
                               int is_bf16, int N, hipStream_t s) {
  if (N <= 0) return 0;
  if (H <= 0 || dn < 0 || dr <= 0 || R <= 0 || rd % 2 || rd < 0 || rd > dr || (rd > 0 && inv_freq == nullptr))
    return JLE_BAD_ARG;
  if (ld < H * (dn + dr) + (writes ? R + dr : 0)) return JLE_BAD_ARG;
  if (writes && (latent_pages == nullptr || rope_pages == nullptr || slot_mapping == nullptr)) return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, dim3(N), dim3(256), 0, s, (bf16_t*)rows, ld, H, dn, dr, R,
                       positions, inv_freq, pairing, rd, norm_w, eps, (bf16_t*)latent_pages, (bf16_t*)rope_pages,
                       slot_mapping, writes);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(N), dim3(256), 0, s, (float*)rows, ld, H, dn, dr, R,
                       positions, inv_freq, pairing, rd, norm_w, eps, (float*)latent_pages, (float*)rope_pages,
                       slot_mapping, writes);
  JLE_LAUNCH_CHECK();
  return 0;
}

// splits > 1: every (token, head) is shared between `splits` wavefronts, tiles_per_split tiles of 64 keys each
// counted from the query's first tile, and merged; ws_ml: [N * H * splits * 2], ws_o: [N * H * splits * R] float32.
JLE_API int jle_latent_attention(const void* q_lat, const void* q, int q_ld, int dn, int dr, const void* latent_pages,
                                 const void* rope_pages, void* out, const int* positions, const int* token_segment,
                                 const int* block_table, int table_width, int window, float scale, int is_bf16, int N,
                                 int H, int R, int ps, int splits, int tiles_per_split, float* ws_ml, float* ws_o,
                                 hipStream_t s) {
  if (N <= 0) return 0;
  if (q_ld < H * (dn + dr) || H <= 0 || R <= 0 || R > 64 * kMaxAcc || dr <= 0 || dn < 0 || ps <= 0 || window < 0) return JLE_BAD_ARG;
  // rows are read 16 bytes at a time where every row starts at a multiple of 16 bytes
  const int per16 = is_bf16 ? 8 : 4;
  const int vec = R % per16 == 0 && (uintptr_t)q_lat % 16 == 0 && (uintptr_t)latent_pages % 16 == 0;
  if (splits < 1 || (splits > 1 && (tiles_per_split < 1 || ws_ml == nullptr || ws_o == nullptr))) return JLE_BAD_ARG;
  const long long items = (long long)N * H * splits;
  if (items > (1ll << 31) - 8) return JLE_BAD_ARG;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
  dim3 gm((unsigned)(((long long)N * H + 3) / 4));
  if (is_bf16) {
    hipLaunchKernelGGL(latent_attention_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)q_lat, (const bf16_t*)q, q_ld, dn, dr,
                       (const bf16_t*)latent_pages, (const bf16_t*)rope_pages, (bf16_t*)out, positions, token_segment,
                       block_table, table_width, window, scale, N, H, R, ps, splits, tiles_per_split, ws_ml, ws_o, vec);
    JLE_LAUNCH_CHECK();
    if (splits > 1)
      hipLaunchKernelGGL(latent_attention_merge_kernel<bf16_t>, gm, b, 0, s, ws_ml, ws_o, (bf16_t*)out, N * H, R,
                         splits);
  } else {
    hipLaunchKernelGGL(latent_attention_kernel<float>, g, b, 0, s, (const float*)q_lat, (const float*)q, q_ld, dn, dr,
                       (const float*)latent_pages, (const float*)rope_pages, (float*)out, positions, token_segment,
                       block_table, table_width, window, scale, N, H, R, ps, splits, tiles_per_split, ws_ml, ws_o, vec);
    JLE_LAUNCH_CHECK();
    if (splits > 1)
      hipLaunchKernelGGL(latent_attention_merge_kernel<float>, gm, b, 0, s, ws_ml, ws_o, (float*)out, N * H, R,
                         splits);
  }
  JLE_LAUNCH_CHECK();
  return 0;
}
