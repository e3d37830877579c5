// Attention over a cached latent: every token leaves a normed latent c (kv_rank numbers) and one rotated key
// part k_r (rope numbers) in pages; all heads share them.  For a token and a head
//     score_j = (q_lat . c_j + q_r . k_r_j) * scale      over the visible j (a window, or all earlier tokens)
//     out     = sum_j softmax(score)_j c_j
// where q_lat is the head's unrotated query taken into the latent's space by the caller and q_r its rotated part.
// Float32 arithmetic on float32 or bfloat16 storage.  With a sink (one learned number per head) the softmax's
// denominator has one more term, exp(sink): no key, no value, not scaled, counted once (where a query's keys are
// shared between wavefronts: by the merge).
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
                                                             float magnitude /* on sines and cosines */,
                                                             const float* __restrict__ norm_w, float eps,
                                                             T* __restrict__ latent_pages, T* __restrict__ rope_pages,
                                                             T* __restrict__ latent_t_pages, int ps,
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
    sn *= magnitude;
    cs *= magnitude;
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
    // the same numbers with the page's tokens as the fastest index, for the matrix-core kernel's second product
    if (latent_t_pages != nullptr) Num<T>::store(latent_t_pages + ((slot / ps) * R + d) * ps + slot % ps, v);
  }
  T* rp = rope_pages + slot * dr;
  for (int j = threadIdx.x; j < half; j += 256) {
    int ia, ib;
    pair_index(pairing, rd, j, ia, ib);
    float sn, cs;
    sincosf(pos * inv_freq[j], &sn, &cs);
    sn *= magnitude;
    cs *= magnitude;
    const float u = Num<T>::load(kr + ia), v = Num<T>::load(kr + ib);
    Num<T>::store(rp + ia, u * cs - v * sn);
    Num<T>::store(rp + ib, v * cs + u * sn);
  }
  for (int d = rd + threadIdx.x; d < dr; d += 256) rp[d] = kr[d];  // what does not turn
}

constexpr int kMaxAcc = 16;  // latent elements per lane: kv_rank up to 1024

// What the sums over the keys (maximum m, denominator l) are multiplied with at the end: 1 / l, or with a sink
// 1 / (l + exp(sink - m)), formed about the larger of m and the sink.
__device__ __forceinline__ float closing_factor(float m, float l, const float* __restrict__ sink, int h) {
  if (sink == nullptr) return 1.0f / l;
  const float sk = sink[h];
  const float top = fmaxf(m, sk);
  const float a = expf(m - top);
  return a / (l * a + expf(sk - top));
}

template <typename T>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    const T* __restrict__ q_lat /* [H, N, R] */, const T* __restrict__ q /* rows of q_ld: [H, dn + dr] first */,
    int q_ld, int dn, int dr,
    const T* __restrict__ latent_pages, const T* __restrict__ rope_pages, T* __restrict__ out /* [N, H, R] */,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, int window, float scale, int N, int H, int R, int ps, int splits, int tiles_per_split,
    float* __restrict__ ws_ml, float* __restrict__ ws_o, int vec /* rows may be read 16 bytes at a time */,
    const float* __restrict__ sink /* [H] or null */) {
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
  const float inv = bad ? __builtin_nanf("") : closing_factor(m, l, sink, h);
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
                                                                     T* __restrict__ out, int NH, int R, int splits,
                                                                     const float* __restrict__ sink, int H) {
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
  if (sink != nullptr) {  // (rows are token * H + head)
    const float sk = sink[nh % H];
    mx = fmaxf(mx, sk);
    l = expf(sk - mx);
  }
  float acc[kMaxAcc];
#pragma unroll
  for (int i = 0; i < kMaxAcc; ++i) acc[i] = 0.f;
  // the sums in the ranges' order; four ranges' rows are asked for before the first is added
  constexpr int U = 4;
  for (int s0 = 0; s0 < splits; s0 += U) {
    float ms[U], ls[U], o[U][kMaxAcc];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int sp = min(s0 + u, splits - 1);  // (past the last: loaded again, not used)
      ms[u] = ml[sp * 2];
      ls[u] = ml[sp * 2 + 1];
      const float* row = ws_o + ((size_t)nh * splits + sp) * R;
#pragma unroll
      for (int i = 0; i < kMaxAcc; ++i) {
        const int d = lane + 64 * i;
        o[u][i] = d < R ? row[d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (s0 + u >= splits) break;
      if (ms[u] == -INFINITY || ms[u] != ms[u]) continue;  // a range without keys
      const float wgt = expf(ms[u] - mx);
      l += ls[u] * wgt;
#pragma unroll
      for (int i = 0; i < kMaxAcc; ++i) acc[i] = __builtin_fmaf(o[u][i], wgt, acc[i]);
    }
  }
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
#pragma unroll
  for (int i = 0; i < kMaxAcc; ++i) {
    const int d = lane + 64 * i;
    if (d < R) Num<T>::store(out + (size_t)nh * R + d, acc[i] * inv);
  }
}


// ------------------------------------------------------------------ on the matrix cores (bfloat16)
// A wavefront takes 16 consecutive (token, head) rows of one segment (in token-major order: with 16 or more heads
// they are heads of one token, with fewer the heads of a few neighbouring tokens) and walks their keys in steps of
// 32 absolute positions.  Everything is transposed so that no operand is shuffled between the two products:
//     S^T [key, row] = [c_key, k_r_key] . [q_lat_row, q_r_row]     (A: a key's row from its page, B: the queries, held)
//     O^T [d, row]  += c^T [d, key] P^T [key, row]                 (A: the latent's transposed copy, B: P as S left it)
// The first product's key rows are dealt so that a lane ends up with the probabilities of eight consecutive keys,
// which is what the second product's B operand wants.  Softmax statistics in float32; a row's masks are its own
// token's position and window.  With few rows the steps are shared between wavefronts and merged.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

__device__ __forceinline__ u32x4 load16(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }

template <int NR>  // chunks of 32 latent elements: kv_rank <= 32 * NR
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(
    const bf16_t* __restrict__ q_lat, const bf16_t* __restrict__ q, int q_ld, int dn, int dr,
    const bf16_t* __restrict__ latent, const bf16_t* __restrict__ latent_t, const bf16_t* __restrict__ rope,
    bf16_t* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_segment,
    const int* __restrict__ block_table, int table_width, int window, float scale, const int* __restrict__ tiles,
    int num_tiles, int N, int H, int R, int ps, int splits, int steps_per_split, float* __restrict__ ws_ml,
    float* __restrict__ ws_o, const float* __restrict__ sink) {
  const int lane = threadIdx.x & 63, g = lane >> 4, r = lane & 15;
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= num_tiles * splits) return;  // whole wavefront leaves; no block-wide barrier below
  const int tile = item / splits, sp = item - tile * splits;
  const int row0 = tiles[2 * tile], nrows = tiles[2 * tile + 1];
  const bool row_ok = r < nrows;
  const int row = row0 + (row_ok ? r : 0);
  const int n = row / H, h = row - n * H;
  const int pos = positions[n];
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int* table = block_table + (size_t)token_segment[__builtin_amdgcn_readfirstlane(row0 / H)] * table_width;
  int lo = row_ok ? first : 0x7fffffff, hi = row_ok ? pos : -1;
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) {
    lo = min(lo, __shfl_xor(lo, o, 64));
    hi = max(hi, __shfl_xor(hi, o, 64));
  }
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  // the queries: B operands, column = this lane's row, 8 consecutive k per lane
  bf16x8 qb[NR + 2];
  {
    const bf16_t* ql = q_lat + ((size_t)h * N + n) * R;
#pragma unroll
    for (int c = 0; c < NR; ++c) {
      const int k0 = c * 32 + g * 8;
      qb[c] = __builtin_bit_cast(bf16x8, k0 < R ? load16(ql + k0) : zero4);
    }
    const bf16_t* qr = q + (size_t)n * q_ld + (size_t)h * (dn + dr) + dn;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int k0 = c * 32 + g * 8;
      qb[NR + c] = __builtin_bit_cast(bf16x8, k0 < dr ? load16(qr + k0) : zero4);
    }
  }
  float m = -INFINITY, l = 0.f;
  f32x4 acc[NR * 2];
#pragma unroll
  for (int dt = 0; dt < NR * 2; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  int t_lo = (lo / 32) * 32, t_hi = hi;
  if (splits > 1) {
    t_lo += sp * steps_per_split * 32;
    t_hi = min(hi, t_lo + steps_per_split * 32 - 1);
  }
  for (int t0 = t_lo; t0 <= t_hi; t0 += 32) {
    f32x4 st[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      st[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      // which key is row r of this A operand; every load is made (from a place that exists) and what must not
      // count is put to zero afterwards: a load under a branch would wait for the one before it
      const int key = t0 + 8 * (r >> 2) + 4 * t + (r & 3);
      const int page = table[min(key, hi) / ps];
      const bool have = key <= hi && page >= 0;
      const size_t slot = (size_t)max(page, 0) * ps + key % ps;
      const bf16_t* crow = latent + slot * R;
      const bf16_t* krow = rope + slot * dr;
      // (no branch in these loops, not even one that all lanes take alike: loads on the far side of a branch are
      // not asked for before the products on this side are done; a chunk past the latent's width is a product
      // with zeros)
      u32x4 ka[NR + 2];
#pragma unroll
      for (int c = 0; c < NR; ++c) {
        ka[c] = load16(crow + min(c * 32, R - 32) + g * 8);
        if (!have || c * 32 >= R) ka[c] = zero4;
      }
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int k0 = c * 32 + g * 8;
        ka[NR + c] = load16(krow + min(k0, dr - 8));
        if (!have || k0 >= dr) ka[NR + c] = zero4;
      }
      __builtin_amdgcn_sched_barrier(0);  // (every load above is asked for before the first product below)
#pragma unroll
      for (int c = 0; c < NR + 2; ++c)
        st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ka[c]), qb[c], st[t], 0, 0, 0);
    }
    // this lane now holds, for its row, the scores of keys t0 + 8 g .. + 7
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = t0 + 8 * g + e;
      const bool ok = row_ok && key >= first && key <= pos;
      sv[e] = ok ? st[e >> 2][e & 3] * scale : -INFINITY;
      mx = fmaxf(mx, sv[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    float p[8];
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = sv[e] == -INFINITY ? 0.f : expf(sv[e] - m_new);
      psum += p[e];
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = m_new;
    const u32x4 pk = {pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
    const bf16x8 pb = __builtin_bit_cast(bf16x8, pk);
    // the latent's transposed copy: row d of a page holds its tokens side by side
    const int key0 = t0 + 8 * g;
    const int vpage = key0 <= hi ? table[key0 / ps] : -1;
    const bf16_t* vbase = latent_t + ((size_t)max(vpage, 0) * R + r) * ps + key0 % ps;
    // tokens behind the rows' last position are not written yet: what lies there must not meet a zero weight
    const int n_ok = min(8, hi - key0 + 1);
    const bool rescale = !__all(corr == 1.f);  // (only when some row's maximum moved)
    u32x4 keep;
#pragma unroll
    for (int w2 = 0; w2 < 4; ++w2)
      keep[w2] = vpage < 0 ? 0u : (n_ok >= 2 * w2 + 2 ? 0xffffffffu : (n_ok == 2 * w2 + 1 ? 0x0000ffffu : 0u));
    if (rescale) {
#pragma unroll
      for (int dt = 0; dt < NR * 2; ++dt) acc[dt] *= corr;
    }
#pragma unroll
    for (int d0 = 0; d0 < NR * 2; d0 += 16) {  // sixteen operands asked for together
      u32x4 v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        if (d0 + u < NR * 2) {
          v[u] = load16(vbase + (size_t)min((d0 + u) * 16, R - 16) * ps);
          v[u] &= keep;
          if ((d0 + u) * 16 >= R) v[u] = zero4;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 16; ++u)
        if (d0 + u < NR * 2)
          acc[d0 + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, v[u]), pb, acc[d0 + u], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (!row_ok) return;
  if (splits > 1) {
    const size_t slot = (size_t)row * splits + sp;
    if (g == 0) {
      ws_ml[slot * 2] = m;
      ws_ml[slot * 2 + 1] = l;
    }
#pragma unroll
    for (int dt = 0; dt < NR * 2; ++dt)
      if (dt * 16 < R) *reinterpret_cast<f32x4*>(ws_o + slot * R + dt * 16 + g * 4) = acc[dt];
    return;
  }
  const float inv = closing_factor(m, l, sink, h);
  bf16_t* o = out + (size_t)row * R;
#pragma unroll
  for (int dt = 0; dt < NR * 2; ++dt) {
    if (dt * 16 < R) {
      const uint2 w = {pack_bf16(acc[dt][0] * inv, acc[dt][1] * inv), pack_bf16(acc[dt][2] * inv, acc[dt][3] * inv)};
      *reinterpret_cast<uint2*>(o + dt * 16 + g * 4) = w;
    }
  }
}


// The same computation for steps of many tokens: the four wavefronts of a block take four neighbouring row tiles
// (64 consecutive (token, head) rows of one segment), whose keys are nearly the same, and share every step's 32
// keys through shared memory: the block brings the keys' rows ([32][kv_rank + rope], rope padded with zeros to a
// multiple of 32) and the transposed latent ([kv_rank][32]) in once, each wavefront reads its operands from there.
// The next step's data is asked for into registers before this step's products start and stored after them.
template <int NR>
__global__ __launch_bounds__(256) void latent_attention_lds_kernel(
    const bf16_t* __restrict__ q_lat, const bf16_t* __restrict__ q, int q_ld, int dn, int dr,
    const bf16_t* __restrict__ latent, const bf16_t* __restrict__ latent_t, const bf16_t* __restrict__ rope,
    bf16_t* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ token_segment,
    const int* __restrict__ block_table, int table_width, int window, float scale, const int* __restrict__ blocks,
    int N, int H, int R, int ps, const float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int drp = (dr + 31) & ~31;
  const int KS = R + drp + 8, VS = 40;  // row pitches in elements (16 bytes of padding: no bank conflicts)
  const int QS = R + 8;
  bf16_t* sk = reinterpret_cast<bf16_t*>(smem_raw);  // [32][KS]: key t0 + kk in row key_row(kk)
  bf16_t* sv = sk + 32 * KS;                         // [R][VS]
  bf16_t* sq = sv + R * VS;                          // [64][QS]: the rows' queries in the latent's space
  const int tid = threadIdx.x, lane = tid & 63, g = lane >> 4, r = lane & 15;
  const int w = wave_index();
  const int brow0 = blocks[2 * blockIdx.x], bnrows = blocks[2 * blockIdx.x + 1];
  const int n_first = brow0 / H, n_last = (brow0 + bnrows - 1) / H;
  const int bhi = positions[n_last];
  const int pos_first = positions[n_first];
  const int blo = window > 0 ? max(0, pos_first - window + 1) : 0;
  const int* table = block_table + (size_t)token_segment[n_first] * table_width;
  // this wavefront's tile
  const int nrows = min(16, bnrows - 16 * w);
  const bool active = nrows > 0;
  const bool row_ok = r < nrows;
  const int row = brow0 + (row_ok ? 16 * w + r : 0);
  const int n = row / H, h = row - n * H;
  const int pos = positions[n];
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  int lo = row_ok ? first : 0x7fffffff, hi = row_ok ? pos : -1;
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) {
    lo = min(lo, __shfl_xor(lo, o, 64));
    hi = max(hi, __shfl_xor(hi, o, 64));
  }
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  // the queries: the rotated part stays in registers, the part in the latent's space (up to 16 operands a row)
  // lies in shared memory and is read again every step - the registers it would take are what the next step's
  // data waits in
  bf16x8 qrot[2];
  {
    const bf16_t* ql = q_lat + ((size_t)h * N + n) * R;
    bf16_t* mine = sq + (16 * w + r) * QS;
#pragma unroll
    for (int c = 0; c < NR; ++c) {
      const int k0 = c * 32 + g * 8;
      if (k0 < R) *reinterpret_cast<u32x4*>(mine + k0) = load16(ql + k0);
    }
    const bf16_t* qr = q + (size_t)n * q_ld + (size_t)h * (dn + dr) + dn;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int k0 = c * 32 + g * 8;
      u32x4 v = load16(qr + min(k0, dr - 8));
      if (k0 >= dr) v = zero4;
      qrot[c] = __builtin_bit_cast(bf16x8, v);
    }
  }
  const bf16_t* qrow = sq + (16 * w + r) * QS + g * 8;
  float m = -INFINITY, l = 0.f;
  f32x4 acc[NR * 2];
#pragma unroll
  for (int dt = 0; dt < NR * 2; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // what this thread brings in per step, in pieces of 16 bytes: of the keys' rows, eight threads take a key and
  // every eighth piece of its row each; of the transposed latent, four threads take a row of 32 tokens
  constexpr int KMAX = (NR * 4 + 8 + 7) / 8;  // (R + drp) / 8 pieces per key over 8 threads
  constexpr int VMAX = (NR + 1) / 2;          // R x 4 pieces over 256 threads
  const int KC = (R + drp) >> 3;              // pieces per key
  const int k_key = tid >> 3, k_piece = tid & 7;
  // key kk of a step lies in row (kk >> 2 & 1) * 16 + (kk >> 3) * 4 + (kk & 3): the 16 rows of an A operand are
  // neighbours, which with this pitch spreads a read over all banks
  const int k_row = ((k_key >> 2) & 1) * 16 + (k_key >> 3) * 4 + (k_key & 3);
  u32x4 stage_k[KMAX], stage_v[VMAX];
  auto prefetch = [&](int t0) {
    // lane j (of every wavefront) looks up the page of key t0 + (j & 31); the pieces' pages come from there.  Every
    // load is made, from a place that exists, and what must not count is put to zero afterwards: a load under a
    // branch would wait for the one before it.
    const int mykey = t0 + (lane & 31);
    const int mypage = table[min(mykey, bhi) / ps];
    const int mine = mykey <= bhi ? mypage : -1;
    const int page = __shfl(mine, k_key, 64);
    const size_t slot = (size_t)max(page, 0) * ps + (t0 + k_key) % ps;
#pragma unroll
    for (int i = 0; i < KMAX; ++i) {
      const int col = min(k_piece + 8 * i, KC - 1) * 8;
      const bf16_t* src = col < R ? latent + slot * R + col : rope + slot * dr + min(col - R, dr - 8);
      u32x4 v = load16(src);
      if (page < 0 || col - R >= dr) v = zero4;
      stage_k[i] = v;
    }
    const int kq = tid & 3;  // (the same for all of this thread's pieces of the transposed latent)
    const int key0 = t0 + 8 * kq;
    const int vpage = __shfl(mine, 8 * kq, 64);
    const int n_ok = min(8, bhi - key0 + 1);  // (tokens behind the block's last position are not written yet)
    u32x4 keep;
#pragma unroll
    for (int w2 = 0; w2 < 4; ++w2)
      keep[w2] = vpage < 0 ? 0u : (n_ok >= 2 * w2 + 2 ? 0xffffffffu : (n_ok == 2 * w2 + 1 ? 0x0000ffffu : 0u));
    const bf16_t* vsrc = latent_t + (size_t)max(vpage, 0) * R * ps + key0 % ps;
#pragma unroll
    for (int j = 0; j < VMAX; ++j) {
      const int d = min((tid + 256 * j) >> 2, R - 1);
      stage_v[j] = load16(vsrc + (size_t)d * ps) & keep;
    }
  };
  const int t_first = (blo / 32) * 32;
  prefetch(t_first);
  for (int t0 = t_first; t0 <= bhi; t0 += 32) {
    __syncthreads();  // everyone has read the step before
#pragma unroll
    for (int i = 0; i < KMAX; ++i)
      if (k_piece + 8 * i < KC) *reinterpret_cast<u32x4*>(sk + k_row * KS + (k_piece + 8 * i) * 8) = stage_k[i];
#pragma unroll
    for (int j = 0; j < VMAX; ++j) {
      const int id = tid + 256 * j;
      if ((id >> 2) < R) *reinterpret_cast<u32x4*>(sv + (id >> 2) * VS + (id & 3) * 8) = stage_v[j];
    }
    __syncthreads();
    if (t0 + 32 <= bhi) prefetch(t0 + 32);
    if (!active || t0 + 31 < lo || t0 > hi) continue;  // none of this tile's rows sees a key of the step
    // (no branch in these loops: reads on the far side of a branch are not asked for before the products on this
    // side are done; a chunk past the latent's width is a product with zeros.  A chunk of the queries is read once
    // for both key tiles.)
    f32x4 st[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    const bf16_t* arow0 = sk + r * KS + g * 8;
    const bf16_t* arow1 = arow0 + 16 * KS;
#pragma unroll
    for (int c0 = 0; c0 < NR; c0 += 2) {  // two chunks' reads under way at a time, no more: registers
      u32x4 a0[2], a1[2], b[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int off = min((c0 + u) * 32, R - 32);
        a0[u] = load16(arow0 + off);
        a1[u] = load16(arow1 + off);
        b[u] = load16(qrow + off);
        if ((c0 + u) * 32 >= R) b[u] = zero4;
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        st[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a0[u]),
                                                        __builtin_bit_cast(bf16x8, b[u]), st[0], 0, 0, 0);
        st[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a1[u]),
                                                        __builtin_bit_cast(bf16x8, b[u]), st[1], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int off = R + min(c * 32, drp - 32);
      u32x4 a0 = load16(arow0 + off), a1 = load16(arow1 + off);
      if (c * 32 >= drp) a0 = a1 = zero4;
      st[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a0), qrot[c], st[0], 0, 0, 0);
      st[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a1), qrot[c], st[1], 0, 0, 0);
    }
    float sv8[8];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = t0 + 8 * g + e;
      const bool ok = row_ok && key >= first && key <= pos;
      sv8[e] = ok ? st[e >> 2][e & 3] * scale : -INFINITY;
      mx = fmaxf(mx, sv8[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float corr = m_new == -INFINITY ? 1.f : expf(m - m_new);
    float p[8];
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = sv8[e] == -INFINITY ? 0.f : expf(sv8[e] - m_new);
      psum += p[e];
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = m_new;
    const u32x4 pk = {pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
    const bf16x8 pb = __builtin_bit_cast(bf16x8, pk);
    const bf16_t* vrow = sv + r * VS + g * 8;
    if (!__all(corr == 1.f)) {  // (only when some row's maximum moved)
#pragma unroll
      for (int dt = 0; dt < NR * 2; ++dt) acc[dt] *= corr;
    }
    // four operands are read while the four before them are multiplied
    u32x4 vcur[4], vnext[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      vcur[u] = load16(vrow + min(u * 16, R - 16) * VS);
      if (u * 16 >= R) vcur[u] = zero4;
    }
#pragma unroll
    for (int d0 = 0; d0 < NR * 2; d0 += 4) {
      if (d0 + 4 < NR * 2) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          vnext[u] = load16(vrow + min((d0 + 4 + u) * 16, R - 16) * VS);
          if ((d0 + 4 + u) * 16 >= R) vnext[u] = zero4;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        acc[d0 + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vcur[u]), pb, acc[d0 + u], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 4; ++u) vcur[u] = vnext[u];
    }
  }
  if (!row_ok) return;
  const float inv = closing_factor(m, l, sink, h);
  bf16_t* o = out + (size_t)row * R;
#pragma unroll
  for (int dt = 0; dt < NR * 2; ++dt) {
    if (dt * 16 < R) {
      const uint2 w2 = {pack_bf16(acc[dt][0] * inv, acc[dt][1] * inv), pack_bf16(acc[dt][2] * inv, acc[dt][3] * inv)};
      *reinterpret_cast<uint2*>(o + dt * 16 + g * 4) = w2;
    }
  }
}

template <int NR>
int launch_latent_lds(dim3 grid, size_t smem, hipStream_t s, const bf16_t* q_lat, const bf16_t* q, int q_ld, int dn,
                      int dr, const bf16_t* latent, const bf16_t* latent_t, const bf16_t* rope, bf16_t* out,
                      const int* positions, const int* token_segment, const int* block_table, int table_width,
                      int window, float scale, const int* blocks, int N, int H, int R, int ps, const float* sink) {
  static size_t allowed = 0;  // (what this kernel has been given leave to use of the compute unit's shared memory)
  if (smem > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attention_lds_kernel<NR>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return (int)e;
    allowed = smem;
  }
  hipLaunchKernelGGL(latent_attention_lds_kernel<NR>, grid, dim3(256), smem, s, q_lat, q, q_ld, dn, dr, latent,
                     latent_t, rope, out, positions, token_segment, block_table, table_width, window, scale, blocks, N,
                     H, R, ps, sink);
  return 0;
}

}  // namespace

// blocks: (first row, rows) pairs, up to 64 consecutive rows (token * H + head) of one segment each.
JLE_API int jle_latent_attention_lds(const void* q_lat, const void* q, int q_ld, int dn, int dr,
                                     const void* latent_pages, const void* latent_t_pages, const void* rope_pages,
                                     void* out, const int* positions, const int* token_segment,
                                     const int* block_table, int table_width, int window, float scale,
                                     const int* blocks, int num_blocks, int N, int H, int R, int ps,
                                     const float* sink, hipStream_t s) {
  if (N <= 0 || num_blocks <= 0) return 0;
  if (!(R > 0 && R % 32 == 0 && R <= 512 && dr > 0 && dr % 8 == 0 && dr <= 64 && dn % 8 == 0 && q_ld % 8 == 0 &&
        ps % 8 == 0) ||
      H <= 0 || window < 0 || blocks == nullptr || latent_t_pages == nullptr || q_ld < H * (dn + dr))
    return JLE_BAD_ARG;
  const int drp = (dr + 31) & ~31;
  const size_t smem = (size_t)(32 * (R + drp + 8) + R * 40 + 64 * (R + 8)) * sizeof(bf16_t);
  dim3 grid((unsigned)num_blocks);
  int rc;
#define JLE_LATENT_LDS(NRV)                                                                                        \
  rc = launch_latent_lds<NRV>(grid, smem, s, (const bf16_t*)q_lat, (const bf16_t*)q, q_ld, dn, dr,                 \
                              (const bf16_t*)latent_pages, (const bf16_t*)latent_t_pages, (const bf16_t*)rope_pages, \
                              (bf16_t*)out, positions, token_segment, block_table, table_width, window, scale, blocks, \
                              N, H, R, ps, sink)
  if (R <= 128)
    JLE_LATENT_LDS(4);
  else if (R <= 256)
    JLE_LATENT_LDS(8);
  else
    JLE_LATENT_LDS(16);
#undef JLE_LATENT_LDS
  if (rc != 0) return rc;
  JLE_LAUNCH_CHECK();
  return 0;
}

// Whether the matrix-core kernel takes these sizes (bfloat16 only): rows read 16 bytes at a time.
JLE_API int jle_latent_attention_mfma_supported(int R, int dn, int dr, int q_ld, int ps) {
  return R > 0 && R % 32 == 0 && R <= 512 && dr > 0 && dr % 8 == 0 && dr <= 64 && dn % 8 == 0 && q_ld % 8 == 0 &&
         ps % 8 == 0;
}

// tiles: (first row, rows) pairs, rows = token * H + head, up to 16 rows of one segment each.  splits > 1: a tile's
// steps of 32 keys are shared between `splits` wavefronts, steps_per_split each, and merged (ws as below).
JLE_API int jle_latent_attention_mfma(const void* q_lat, const void* q, int q_ld, int dn, int dr,
                                      const void* latent_pages, const void* latent_t_pages, const void* rope_pages,
                                      void* out, const int* positions, const int* token_segment,
                                      const int* block_table, int table_width, int window, float scale,
                                      const int* tiles, int num_tiles, int N, int H, int R, int ps, int splits,
                                      int steps_per_split, float* ws_ml, float* ws_o, const float* sink,
                                      hipStream_t s) {
  if (N <= 0 || num_tiles <= 0) return 0;
  if (!jle_latent_attention_mfma_supported(R, dn, dr, q_ld, ps) || H <= 0 || window < 0 || tiles == nullptr ||
      latent_t_pages == nullptr || q_ld < H * (dn + dr))
    return JLE_BAD_ARG;
  if (splits < 1 || (splits > 1 && (steps_per_split < 1 || ws_ml == nullptr || ws_o == nullptr))) return JLE_BAD_ARG;
  const long long items = (long long)num_tiles * splits;
  if (items > (1ll << 31) - 8) return JLE_BAD_ARG;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
#define JLE_LATENT_MFMA(NRV)                                                                                        \
  hipLaunchKernelGGL(latent_attention_mfma_kernel<NRV>, g, b, 0, s, (const bf16_t*)q_lat, (const bf16_t*)q, q_ld,   \
                     dn, dr, (const bf16_t*)latent_pages, (const bf16_t*)latent_t_pages, (const bf16_t*)rope_pages, \
                     (bf16_t*)out, positions, token_segment, block_table, table_width, window, scale, tiles,        \
                     num_tiles, N, H, R, ps, splits, steps_per_split, ws_ml, ws_o, sink)
  if (R <= 128)
    JLE_LATENT_MFMA(4);
  else if (R <= 256)
    JLE_LATENT_MFMA(8);
  else
    JLE_LATENT_MFMA(16);
#undef JLE_LATENT_MFMA
  JLE_LAUNCH_CHECK();
  if (splits > 1) {
    dim3 gm((unsigned)(((long long)N * H + 3) / 4));
    hipLaunchKernelGGL(latent_attention_merge_kernel<bf16_t>, gm, b, 0, s, ws_ml, ws_o, (bf16_t*)out, N * H, R, splits,
                       sink, H);
    JLE_LAUNCH_CHECK();
  }
  return 0;
}

// out[b][a][:] = in[a][b][:] for rows of row_bytes bytes (a multiple of 4; of 16 where the arrays allow it).
__global__ __launch_bounds__(256) void swap_leading_kernel(const uint32_t* __restrict__ in, uint32_t* __restrict__ out,
                                                           int A, int B, int words) {
  const size_t pair = blockIdx.x;  // = b * A + a
  const int b = (int)(pair / A), a = (int)(pair - (size_t)b * A);
  const uint32_t* src = in + ((size_t)a * B + b) * words;
  uint32_t* dst = out + pair * words;
  if (words % 4 == 0 && ((uintptr_t)in | (uintptr_t)out) % 16 == 0) {
    for (int i = threadIdx.x * 4; i < words; i += 256 * 4)
      *reinterpret_cast<uint4*>(dst + i) = *reinterpret_cast<const uint4*>(src + i);
  } else {
    for (int i = threadIdx.x; i < words; i += 256) dst[i] = src[i];
  }
}

JLE_API int jle_swap_leading(const void* in, void* out, int A, int B, int row_bytes, hipStream_t s) {
  if (A <= 0 || B <= 0) return 0;
  if (row_bytes <= 0 || row_bytes % 4 || (long long)A * B > (1ll << 31) - 1) return JLE_BAD_ARG;
  hipLaunchKernelGGL(swap_leading_kernel, dim3((unsigned)((long long)A * B)), dim3(256), 0, s, (const uint32_t*)in,
                     (uint32_t*)out, A, B, row_bytes / 4);
  JLE_LAUNCH_CHECK();
  return 0;
}

JLE_API int jle_latent_prepare(void* rows, int ld, int H, int dn, int dr, int R, const int* positions,
                               const float* inv_freq, int pairing, int rd, float magnitude, const float* norm_w,
                               float eps, void* latent_pages, void* rope_pages, void* latent_t_pages, int ps,
                               const int* slot_mapping, int writes, int is_bf16, int N, hipStream_t s) {
  if (N <= 0) return 0;
  if (H <= 0 || dn < 0 || dr <= 0 || R <= 0 || rd % 2 || rd < 0 || rd > dr || (rd > 0 && inv_freq == nullptr))
    return JLE_BAD_ARG;
  if (ld < H * (dn + dr) + (writes ? R + dr : 0)) return JLE_BAD_ARG;
  if (writes && (latent_pages == nullptr || rope_pages == nullptr || slot_mapping == nullptr || ps <= 0))
    return JLE_BAD_ARG;
  if (is_bf16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, dim3(N), dim3(256), 0, s, (bf16_t*)rows, ld, H, dn, dr, R,
                       positions, inv_freq, pairing, rd, magnitude, norm_w, eps, (bf16_t*)latent_pages, (bf16_t*)rope_pages,
                       (bf16_t*)latent_t_pages, ps, slot_mapping, writes);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(N), dim3(256), 0, s, (float*)rows, ld, H, dn, dr, R,
                       positions, inv_freq, pairing, rd, magnitude, norm_w, eps, (float*)latent_pages, (float*)rope_pages,
                       (float*)latent_t_pages, ps, slot_mapping, writes);
  JLE_LAUNCH_CHECK();
  return 0;
}

// splits > 1: every (token, head) is shared between `splits` wavefronts, tiles_per_split tiles of 64 keys each
// counted from the query's first tile, and merged; ws_ml: [N * H * splits * 2], ws_o: [N * H * splits * R] float32.
JLE_API int jle_latent_attention(const void* q_lat, const void* q, int q_ld, int dn, int dr, const void* latent_pages,
                                 const void* rope_pages, void* out, const int* positions, const int* token_segment,
                                 const int* block_table, int table_width, int window, float scale, int is_bf16, int N,
                                 int H, int R, int ps, int splits, int tiles_per_split, float* ws_ml, float* ws_o,
                                 const float* sink, hipStream_t s) {
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
                       block_table, table_width, window, scale, N, H, R, ps, splits, tiles_per_split, ws_ml, ws_o, vec,
                       sink);
    JLE_LAUNCH_CHECK();
    if (splits > 1)
      hipLaunchKernelGGL(latent_attention_merge_kernel<bf16_t>, gm, b, 0, s, ws_ml, ws_o, (bf16_t*)out, N * H, R,
                         splits, sink, H);
  } else {
    hipLaunchKernelGGL(latent_attention_kernel<float>, g, b, 0, s, (const float*)q_lat, (const float*)q, q_ld, dn, dr,
                       (const float*)latent_pages, (const float*)rope_pages, (float*)out, positions, token_segment,
                       block_table, table_width, window, scale, N, H, R, ps, splits, tiles_per_split, ws_ml, ws_o, vec,
                       sink);
    JLE_LAUNCH_CHECK();
    if (splits > 1)
      hipLaunchKernelGGL(latent_attention_merge_kernel<float>, gm, b, 0, s, ws_ml, ws_o, (float*)out, N * H, R,
                         splits, sink, H);
  }
  JLE_LAUNCH_CHECK();
  return 0;
}
