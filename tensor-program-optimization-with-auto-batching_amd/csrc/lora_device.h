// Device-side building blocks of the adapter-indexed LoRA delta, shared by the stand-alone gather-matmul
// kernels and by the decode kernels that carry LoRA work inside their own launch.
#pragma once
#include "common.h"

constexpr int LORA_KCHUNK = 512;   // K elements one wave covers per pass: 64 lanes x 8 fp16
constexpr int LORA_MAX_KC = 8;     // K-slices (fp32 partials) per token
constexpr int LORA_MAX_PROJ = 3;   // projections that share x in one batched shrink (q, k, v)
constexpr int LORA_MAX_KQ = 4;     // K-range blocks of dense shrink results

struct LoraKSplit { int ci; int kc; };

static inline LoraKSplit lora_k_split(int K) {
  int ci = ceil_div(K, LORA_KCHUNK * LORA_MAX_KC);
  if (ci < 1) ci = 1;
  return {ci, ceil_div(K, LORA_KCHUNK * ci)};
}

// A batch of shrink problems that share x and the token->adapter table:
//   v_part[p][c][t][:] = A[p][id_t][:, slice c] . x[t, slice c]        (fp32, one partial per K-slice c)
struct LoraShrinkBatch {
  const f16* A[LORA_MAX_PROJ];   // [n_ad, r, K] each
  int n_proj;
  float* vpart;                  // [n_proj][kc][T][r]
  const f16* x;
  const int32_t* ids;
  int T, K, r, n_ad, ci, kc, frag_tt;
  int speculate;                 // request A before the adapter table is read (adapters expected to be in use)
  const int32_t* bucket_of;      // optional [T]: rank bucket of each token; tokens of other buckets count as unadapted
  int bucket;
};

// Adapter id of token t as this launch sees it: -1 outside the table and for tokens of another rank bucket.
__device__ __forceinline__ int lora_token_id(const int32_t* __restrict__ ids, const int32_t* __restrict__ bucket_of,
                                             int bucket, int t, int T) {
  if (t >= T) return -1;
  if (bucket_of != nullptr && bucket_of[t] != bucket) return -1;
  return ids[t];
}

static inline int lora_shrink_units(const LoraShrinkBatch& b) { return b.n_proj * b.n_ad * b.kc; }

// Reduce G per-lane partials across the 64 lanes.  On return every lane holds in p[0] the full sum
// of partial index j (returned); lanes sharing j hold the same value.
template <int G>
__device__ __forceinline__ int reduce_transpose(float (&p)[G], int lane) {
  int j = 0;
  int off = 32;
#pragma unroll
  for (int n = G; n > 1; n >>= 1) {
    const int half = n >> 1;
    const bool hi = (lane & off) != 0;
#pragma unroll
    for (int i = 0; i < half; ++i) {
      // The two candidates are pinned in registers of their own (empty asm): left to itself the compiler folds the
      // selects of all levels into one dynamically indexed read of p[], which it lowers to a 16-way compare/select
      // chain per element - hundreds of instructions instead of two.
      float a = p[i], b = p[i + half];
      asm volatile("" : "+v"(a), "+v"(b));
      const float send = hi ? a : b;
      const float keep = hi ? b : a;
      p[i] = keep + __shfl_xor(send, off, WAVE);
    }
    j += hi ? half : 0;
    off >>= 1;
  }
#pragma unroll
  for (; off > 0; off >>= 1) p[0] += __shfl_xor(p[0], off, WAVE);
  return j;
}

// One wave: adapter a of projection p, K-slice c.  The first 16 rows of its slice of A[a] are requested before the
// token->adapter table has been read (when `speculate` is set: adapters are expected to be in use), so the wave
// pays one memory round trip, not two, before it can start; that matters when the unit shares a launch with a
// bandwidth-saturating GEMV and every round trip queues behind the weight stream.  Tokens bound to a are found
// with ballots; A stays in registers across token pairs whenever the whole slice fits (r <= 16, one chunk).
__device__ __forceinline__ void lora_shrink_unit(const LoraShrinkBatch& b, int unit, int lane) {
  constexpr int G = 16, TB = 2;
  const int c = unit % b.kc;
  const int a = (unit / b.kc) % b.n_ad;
  const int pj = unit / (b.kc * b.n_ad);
  if (b.A[pj] == nullptr) return;   // projection slot not adapted
  const f16* __restrict__ A = b.A[pj] + (size_t)a * b.r * b.K;
  float* __restrict__ vp = b.vpart + ((size_t)pj * b.kc + c) * b.T * b.r;
  const int kbase = c * b.ci * LORA_KCHUNK + lane * 8;
  const bool resident = b.r <= G && b.ci == 1;   // the wave's whole slice of A fits the register file
  const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  f16x8 areg[G];
  int id = lora_token_id(b.ids, b.bucket_of, b.bucket, lane, b.T);
  if (resident && b.speculate) {
#pragma unroll
    for (int j = 0; j < G; ++j) areg[j] = (j < b.r && kbase < b.K) ? ld8(A + (size_t)j * b.K + kbase) : zero8;
  }
  bool loaded = resident && b.speculate;
  for (int t0 = 0; t0 < b.T; t0 += WAVE) {
    if (t0 > 0) id = lora_token_id(b.ids, b.bucket_of, b.bucket, t0 + lane, b.T);
    unsigned long long mask = __ballot(id == a);
    if (mask && resident && !loaded) {
      loaded = true;
#pragma unroll
      for (int j = 0; j < G; ++j) areg[j] = (j < b.r && kbase < b.K) ? ld8(A + (size_t)j * b.K + kbase) : zero8;
    }
    while (mask) {
      int tt[TB];
#pragma unroll
      for (int u = 0; u < TB; ++u) {
        tt[u] = -1;
        if (mask) {
          tt[u] = t0 + __builtin_ctzll(mask);
          mask &= mask - 1;
        }
      }
      for (int jb = 0; jb < b.r; jb += G) {
        float p[TB][G];
#pragma unroll
        for (int u = 0; u < TB; ++u)
#pragma unroll
          for (int j = 0; j < G; ++j) p[u][j] = 0.f;
        for (int ci = 0; ci < b.ci; ++ci) {
          const int k = kbase + ci * LORA_KCHUNK;
          f16x8 xv[TB];
#pragma unroll
          for (int u = 0; u < TB; ++u) {
            const int t = tt[u] >= 0 ? tt[u] : tt[0];
            xv[u] = k < b.K ? ld8(b.x + (b.frag_tt ? frag_offset(t, k, b.frag_tt) : (size_t)t * b.K + k)) : zero8;
          }
          if (!resident) {
#pragma unroll
            for (int j = 0; j < G; ++j) areg[j] = (jb + j < b.r && k < b.K) ? ld8(A + (size_t)(jb + j) * b.K + k) : zero8;
          }
#pragma unroll
          for (int j = 0; j < G; ++j)
#pragma unroll
            for (int u = 0; u < TB; ++u) p[u][j] = dot8(areg[j], xv[u], p[u][j]);
        }
#pragma unroll
        for (int u = 0; u < TB; ++u) {
          const int j = reduce_transpose<G>(p[u], lane);
          if (tt[u] >= 0 && jb + j < b.r && (lane & (WAVE / G - 1)) == 0) vp[(size_t)tt[u] * b.r + jb + j] = p[u][0];
        }
      }
    }
  }
}

// v[j] = scaling * sum_c v_part[c][t][j] for one token, summed in slice order (the order every consumer uses,
// so fused and stand-alone expands agree bit for bit).
// The slices are requested together and then added one by one: as a loop over kc, every addition waited for its own
// load - up to eight dependent round trips in front of an expand.
__device__ __forceinline__ float lora_v(const float* __restrict__ vpart_proj, int kc, int T, int r, int t, int j, float scaling) {
  float part[LORA_MAX_KC];
#pragma unroll
  for (int c = 0; c < LORA_MAX_KC; ++c) part[c] = c < kc ? vpart_proj[((size_t)c * T + t) * r + j] : 0.f;
  float v = 0.f;
#pragma unroll
  for (int c = 0; c < LORA_MAX_KC; ++c)
    if (c < kc) v += part[c];
  return v * scaling;
}

// Where an expand finds v for (token t, projection slot p, adapter id):
//   kc > 0  : K-slice partials v_part[p][c][t][:]                    (written by the shrink units)
//   kc == 0 : dense shrink results v_all[q][t][(p * n_ad + id) * r + :]  (written by a GEMV over weight rows that have
//             the A tables of all adapters appended; the adapter is picked here, by index).  kq >= 1 blocks q hold
//             the partial sums of kq ranges of K, added here in range order.
struct LoraVSource {
  const float* v;
  int kc, T, n_ad, ld, kq;
};

__device__ __forceinline__ float lora_v_from(const LoraVSource& s, int slot, int id, int r, int t, int j, float scaling) {
  if (s.kc > 0) return lora_v(s.v + (size_t)slot * s.kc * s.T * r, s.kc, s.T, r, t, j, scaling);
  const float* __restrict__ p = s.v + (size_t)t * s.ld + ((size_t)slot * s.n_ad + id) * r + j;
  float part[LORA_MAX_KQ];
#pragma unroll
  for (int q = 0; q < LORA_MAX_KQ; ++q) part[q] = q == 0 || q < s.kq ? p[(size_t)q * s.T * s.ld] : 0.f;   // all blocks requested together
  float a = part[0];
#pragma unroll
  for (int q = 1; q < LORA_MAX_KQ; ++q)
    if (q < s.kq) a += part[q];
  return a * scaling;
}

// The same dot product in two halves, so that a caller can issue the row's loads before the v values are ready:
// lora_row_load fetches up to 8 groups of 8 (r <= 64), lora_row_dot_regs consumes them in lora_row_dot's order.
template <int NGMAX>
__device__ __forceinline__ void lora_row_load(const f16* __restrict__ brow, int r, f16x8 (&bv)[NGMAX]) {
  const int ng = r >> 3;
#pragma unroll
  for (int q = 0; q < NGMAX; ++q) {
    bv[q] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (q < ng) bv[q] = ld8(brow + q * 8);
  }
}

template <int NGMAX>
__device__ __forceinline__ float lora_row_dot_regs(const f16x8 (&bv)[NGMAX], const float* __restrict__ v, int r) {
  float g[8];                           // r <= 8 * NGMAX; groups past NGMAX are empty
  const int ng = r >> 3;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    float s = 0.f;
    if (q < NGMAX) {
      if (q < ng) {
#pragma unroll
        for (int e = 0; e < 8; ++e) s = fmaf((float)bv[q < NGMAX ? q : 0][e], v[q * 8 + e], s);
      }
    }
    g[q] = s;
  }
  if (ng > 4) {
    g[0] = g[0] + g[1]; g[1] = g[2] + g[3]; g[2] = g[4] + g[5]; g[3] = g[6] + g[7];
  }
  if (ng > 2) {
    g[0] = g[0] + g[1]; g[1] = g[2] + g[3];
  }
  if (ng > 1) g[0] = g[0] + g[1];
  return g[0];
}

// delta = B_row[0..r) . v[0..r) with the summation tree of the stand-alone expand kernel: an fma chain over each
// group of 8, then pairwise sums of neighbouring groups.
__device__ __forceinline__ float lora_row_dot(const f16* __restrict__ brow, const float* __restrict__ v, int r) {
  float g[8];
  const int ng = r >> 3;
  for (int q = 0; q < ng; ++q) {
    const f16x8 bv = ld8(brow + q * 8);
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s = fmaf((float)bv[e], v[q * 8 + e], s);
    g[q] = s;
  }
  for (int n = ng; n > 1; n >>= 1)
    for (int q = 0; q < n / 2; ++q) g[q] = g[2 * q] + g[2 * q + 1];
  return g[0];
}
