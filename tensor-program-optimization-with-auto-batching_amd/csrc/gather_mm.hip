// Adapter-indexed LoRA delta (gather-matmul) for gfx950:
//     y[t] += scaling * B[id_t] . (A[id_t] . x[t])
// Two HBM-bound kernels, one wavefront per (adapter, slice):
//   shrink  - a wave owns adapter a and a K-slice; it finds the tokens bound to a by scanning the
//             token->adapter table with ballots, streams its slice of A[a] once into registers
//             (coalesced 1 KiB rows), dots it against each token's x slice (v_dot2_f32_f16) and
//             reduces the r partial sums across lanes with a transposing butterfly, so that r
//             results cost r + log(64/r) shuffles instead of 6 r.
//   expand  - a wave owns adapter a and a block of output rows; it streams its rows of B[a] once
//             into registers, sums the K-slice partials of each token, and read-modify-writes y
//             through a small LDS transpose so every lane touches contiguous y elements.
// The adapter table is never materialised per token: the index lookup happens inside the kernels,
// which is the optimisation of tvm/custom/fuse_take_matmul.py:85-105 kept in hand-written form.
#include <mutex>
#include <type_traits>

#include "gather_mm_batch.h"

namespace {

__global__ __launch_bounds__(64) void lora_shrink_kernel(LoraShrinkBatch b) { lora_shrink_unit(b, blockIdx.x, threadIdx.x); }

template <typename YT, int N>
struct YVec;
template <> struct YVec<f16, 8> { typedef f16x8 type; };
template <> struct YVec<f16, 4> { typedef f16x4 type; };
template <> struct YVec<f16, 2> { typedef f16x2 type; };
template <> struct YVec<float, 4> { typedef f32x4 type; };
template <> struct YVec<float, 2> { typedef f32x2 type; };

// y[0..RPL) += d[0..RPL), converting through fp32; p is RPL-element aligned.
template <typename YT, int RPL>
__device__ __forceinline__ void rmw_add(YT* p, const float* d) {
  if constexpr (RPL == 1) {
    p[0] = (YT)((float)p[0] + d[0]);
  } else if constexpr (sizeof(YT) == 4 && RPL == 8) {
    rmw_add<YT, 4>(p, d);
    rmw_add<YT, 4>(p + 4, d + 4);
  } else {
    typedef typename YVec<YT, RPL>::type V;
    V v = *reinterpret_cast<V*>(p);
#pragma unroll
    for (int q = 0; q < RPL; ++q) v[q] = (YT)((float)v[q] + d[q]);
    *reinterpret_cast<V*>(p) = v;
  }
}

template <int R, typename YT>
__global__ __launch_bounds__(64) void lora_expand_kernel(YT* __restrict__ y, const float* __restrict__ vpart,
                                                         const f16* __restrict__ B,
                                                         const int32_t* __restrict__ ids, float scaling,
                                                         int T, int N, int ldy, int KC,
                                                         const int32_t* __restrict__ bucket_of, int bucket) {
  constexpr int LPR = R / 8;           // lanes sharing one row of B
  constexpr int RPI = WAVE / LPR;      // rows per load instruction
  constexpr int NI = 8;                // load instructions (1 KiB each) per wave
  constexpr int CH = NI * RPI;         // output rows per wave
  constexpr int RPL = CH / WAVE;       // consecutive y elements per lane at write-back
  __shared__ float stage[2][CH];

  const int a = blockIdx.x;
  const int n0 = blockIdx.y * CH;
  const int lane = threadIdx.x;
  const int sub = lane % LPR;
  const int rloc = lane / LPR;

  bool loaded = false;
  float bf[NI][8];
  int parity = 0;

  for (int t0 = 0; t0 < T; t0 += WAVE) {
    const int id = lora_token_id(ids, bucket_of, bucket, t0 + lane, T);
    unsigned long long mask = __ballot(id == a);
    if (mask && !loaded) {
      loaded = true;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int row = n0 + i * RPI + rloc;
        f16x8 b = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (row < N) b = ld8(B + ((size_t)a * N + row) * R + sub * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) bf[i][e] = (float)b[e];
      }
    }
    while (mask) {
      const int t = t0 + __builtin_ctzll(mask);
      mask &= mask - 1;
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = 0.f;
      for (int c = 0; c < KC; ++c) {
        const f32x4* vp = reinterpret_cast<const f32x4*>(vpart + ((size_t)c * T + t) * R + sub * 8);
        const f32x4 lo = vp[0], hi = vp[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] += lo[e];
          v[4 + e] += hi[e];
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= scaling;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s = fmaf(bf[i][e], v[e], s);
#pragma unroll
        for (int o = 1; o < LPR; o <<= 1) s += __shfl_xor(s, o, WAVE);   // neighbouring groups of 8 first
        if (sub == 0) stage[parity][i * RPI + rloc] = s;
      }
      __syncthreads();
      const int n = n0 + lane * RPL;
      if (n < N) {   // N % 8 == 0 and RPL | 8, so a lane's RPL rows are all inside or all outside
        float d[RPL];
#pragma unroll
        for (int q = 0; q < RPL; ++q) d[q] = stage[parity][lane * RPL + q];
        rmw_add<YT, RPL>(y + (size_t)t * ldy + n, d);
      }
      parity ^= 1;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Decode-shaped gather-matmul (T <= 64) in ONE launch.  A workgroup of 8 waves owns (adapter a, slice p of the
// output rows):
//   1. wave c runs the shrink unit of K-slice c of A[a] for the tokens bound to a (found with ballots) and leaves
//      its fp32 partials in LDS - the P workgroups of an adapter repeat this, which costs L2 reads of A[a] but no
//      grid-wide dependency; the workgroup index is laid out so that all slices of an adapter run on the same XCD
//      (index % 8) and share that XCD's L2;
//   2. the partials are summed in slice order and scaled (LDS);
//   3. every thread owns output rows n of the slice: it loads row n of B[a] once and read-modify-writes y[t, n]
//      for each token of the adapter.
// Same arithmetic, in the same order, as lora_shrink_kernel followed by lora_expand_kernel.
// A launch can cover several independent problems (sets of y, x, A, B with a common shape and adapter table):
// blockIdx.y selects the set.
// ---------------------------------------------------------------------------------------------
constexpr int GMM_WAVES = 8;
constexpr int GMM_THREADS = GMM_WAVES * WAVE;

// Adapter tables of several ranks - and of several projections that read the same x - served by ONE launch (MULTI).
// Entry e is one (projection, rank bucket) pair: its tables, rank and scaling, the token bucket it serves, and the
// column range of y it adds to; it holds adapters first[e] .. first[e+1]-1 of the launch's global adapter numbering.
// A token names its bucket and its adapter inside the bucket.  The kernel is instantiated for the largest rank; a
// workgroup (one adapter of one entry) runs with its entry's rank, and the rank entries it does not have enter every
// sum as zeros - which leaves the bits of the single-rank kernel: the reduction trees only gain exact zero terms.
constexpr int GMM_MAX_BUCKETS = 8;
struct GmmBuckets {
  const f16* A[GMM_MAX_BUCKETS];
  const f16* B[GMM_MAX_BUCKETS];
  int r[GMM_MAX_BUCKETS];
  int first[GMM_MAX_BUCKETS + 1];
  float scaling[GMM_MAX_BUCKETS];
  int tok_bucket[GMM_MAX_BUCKETS];   // value of the per-token bucket array this entry serves
  int ycol[GMM_MAX_BUCKETS];         // first column of y and number of columns (rows of B) of the entry's projection
  int ncols[GMM_MAX_BUCKETS];
  int n;
};

// B[n, 0..R) . v[0..R): an fma chain over each group of 8, then pairwise sums of neighbouring groups
// (the order of lora_expand_kernel and lora_row_dot).
template <int R>
__device__ __forceinline__ float row_dot(const f16x8 (&bv)[R / 8], const float* __restrict__ v) {
  constexpr int NG = R / 8;
  float g[NG];
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s = fmaf((float)bv[q][e], v[q * 8 + e], s);
    g[q] = s;
  }
#pragma unroll
  for (int n = NG; n > 1; n >>= 1)
#pragma unroll
    for (int q = 0; q < n / 2; ++q) g[q] = g[2 * q] + g[2 * q + 1];
  return g[0];
}

// GR: rows of A a wave reduces together.  16 reads x once per 16 rows (shortest single problem); 8 keeps the kernel
// under 128 VGPRs, i.e. two workgroups per CU, which is what a launch over many problems wants.  Same result bits.
template <int R, typename YT, int GR, bool MULTI = false>
__global__ __launch_bounds__(GMM_THREADS, (GR == 8 ? 4 : 2)) void gather_mm_decode_kernel(GmmSet one, const GmmSet* __restrict__ sets,
                                                                        const int32_t* __restrict__ ids, float scaling,
                                                                        int T, int K, int N, int n_ad, int ldy,
                                                                        int frag_tt, int P, int ci_n, int kc,
                                                                        const int32_t* __restrict__ bucket_of, int bucket,
                                                                        GmmBuckets mb) {
  constexpr int G = R < GR ? R : GR;         // rows of A reduced together
  constexpr int NG = R / 8;
  extern __shared__ float lds[];             // part [kc][T][R], then v [T][R]
  float* part = lds;
  float* vfin = lds + (size_t)kc * T * R;
  const int wg = blockIdx.x;
  int a = (wg & 7) + 8 * (wg / (8 * P));                // MULTI: numbered over all buckets, n_ad their total
  const int p = (wg >> 3) % P;
  if (a >= n_ad) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  // the problem's pointers and the table row are independent requests: both are in flight before either is awaited
  // (the empty asm keeps the pointer load in this block, ahead of the early exit)
  GmmSet s = sets ? sets[blockIdx.y] : one;
  int ra = R;                                           // rank of this workgroup's adapter
  int ycol = 0;
  if constexpr (MULTI) {
    int b = 0;
#pragma unroll
    for (int i = 1; i < GMM_MAX_BUCKETS; ++i)
      if (i < mb.n && a >= mb.first[i]) b = i;
#pragma unroll
    for (int i = 0; i < GMM_MAX_BUCKETS; ++i)
      if (i == b) {                                     // uniform selects: the struct is never indexed dynamically
        s.A = mb.A[i];
        s.B = mb.B[i];
        ra = mb.r[i];
        scaling = mb.scaling[i];
        a -= mb.first[i];
        bucket = mb.tok_bucket[i];
        ycol = mb.ycol[i];
        N = mb.ncols[i];
      }
    if (s.A == nullptr) return;                         // the bucket's adapters do not target this projection
  }
  const int id = lora_token_id(ids, bucket_of, bucket, lane, T);   // T <= 64: one table row per lane
  asm volatile("" ::"s"(s.A), "s"(s.B), "s"(s.x), "s"(s.y));
  const unsigned long long mine = __ballot(id == a);
  if (!mine) return;                                    // workgroup-uniform
  const f16* __restrict__ A = s.A + (size_t)a * ra * K;
  const f16* __restrict__ B = s.B + (size_t)a * N * ra;
  YT* __restrict__ y = (YT*)s.y + ycol;
  const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};

  // Requests that depend on the adapter table only go out first, ahead of the shrink: the thread's first row(s) of B
  // and the y elements of those rows for the first two tokens of the adapter.
  constexpr int EB = (GR == 8 && R <= 16) ? 4 : 1;      // rows per thread whose loads are in flight together
  const int NS = ((N + P - 1) / P + 7) & ~7;            // rows per slice
  const int n1 = min(N, (p + 1) * NS);
  const int nf = p * NS + threadIdx.x;
  const int ta = __builtin_ctzll(mine);
  const unsigned long long rest1 = mine & (mine - 1);
  const int tb = rest1 ? __builtin_ctzll(rest1) : -1;
  const unsigned long long rest2 = tb >= 0 ? rest1 & (rest1 - 1) : 0ull;   // tokens beyond the first two
  f16x8 bpre[EB][NG];
  float ya[EB], yb[EB];
  auto request = [&](int nbase) {
#pragma unroll
    for (int i = 0; i < EB; ++i) {
      const int n = nbase + i * GMM_THREADS;
      ya[i] = yb[i] = 0.f;
      if (n < n1) {
#pragma unroll
        for (int q = 0; q < NG; ++q) bpre[i][q] = q * 8 < ra ? ld8(B + (size_t)n * ra + q * 8) : zero8;
        ya[i] = (float)y[(size_t)ta * ldy + n];
        if (tb >= 0) yb[i] = (float)y[(size_t)tb * ldy + n];
      }
    }
  };
  request(nf);

  // ---- shrink: wave c owns K-slice c; tokens two at a time; same arithmetic as lora_shrink_unit
  if (wave < kc) {
    const int kbase = wave * ci_n * LORA_KCHUNK + lane * 8;
    float* __restrict__ vp = part + (size_t)wave * T * R;
    if (GR == 16 && ci_n == 1) {
      // the slice is one 512-wide chunk: a group of G rows of A stays in registers over all tokens of the adapter
      // (the single-problem variant; the many-problem variant has no registers to spare for it)
      const bool in = kbase < K;
#pragma unroll
      for (int jb = 0; jb < R; jb += G) {
        if (jb >= ra) break;                              // uniform; the rank entries beyond ra are zeroed below
        f16x8 areg[G];
#pragma unroll
        for (int j = 0; j < G; ++j) areg[j] = (in && jb + j < ra) ? ld8(A + (size_t)(jb + j) * K + kbase) : zero8;
        unsigned long long m = mine;
        while (m) {
          const int t0 = __builtin_ctzll(m);
          m &= m - 1;
          int t1 = -1;
          if (m) {
            t1 = __builtin_ctzll(m);
            m &= m - 1;
          }
          const int t1x = t1 >= 0 ? t1 : t0;
          const f16x8 x0 = in ? ld8(s.x + (frag_tt ? frag_offset(t0, kbase, frag_tt) : (size_t)t0 * K + kbase)) : zero8;
          const f16x8 x1 = in ? ld8(s.x + (frag_tt ? frag_offset(t1x, kbase, frag_tt) : (size_t)t1x * K + kbase)) : zero8;
          float acc0[G], acc1[G];
#pragma unroll
          for (int j = 0; j < G; ++j) {
            acc0[j] = dot8(areg[j], x0, 0.f);
            acc1[j] = dot8(areg[j], x1, 0.f);
          }
          const int j0 = reduce_transpose<G>(acc0, lane);
          if ((lane & (WAVE / G - 1)) == 0) vp[(size_t)t0 * R + jb + j0] = acc0[0];
          const int j1 = reduce_transpose<G>(acc1, lane);
          if (t1 >= 0 && (lane & (WAVE / G - 1)) == 0) vp[(size_t)t1 * R + jb + j1] = acc1[0];
        }
      }
    } else {
      unsigned long long m = mine;
      while (m) {
        int tt[2];
        tt[0] = __builtin_ctzll(m);
        m &= m - 1;
        tt[1] = -1;
        if (m) {
          tt[1] = __builtin_ctzll(m);
          m &= m - 1;
        }
        const int t1 = tt[1] >= 0 ? tt[1] : tt[0];
#pragma unroll
        for (int jb = 0; jb < R; jb += G) {
          if (jb >= ra) break;                            // uniform
          float acc0[G], acc1[G];
#pragma unroll
          for (int j = 0; j < G; ++j) acc0[j] = acc1[j] = 0.f;
          for (int ci = 0; ci < ci_n; ++ci) {
            const int k = kbase + ci * LORA_KCHUNK;
            const bool in = k < K;
            const f16x8 x0 = in ? ld8(s.x + (frag_tt ? frag_offset(tt[0], k, frag_tt) : (size_t)tt[0] * K + k)) : zero8;
            const f16x8 x1 = in ? ld8(s.x + (frag_tt ? frag_offset(t1, k, frag_tt) : (size_t)t1 * K + k)) : zero8;
            f16x8 areg[G];
#pragma unroll
            for (int j = 0; j < G; ++j) areg[j] = (in && jb + j < ra) ? ld8(A + (size_t)(jb + j) * K + k) : zero8;
#pragma unroll
            for (int j = 0; j < G; ++j) {
              acc0[j] = dot8(areg[j], x0, acc0[j]);
              acc1[j] = dot8(areg[j], x1, acc1[j]);
            }
          }
          const int j0 = reduce_transpose<G>(acc0, lane);
          if ((lane & (WAVE / G - 1)) == 0) vp[(size_t)tt[0] * R + jb + j0] = acc0[0];
          const int j1 = reduce_transpose<G>(acc1, lane);
          if (tt[1] >= 0 && (lane & (WAVE / G - 1)) == 0) vp[(size_t)tt[1] * R + jb + j1] = acc1[0];
        }
      }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < T * R; e += GMM_THREADS) {
    const int t = e / R, j = e % R;
    if ((mine >> t) & 1) vfin[e] = j < ra ? lora_v(part, kc, T, R, t, j, scaling) : 0.f;
  }
  __syncthreads();

  // ---- expand: the thread's rows of the slice, every token of the adapter
  if constexpr (EB > 1) {
    // EB rows per pass; the next pass's loads are requested before this pass's remaining tokens are worked off
    for (int nbase = nf; nbase < n1; nbase += EB * GMM_THREADS) {
      f16x8 bcur[EB][NG];
#pragma unroll
      for (int i = 0; i < EB; ++i) {
        const int n = nbase + i * GMM_THREADS;
        if (n < n1) {
#pragma unroll
          for (int q = 0; q < NG; ++q) bcur[i][q] = bpre[i][q];
          y[(size_t)ta * ldy + n] = (YT)(ya[i] + row_dot<R>(bcur[i], vfin + ta * R));
          if (tb >= 0) y[(size_t)tb * ldy + n] = (YT)(yb[i] + row_dot<R>(bcur[i], vfin + tb * R));
        }
      }
      if (nbase + EB * GMM_THREADS < n1) request(nbase + EB * GMM_THREADS);
      if (rest2) {
#pragma unroll
        for (int i = 0; i < EB; ++i) {
          const int n = nbase + i * GMM_THREADS;
          if (n < n1) {
            unsigned long long m = rest2;
            while (m) {
              const int t = __builtin_ctzll(m);
              m &= m - 1;
              YT* yp = y + (size_t)t * ldy + n;
              *yp = (YT)((float)*yp + row_dot<R>(bcur[i], vfin + t * R));
            }
          }
        }
      }
    }
  } else {
    if (nf < n1) {
      y[(size_t)ta * ldy + nf] = (YT)(ya[0] + row_dot<R>(bpre[0], vfin + ta * R));
      if (tb >= 0) y[(size_t)tb * ldy + nf] = (YT)(yb[0] + row_dot<R>(bpre[0], vfin + tb * R));
      unsigned long long m = rest2;
      while (m) {
        const int t = __builtin_ctzll(m);
        m &= m - 1;
        YT* yp = y + (size_t)t * ldy + nf;
        *yp = (YT)((float)*yp + row_dot<R>(bpre[0], vfin + t * R));
      }
    }
    for (int n = nf + GMM_THREADS; n < n1; n += GMM_THREADS) {
      f16x8 bv[NG];
#pragma unroll
      for (int q = 0; q < NG; ++q) bv[q] = q * 8 < ra ? ld8(B + (size_t)n * ra + q * 8) : zero8;
      unsigned long long m = mine;
      while (m) {
        const int t = __builtin_ctzll(m);
        m &= m - 1;
        YT* yp = y + (size_t)t * ldy + n;
        *yp = (YT)((float)*yp + row_dot<R>(bv, vfin + t * R));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Prefill-sized gather-matmul (T > 64) on the matrix cores.  Tokens arrive grouped in adapter segments, so a tile
// of 16 consecutive tokens holds one adapter, two at a segment boundary; a tile is processed once per distinct
// adapter in it and rows of other adapters are masked at the store.
//   shrink: workgroup per token tile, 4 waves split K;  V^T[r, 16 tok] = A[a] . X^T  with A[a] as the A operand
//           (rows = rank index) and the token tile as the B operand, so a lane ends up with 4 consecutive rank
//           entries of one token (one 16-byte store of v[t, 4g..4g+3]); fixed-order LDS sum of the 4 waves.
//   expand: wave per (token tile, 64 output columns);  D[n, tok] = B[a] . V^T with v split into fp16 hi + lo halves
//           (two MFMAs, ~22 mantissa bits of v); a lane read-modify-writes 4 consecutive y elements of one token.
// v is [T, r] fp32 (one full sum per token, no K-slices).
// ---------------------------------------------------------------------------------------------
constexpr int SEG_WAVES = 4;

// Projections that share x, the token table, the rank and the scaling (q, k, v; gate, up): blockIdx.z selects one.
// Projection z keeps its shrink results in slice z of the workspace.
constexpr int SEG_MAX_PROJ = 3;
struct SegProjs {
  const f16* A[SEG_MAX_PROJ];
  const f16* B[SEG_MAX_PROJ];
  void* y[SEG_MAX_PROJ];
  int N[SEG_MAX_PROJ];
  int n;
};

// The distinct adapters of a 16-token tile (lanes 0..15 hold the tokens' ids, -1 = none) and, per adapter, the mask of
// tile rows bound to it.  Everything is wave-uniform and lives in scalar registers; the loops over the list are fully
// unrolled with a uniform `i < n` guard, so the list is never indexed dynamically.
struct TileAdapters {
  int a[16];
  unsigned rows[16];
  int n;
  unsigned all;     // rows with any adapter
};

__device__ __forceinline__ TileAdapters tile_adapters(int id) {
  TileAdapters ta;
  unsigned todo = (unsigned)__ballot(id >= 0) & 0xffffu;
  ta.all = todo;
  ta.n = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    ta.a[i] = -1;
    ta.rows[i] = 0u;
    if (todo) {
      const int first = __builtin_ctz(todo);
      const int a = __builtin_amdgcn_readfirstlane(__shfl(id, first, WAVE));
      const unsigned rows = (unsigned)__ballot(id == a) & 0xffffu & todo;
      todo &= ~rows;
      ta.a[i] = a;
      ta.rows[i] = rows;
      ta.n = i + 1;
    }
  }
  return ta;
}

// Shrink.  The adapters of the tile are worked GA at a time inside ONE pass over K: per 32-k step the token fragment is
// loaded once and every adapter of the group contributes one A fragment and one MFMA - a decode batch, where a tile of
// 16 tokens holds up to 16 adapters, costs one K loop instead of 16, with all the groups' loads in flight together.
// Shrink of one 16-token tile by the four waves of a workgroup: K steps kb0 .. kb1-1 dealt to the waves in turn, the
// waves' sums added in wave order through `red`, partial result rows written to v [T][R].
// Where lane (token t, k-group g) finds its 8 k-entries of 32-k step 0, and the distance between consecutive steps:
// row-major x [T, K] (frag_tt == 0) or fragment order with frag_tt sixteen-token tiles per 32-k step.
__device__ __forceinline__ const f16* x_operand(const f16* __restrict__ x, int t, int g, int K, int frag_tt, int& step) {
  if (frag_tt) {
    step = frag_tt * 512;
    return x + (size_t)(t >> 4) * 512 + g * 128 + (t & 15) * 8;
  }
  step = 32;
  return x + (size_t)t * K + g * 8;
}

// sum over the K ranges of a shrink's partial results, four rank entries at a time, in range order; the ranges are
// requested together (a loop with a load and an addition per turn waits out a round trip per range)
__device__ __forceinline__ f32x4 sum_ranges(const float* __restrict__ p, int splits, size_t stride) {
  f32x4 part[LORA_MAX_KC];
#pragma unroll
  for (int sp = 0; sp < LORA_MAX_KC; ++sp) part[sp] = sp < splits ? *reinterpret_cast<const f32x4*>(p + sp * stride) : f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 sum = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int sp = 0; sp < LORA_MAX_KC; ++sp)
    if (sp < splits) sum += part[sp];
  return sum;
}

template <int R>
__device__ __forceinline__ void shrink_tile_mfma(float* __restrict__ v, const f16* __restrict__ x, int frag_tt, const f16* __restrict__ A,
                                                 const int32_t* __restrict__ ids, int T, int K, int n_ad,
                                                 const int32_t* __restrict__ bucket_of, int bucket, int t0, int kb0, int kb1,
                                                 f32x4 (*red)[8][WAVE], int only_group = -1) {
  constexpr int NT = (R + 15) / 16;     // 16-row tiles of A[a]; rank 8 uses half a tile
  constexpr int GA = 8 / NT;            // adapters per pass: 32 accumulator registers
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const int tl = min(t0 + col, T - 1);                          // token whose x row this lane supplies
  const int raw = lora_token_id(ids, bucket_of, bucket, t0 + col, T);
  const int id = (raw >= 0 && raw < n_ad) ? raw : -1;
  const TileAdapters ta = tile_adapters(id);
  int xstep;
  const f16* __restrict__ xr = x_operand(x, tl, g, K, frag_tt, xstep);
#pragma unroll
  for (int g0 = 0; g0 < 16; g0 += GA) {
    if (g0 < ta.n && (only_group < 0 || g0 == only_group * GA)) {   // uniform
      f32x4 acc[GA][NT];
#pragma unroll
      for (int u = 0; u < GA; ++u)
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[u][i] = f32x4{0.f, 0.f, 0.f, 0.f};
      // two register sets: the k-step after this one is requested before this one is multiplied
      f16x8 xf[2], af[2][GA][NT];
      auto load = [&](int s, int kb) {
        const int kk = kb < kb1 ? kb : kb1 - 1;                  // past the range: a valid address, the data is not multiplied
        xf[s] = ld8(xr + (size_t)kk * xstep);
#pragma unroll
        for (int u = 0; u < GA; ++u) {
          if (g0 + u < ta.n) {
            const f16* __restrict__ Aa = A + (size_t)ta.a[g0 + u] * R * K + g * 8;
#pragma unroll
            for (int i = 0; i < NT; ++i) {
              const int row = i * 16 + col;
              af[s][u][i] = row < R ? ld8(Aa + (size_t)row * K + kk * 32) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            }
          }
        }
      };
      auto multiply = [&](int s) {
#pragma unroll
        for (int u = 0; u < GA; ++u) {
          if (g0 + u < ta.n) {
#pragma unroll
            for (int i = 0; i < NT; ++i)
              acc[u][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[s][u][i], xf[s], acc[u][i], 0, 0, 0);   // rows: rank index, cols: tokens
          }
        }
      };
      int kb = kb0 + wave;
      if (kb < kb1) load(0, kb);
      for (; kb < kb1; kb += 2 * SEG_WAVES) {
        load(1, kb + SEG_WAVES);
        multiply(0);
        if (kb + SEG_WAVES < kb1) {
          load(0, kb + 2 * SEG_WAVES);
          multiply(1);
        }
      }
#pragma unroll
      for (int u = 0; u < GA; ++u)
#pragma unroll
        for (int i = 0; i < NT; ++i) red[wave][u * NT + i][lane] = acc[u][i];
      __syncthreads();
      // wave w sums and stores the adapters u = w, w + 4, ... of the group (fixed order over the four K parts)
#pragma unroll
      for (int u = 0; u < GA; ++u) {
        if (g0 + u < ta.n && (u % SEG_WAVES) == wave) {
#pragma unroll
          for (int i = 0; i < NT; ++i) {
            f32x4 sum = red[0][u * NT + i][lane];
#pragma unroll
            for (int w = 1; w < SEG_WAVES; ++w) sum += red[w][u * NT + i][lane];
            const int j = i * 16 + 4 * g;                          // first of this lane's 4 rank entries
            if (((ta.rows[g0 + u] >> col) & 1u) && j < R) *reinterpret_cast<f32x4*>(v + (size_t)(t0 + col) * R + j) = sum;
          }
        }
      }
      __syncthreads();
    }
  }
}

template <int R>
__global__ __launch_bounds__(SEG_WAVES * WAVE) void lora_shrink_mfma_kernel(float* __restrict__ v, const f16* __restrict__ x, int frag_tt,
                                                                            SegProjs pj,
                                                                            const int32_t* __restrict__ ids, int T, int K,
                                                                            int n_ad, const int32_t* __restrict__ bucket_of,
                                                                            int bucket) {
  // blockIdx.y selects one of gridDim.y contiguous ranges of 32-k steps; its partial sums go to v[blockIdx.y][T][R].
  // blockIdx.z = projection * NG + group: the tile's adapters are taken in the order of their first token, GA to a group,
  // and every group has a workgroup of its own (a tile of a decode batch holds up to 16 adapters: their passes over K
  // run side by side instead of one after the other; a workgroup whose group is empty leaves at once).
  constexpr int NG = 16 / (8 / ((R + 15) / 16));
  __shared__ f32x4 red[SEG_WAVES][8][WAVE];
  const int proj = blockIdx.z / NG, group = blockIdx.z % NG;
  const f16* __restrict__ A = pj.A[0];
#pragma unroll
  for (int i = 1; i < SEG_MAX_PROJ; ++i)
    if (i == proj) A = pj.A[i];                          // uniform select: the struct is never indexed dynamically
  const int KB = K / 32;
  const int per = (KB + gridDim.y - 1) / gridDim.y;
  const int kb0 = blockIdx.y * per, kb1 = min(KB, kb0 + per);
  v += ((size_t)proj * gridDim.y + blockIdx.y) * T * R;
  shrink_tile_mfma<R>(v, x, frag_tt, A, ids, T, K, n_ad, bucket_of, bucket, blockIdx.x * 16, kb0, kb1, red, group);
}

// Prefill-sized shrink: FOUR token tiles per workgroup.  When all adapted tokens of the four tiles use one adapter (an
// adapter segment of 64 tokens or more), an A fragment is loaded once per 64 tokens instead of once per 16; otherwise
// the tiles are worked off one after the other as above.  Same sums, in the same order, either way.
template <int R>
__global__ __launch_bounds__(SEG_WAVES * WAVE, 2) void lora_shrink_quad_mfma_kernel(float* __restrict__ v, const f16* __restrict__ x, int frag_tt,
                                                                                   SegProjs pj,
                                                                                   const int32_t* __restrict__ ids, int T, int K,
                                                                                   int n_ad, const int32_t* __restrict__ bucket_of,
                                                                                   int bucket) {
  constexpr int NT = (R + 15) / 16;
  constexpr int QT = 4;
  __shared__ f32x4 red[SEG_WAVES][8][WAVE];
  const f16* __restrict__ A = pj.A[0];
#pragma unroll
  for (int i = 1; i < SEG_MAX_PROJ; ++i)
    if (i == blockIdx.z) A = pj.A[i];                    // uniform select: the struct is never indexed dynamically
  const int KB = K / 32;
  const int per = (KB + gridDim.y - 1) / gridDim.y;
  const int kb0 = blockIdx.y * per, kb1 = min(KB, kb0 + per);
  v += ((size_t)blockIdx.z * gridDim.y + blockIdx.y) * T * R;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const int tq = blockIdx.x * 16 * QT;
  // lane l looks at token tq + l: do all adapted tokens of the four tiles name the same adapter?
  const int raw = lora_token_id(ids, bucket_of, bucket, tq + lane, T);
  const int idl = (raw >= 0 && raw < n_ad) ? raw : -1;
  const unsigned long long have = __ballot(idl >= 0);
  if (!have) return;                                     // the same for every wave
  const int a = __shfl(idl, __builtin_ctzll(have), WAVE);
  const bool same = __ballot(idl == a) == have;
  if (!same) {
    for (int u = 0; u < QT; ++u)
      if (tq + u * 16 < T) shrink_tile_mfma<R>(v, x, frag_tt, A, ids, T, K, n_ad, bucket_of, bucket, tq + u * 16, kb0, kb1, red);
    return;
  }
  const f16* __restrict__ Aa = A + (size_t)a * R * K + g * 8;
  const f16* xr[QT];
  int xstep = 32;
#pragma unroll
  for (int u = 0; u < QT; ++u) xr[u] = x_operand(x, min(tq + u * 16 + col, T - 1), g, K, frag_tt, xstep);
  f32x4 acc[QT][NT];
#pragma unroll
  for (int u = 0; u < QT; ++u)
#pragma unroll
    for (int i = 0; i < NT; ++i) acc[u][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  // two register sets: the k-step after this one is requested before this one is multiplied
  f16x8 af[2][NT], xf[2][QT];
  auto load = [&](int s, int kb) {
    const int kk = kb < kb1 ? kb : kb1 - 1;      // past the range: a valid address, the data is not multiplied
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int row = i * 16 + col;
      af[s][i] = row < R ? ld8(Aa + (size_t)row * K + kk * 32) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < QT; ++u) xf[s][u] = ld8(xr[u] + (size_t)kk * xstep);
  };
  auto multiply = [&](int s) {
#pragma unroll
    for (int u = 0; u < QT; ++u)
#pragma unroll
      for (int i = 0; i < NT; ++i) acc[u][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[s][i], xf[s][u], acc[u][i], 0, 0, 0);
  };
  int kb = kb0 + wave;
  if (kb < kb1) load(0, kb);
  for (; kb < kb1; kb += 2 * SEG_WAVES) {
    load(1, kb + SEG_WAVES);
    multiply(0);
    if (kb + SEG_WAVES < kb1) {
      load(0, kb + 2 * SEG_WAVES);
      multiply(1);
    }
  }
  // the four waves' sums, tile by tile, added in wave order; wave w stores A-tile i = w, w + 4, ... of the token tile
#pragma unroll
  for (int u = 0; u < QT; ++u) {
#pragma unroll
    for (int i = 0; i < NT; ++i) red[wave][i][lane] = acc[u][i];
    __syncthreads();
    const unsigned rows = (unsigned)(have >> (16 * u)) & 0xffffu;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      if ((i % SEG_WAVES) == wave) {
        f32x4 sum = red[0][i][lane];
#pragma unroll
        for (int w = 1; w < SEG_WAVES; ++w) sum += red[w][i][lane];
        const int j = i * 16 + 4 * g;
        if (((rows >> col) & 1u) && j < R) *reinterpret_cast<f32x4*>(v + (size_t)(tq + u * 16 + col) * R + j) = sum;
      }
    }
    __syncthreads();
  }
}

// adapter of the first unprocessed token of the tile and the mask of tile rows bound to it; lanes 0..15 hold ids
__device__ __forceinline__ bool next_tile_adapter(int id, unsigned& todo, int& a, unsigned& rows) {
  if (!todo) return false;
  const int first = __builtin_ctz(todo);
  a = __shfl(id, first, WAVE);
  rows = (unsigned)__ballot(id == a) & 0xffffu & todo;
  todo &= ~rows;
  return true;
}

// Expand for segment-ordered tokens (prefill): TWO token tiles per workgroup and 256 registers per lane (two workgroups
// per CU, which is what a prefill-sized launch fills the chip with anyway).  In the common case - both tiles belong to
// one adapter segment - a B fragment serves 32 tokens, the next column block's fragments are requested a block ahead
// and the y rows at the top of the block, so a block costs one memory round.  Tiles that hold several adapters, or
// different ones, are worked off one tile and one adapter at a time (one pass per distinct adapter of the tile, rows of
// other adapters masked at the store).
template <int R, typename YT>
__global__ __launch_bounds__(SEG_WAVES * WAVE, 2) void lora_expand_pair_mfma_kernel(SegProjs pj, const float* __restrict__ v,
                                                                                   const int32_t* __restrict__ ids, float scaling,
                                                                                   int T, int ldy, int n_ad,
                                                                                   const int32_t* __restrict__ bucket_of, int bucket,
                                                                                   int splits, int nit) {
  YT* __restrict__ y = (YT*)pj.y[0];
  const f16* __restrict__ B = pj.B[0];
  int N = pj.N[0];
#pragma unroll
  for (int i = 1; i < SEG_MAX_PROJ; ++i)
    if (i == blockIdx.z) {                               // uniform select: the struct is never indexed dynamically
      y = (YT*)pj.y[i];
      B = pj.B[i];
      N = pj.N[i];
    }
  v += (size_t)blockIdx.z * splits * T * R;
  constexpr int KS = (R + 31) / 32;     // k-steps of 32 rank entries (ranks 8 and 16: one partly filled step)
  constexpr int CT = 4;                 // 16-column tiles per wave
  constexpr int LD = 16 * CT + 4;       // padded row of the transposition buffer (floats): conflict-free both ways
  typedef typename YVec<YT, sizeof(YT) == 2 ? 8 : 4>::type YV;      // 16 bytes of y
  constexpr int NYV = sizeof(YT) == 2 ? 2 : 4;                       // ... of which a lane's 16 columns take 2 or 4
  constexpr int EPV = 16 / NYV;
  __shared__ float stage[2][SEG_WAVES][16][LD];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nbase = blockIdx.y * nit * SEG_WAVES * 16 * CT + wave * 16 * CT;
  const int col = lane & 15, g = lane >> 4;
  const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  int t0[2], id[2];
  unsigned todo[2];
  f16x8 vh[2][KS], vl[2][KS];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    t0[u] = (blockIdx.x * 2 + u) * 16;
    const int raw = lora_token_id(ids, bucket_of, bucket, t0[u] + col, T);
    id[u] = (raw >= 0 && raw < n_ad) ? raw : -1;
    todo[u] = (unsigned)__ballot(id[u] >= 0) & 0xffffu;
  }
  // v of the two token tiles, once per workgroup: thread e sums four rank entries of one token over the K-range
  // partials of the shrink (in range order), scales them and leaves them in LDS; rows of unadapted tokens are never
  // read (their v holds nothing) and enter the products as zeros
  float* __restrict__ vs = &stage[0][0][0][0];           // [2][16][R] floats, before the buffer serves the transposition
  static_assert(2 * 16 * R <= 2 * SEG_WAVES * 16 * LD, "v of two token tiles fits the transposition buffer");
  for (int e = threadIdx.x; e < 2 * 16 * (R / 4); e += SEG_WAVES * WAVE) {
    const int u = e / (16 * (R / 4)), tok = (e / (R / 4)) % 16, j = (e % (R / 4)) * 4;
    f32x4 sum = f32x4{0.f, 0.f, 0.f, 0.f};
    if ((todo[u] >> tok) & 1u) {
      const int t = t0[u] + tok;
      sum = sum_ranges(v + (size_t)t * R + j, splits, (size_t)T * R);
#pragma unroll
      for (int q = 0; q < 4; ++q) sum[q] *= scaling;
    }
    *reinterpret_cast<f32x4*>(vs + ((size_t)u * 16 + tok) * R + j) = sum;
  }
  __syncthreads();
  // the token tiles of v as the B operand, hi and lo halves: lane holds v[token col][ks*32 + 8g .. +7]
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int j = ks * 32 + g * 8;
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = 0.f;
      if (j < R) {
        const f32x4 lo = *reinterpret_cast<const f32x4*>(vs + ((size_t)u * 16 + col) * R + j);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(vs + ((size_t)u * 16 + col) * R + j + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          f[e] = lo[e];
          f[4 + e] = hi[e];
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const f16 h = (f16)f[e];
        vh[u][ks][e] = h;
        vl[u][ks][e] = (f16)(f[e] - (float)h);
      }
    }
  __syncthreads();                                       // vs is dead: the buffer goes back to the transposition
  if (!(todo[0] | todo[1])) return;     // the same for every wave of the workgroup
  // write-back role of the lane: token lane / 4, the 16 columns of column tile lane % 4 (contiguous in y)
  const int wt = lane >> 2, wc = lane & 3;
  // the B fragments of column block `it` of adapter a
  auto load_b = [&](f16x8 (&bf)[CT][KS], const f16* __restrict__ Ba, int it) {
    const int n0 = nbase + it * SEG_WAVES * 16 * CT;
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int nb = n0 + c * 16;
        bf[c][ks] = (nb < N && ks * 32 + g * 8 < R) ? ld8(Ba + (size_t)(nb + col) * R + ks * 32) : zero8;
      }
  };
  // products of tile u with the fragments bf, into the tile's transposition buffer
  auto products = [&](int u, const f16x8 (&bf)[CT][KS], int it) {
    const int n0 = nbase + it * SEG_WAVES * 16 * CT;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      if (n0 + c * 16 < N) {                                          // wave-uniform
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[c][ks], vh[u][ks], acc, 0, 0, 0);    // rows: output column, cols: tokens
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[c][ks], vl[u][ks], acc, 0, 0, 0);
        }
        *reinterpret_cast<f32x4*>(&stage[u][wave][col][c * 16 + 4 * g]) = acc;           // D[n = 4g.., token col]
      }
    }
  };
  // y rows of tile u (already loaded into yv) plus the tile's products, stored
  auto add_store = [&](int u, YV (&yv)[NYV], YT* __restrict__ yrow) {
#pragma unroll
    for (int q = 0; q < NYV; ++q) {
#pragma unroll
      for (int e4 = 0; e4 < EPV / 4; ++e4) {
        const f32x4 s4 = *reinterpret_cast<const f32x4*>(&stage[u][wave][wt][wc * 16 + q * EPV + 4 * e4]);
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[q][4 * e4 + e] = (YT)((float)yv[q][4 * e4 + e] + s4[e]);
      }
      *reinterpret_cast<YV*>(yrow + q * EPV) = yv[q];
    }
  };
  // one adapter for every adapted row of both tiles?
  const int a_first = todo[0] ? __shfl(id[0], __builtin_ctz(todo[0] | 0x10000u) & 15, WAVE) : __shfl(id[1], __builtin_ctz(todo[1] | 0x10000u) & 15, WAVE);
  const bool same = (((unsigned)__ballot(id[0] == a_first) & 0xffffu) == todo[0]) && (((unsigned)__ballot(id[1] == a_first) & 0xffffu) == todo[1]);
  if (same) {
    const f16* __restrict__ Ba = B + (size_t)a_first * N * R + g * 8;
    auto block = [&](int it, f16x8 (&cur)[CT][KS], f16x8 (&nxt)[CT][KS]) {
      const int nw = nbase + it * SEG_WAVES * 16 * CT + wc * 16;
      YV yv[2][NYV];
      bool wr[2];
      YT* yrow[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        yrow[u] = y + (size_t)(t0[u] + wt) * ldy + nw;
        wr[u] = nw < N && ((todo[u] >> wt) & 1u);
        if (wr[u]) {
#pragma unroll
          for (int q = 0; q < NYV; ++q) yv[u][q] = *reinterpret_cast<const YV*>(yrow[u] + q * EPV);
        }
      }
      if (it + 1 < nit) load_b(nxt, Ba, it + 1);
      if (todo[0]) products(0, cur, it);
      if (todo[1]) products(1, cur, it);
      __syncthreads();
#pragma unroll
      for (int u = 0; u < 2; ++u)
        if (wr[u]) add_store(u, yv[u], yrow[u]);
      __syncthreads();
    };
    f16x8 b0[CT][KS], b1[CT][KS];
    load_b(b0, Ba, 0);
    for (int it = 0; it < nit; it += 2) {
      block(it, b0, b1);
      if (it + 1 < nit) block(it + 1, b1, b0);
    }
    return;
  }
  // general case: tile by tile, adapter by adapter
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    int a;
    unsigned rows;
    unsigned left = todo[u];
    while (next_tile_adapter(id[u], left, a, rows)) {
      const f16* __restrict__ Ba = B + (size_t)a * N * R + g * 8;
      for (int it = 0; it < nit; ++it) {
        const int nw = nbase + it * SEG_WAVES * 16 * CT + wc * 16;
        YT* __restrict__ yrow = y + (size_t)(t0[u] + wt) * ldy + nw;
        const bool wr = nw < N && ((rows >> wt) & 1u);
        f16x8 bf[CT][KS];
        load_b(bf, Ba, it);
        YV yv[NYV];
        if (wr) {
#pragma unroll
          for (int q = 0; q < NYV; ++q) yv[q] = *reinterpret_cast<const YV*>(yrow + q * EPV);
        }
        products(u, bf, it);
        __syncthreads();
        if (wr) add_store(u, yv, yrow);
        __syncthreads();
      }
    }
  }
}

// Expand for token tiles that mix many adapters (decode batches).  Per block of 16 output columns every adapter of the tile contributes B[a] . v^T (two MFMAs: hi and lo half of
// v); a token's column of the result is taken from the product of its own adapter, so all adapters are worked off before
// the one read-modify-write of y.  The B fragments of up to GB adapters are requested together.
template <int R, typename YT>
__global__ __launch_bounds__(SEG_WAVES * WAVE) void lora_expand_mixed_mfma_kernel(SegProjs pj, const float* __restrict__ v,
                                                                            const int32_t* __restrict__ ids, float scaling,
                                                                            int T, int ldy, int n_ad,
                                                                            const int32_t* __restrict__ bucket_of, int bucket,
                                                                            int splits, int nit) {
  YT* __restrict__ y = (YT*)pj.y[0];
  const f16* __restrict__ B = pj.B[0];
  int N = pj.N[0];
#pragma unroll
  for (int i = 1; i < SEG_MAX_PROJ; ++i)
    if (i == blockIdx.z) {                               // uniform select: the struct is never indexed dynamically
      y = (YT*)pj.y[i];
      B = pj.B[i];
      N = pj.N[i];
    }
  v += (size_t)blockIdx.z * splits * T * R;
  constexpr int KS = (R + 31) / 32;     // k-steps of 32 rank entries (ranks 8 and 16: one partly filled step)
  constexpr int GB = 16 / KS;           // adapters whose fragments are in flight together: 64 registers
  constexpr int CT = 4;                 // 16-column tiles per wave
  constexpr int LD = 16 * CT + 4;       // padded row of the transposition buffer (floats): conflict-free both ways
  __shared__ float stage[SEG_WAVES][16][LD];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t0 = blockIdx.x * 16;
  // a workgroup covers nit consecutive blocks of 4 waves x 64 columns; the token tile of v stays in registers
  const int nbase = blockIdx.y * nit * SEG_WAVES * 16 * CT + wave * 16 * CT;
  const int col = lane & 15, g = lane >> 4;
  const int tl = min(t0 + col, T - 1);
  const int raw = lora_token_id(ids, bucket_of, bucket, t0 + col, T);
  const int id = (raw >= 0 && raw < n_ad) ? raw : -1;
  const unsigned all = (unsigned)__ballot(id >= 0) & 0xffffu;    // tile rows with an adapter
  if (!all) return;                     // the same for every wave of the workgroup
  const int a_first = __builtin_amdgcn_readfirstlane(__shfl(id, __builtin_ctz(all), WAVE));
  const bool one_adapter = ((unsigned)__ballot(id == a_first) & 0xffffu) == all;
  const TileAdapters ta = tile_adapters(id);                     // the tile's distinct adapters and their rows, found once
  // the token tile of v as the B operand, hi and lo halves: lane holds v[token col][ks*32 + 8g .. +7]
  f16x8 vh[KS], vl[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int j = ks * 32 + g * 8;
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = 0.f;
    // rows of unadapted tokens are never read (their v holds nothing) and enter the product as zeros
    if (j < R && id >= 0) {
      // the K-range partials of the shrink, summed in range order
      const f32x4 lo = sum_ranges(v + (size_t)tl * R + j, splits, (size_t)T * R);
      const f32x4 hi = sum_ranges(v + (size_t)tl * R + j + 4, splits, (size_t)T * R);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f[e] = lo[e] * scaling;
        f[4 + e] = hi[e] * scaling;
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const f16 h = (f16)f[e];
      vh[ks][e] = h;
      vl[ks][e] = (f16)(f[e] - (float)h);
    }
  }
  // write-back role of the lane: token lane / 4, the 16 columns of column tile lane % 4 (contiguous in y)
  const int wt = lane >> 2, wc = lane & 3;
  // SINGLE: the tile holds one adapter (a prefill segment) - the products accumulate directly, no per-token selection
  auto run = [&](auto single) {
    constexpr bool SINGLE = decltype(single)::value;
    for (int it = 0; it < nit; ++it) {
      const int n0 = nbase + it * SEG_WAVES * 16 * CT;
      const int nw = n0 + wc * 16;
      YT* __restrict__ yrow = y + (size_t)(t0 + wt) * ldy + nw;
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const int nb = n0 + c * 16;
        if (nb < N) {                                                // wave-uniform
          f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};                     // D[n = nb + 4g.., token col] of the token's own adapter
          if constexpr (SINGLE) {
            const f16* __restrict__ Ba = B + (size_t)a_first * N * R + g * 8;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
              const int j = ks * 32 + g * 8;
              const f16x8 bf = j < R ? ld8(Ba + (size_t)(nb + col) * R + ks * 32) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
              acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf, vh[ks], acc, 0, 0, 0);    // rows: output column, cols: tokens
              acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf, vl[ks], acc, 0, 0, 0);
            }
          } else {
            // the tile's adapters GB at a time (ranks up to 32: all sixteen at once): their B fragments are requested
            // together, then every adapter's product goes to the tokens bound to it
#pragma unroll
            for (int g0 = 0; g0 < 16; g0 += GB) {
              if (g0 < ta.n) {                                         // uniform
                f16x8 bf[GB][KS];
#pragma unroll
                for (int u = 0; u < GB; ++u) {
                  if (g0 + u < ta.n) {
                    const f16* __restrict__ Ba = B + (size_t)ta.a[g0 + u] * N * R + g * 8;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                      bf[u][ks] = (ks * 32 + g * 8) < R ? ld8(Ba + (size_t)(nb + col) * R + ks * 32) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                  }
                }
#pragma unroll
                for (int u = 0; u < GB; ++u) {
                  if (g0 + u < ta.n) {
                    f32x4 d = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                      d = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[u][ks], vh[ks], d, 0, 0, 0);
                      d = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[u][ks], vl[ks], d, 0, 0, 0);
                    }
                    if ((ta.rows[g0 + u] >> col) & 1u) acc = d;
                  }
                }
              }
            }
          }
          *reinterpret_cast<f32x4*>(&stage[wave][col][c * 16 + 4 * g]) = acc;
        }
      }
      __syncthreads();
      if (nw < N && ((all >> wt) & 1u)) {
        float d[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 s4 = *reinterpret_cast<const f32x4*>(&stage[wave][wt][wc * 16 + 4 * q]);
          d[4 * q] = s4[0]; d[4 * q + 1] = s4[1]; d[4 * q + 2] = s4[2]; d[4 * q + 3] = s4[3];
        }
        if constexpr (sizeof(YT) == 2) {
          rmw_add<YT, 8>(yrow, d);
          rmw_add<YT, 8>(yrow + 8, d + 8);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) rmw_add<YT, 4>(yrow + 4 * q, d + 4 * q);
        }
      }
      __syncthreads();
    }
  };
  if (one_adapter) run(std::true_type{});
  else run(std::false_type{});
}

__global__ void write_tensor_part_kernel(f16* __restrict__ Z, const f16* __restrict__ X, const f16* __restrict__ Y,
                                         const int32_t* __restrict__ ids, int B, int A, int PH) {
  // Phase split by blockIdx.y: 0 copies X -> Z (skipped when Z aliases X), 1 scatters Y rows.
  const int row = blockIdx.x;
  if (blockIdx.y == 0) {
    if (Z == X || row >= B) return;
    for (int i = threadIdx.x * 8; i < PH; i += blockDim.x * 8) st8(Z + (size_t)row * PH + i, ld8(X + (size_t)row * PH + i));
  } else {
    if (row >= A) return;
    const int dst = ids[row];
    if (dst < 0 || dst >= B) return;
    for (int i = threadIdx.x * 8; i < PH; i += blockDim.x * 8) st8(Z + (size_t)dst * PH + i, ld8(Y + (size_t)row * PH + i));
  }
}

int check_lora_shape(int T, int K, int N, int r, int n_ad) {
  MLORA_CHECK(T >= 0 && K > 0 && N > 0 && n_ad > 0, MLORA_ERR_INVALID, "gather_mm: bad shape T=%d K=%d N=%d n_ad=%d", T, K, N, n_ad);
  MLORA_CHECK(r == 8 || r == 16 || r == 32 || r == 64, MLORA_ERR_UNSUPPORTED, "gather_mm: rank %d not in {8,16,32,64}", r);
  MLORA_CHECK(K % 8 == 0 && N % 8 == 0, MLORA_ERR_UNSUPPORTED, "gather_mm: K=%d and N=%d must be multiples of 8", K, N);
  MLORA_CHECK(n_ad <= 65535 && T <= (1 << 20), MLORA_ERR_UNSUPPORTED, "gather_mm: n_ad=%d or T=%d too large", n_ad, T);
  return MLORA_OK;
}

template <int R, typename YT>
void launch_expand(YT* y, int ldy, const float* vpart, const f16* B, const int32_t* ids, float scaling, int T, int K, int N,
                   int n_ad, hipStream_t s, const int32_t* bucket_of, int bucket) {
  constexpr int CH = 8 * (WAVE / (R / 8));
  hipLaunchKernelGGL((lora_expand_kernel<R, YT>), dim3(n_ad, ceil_div(N, CH)), dim3(64), 0, s, y, vpart, B, ids, scaling,
                     T, N, ldy, lora_k_split(K).kc, bucket_of, bucket);
}

}  // namespace

extern "C" size_t mlora_gather_mm_workspace_bytes(int T, int K, int r) {
  if (T <= 0 || K <= 0 || r <= 0) return 0;
  return (size_t)lora_k_split(K).kc * (size_t)T * (size_t)r * sizeof(float);
}

// A rank bucket restricts a launch to the tokens whose bucket_of[t] equals `bucket` (bucket_of == nullptr: all tokens).
struct BucketFilter {
  const int32_t* bucket_of;
  int bucket;
};

static int shrink_impl(void* v_part, const void* x, int x_layout, const void* A, const int32_t* tok_adapter,
                       int T, int K, int r, int n_ad, BucketFilter bf, void* stream) {
  if (int e = check_lora_shape(T, K, 8, r, n_ad)) return e;
  MLORA_CHECK(x_layout == MLORA_ROWMAJOR || (x_layout == MLORA_FRAG && K % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "lora_shrink: fragment-ordered x needs K %% 32 == 0 (layout=%d K=%d)", x_layout, K);
  MLORA_CHECK(v_part && x && A && tok_adapter, MLORA_ERR_INVALID, "lora_shrink: null pointer");
  if (T == 0) return MLORA_OK;
  const LoraKSplit ks = lora_k_split(K);
  LoraShrinkBatch b = {};
  b.A[0] = (const f16*)A;
  b.n_proj = 1;
  b.vpart = (float*)v_part;
  b.x = (const f16*)x;
  b.ids = tok_adapter;
  b.T = T; b.K = K; b.r = r; b.n_ad = n_ad; b.ci = ks.ci; b.kc = ks.kc;
  b.frag_tt = x_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  b.speculate = n_ad <= 2 * T;
  b.bucket_of = bf.bucket_of;
  b.bucket = bf.bucket;
  hipLaunchKernelGGL(lora_shrink_kernel, dim3(lora_shrink_units(b)), dim3(64), 0, (hipStream_t)stream, b);
  return mlora_launch_status("lora_shrink");
}

extern "C" int mlora_lora_shrink(void* v_part, const void* x, int x_layout, const void* A, const int32_t* tok_adapter,
                                 int T, int K, int r, int n_ad, void* stream) {
  return shrink_impl(v_part, x, x_layout, A, tok_adapter, T, K, r, n_ad, BucketFilter{nullptr, 0}, stream);
}

static int expand_impl(void* y, int y_dtype, int ldy, const void* v_part, const void* B, const int32_t* tok_adapter,
                       float scaling, int T, int K, int N, int r, int n_ad, BucketFilter bf, void* stream) {
  if (int e = check_lora_shape(T, K, N, r, n_ad)) return e;
  MLORA_CHECK(ldy >= N && ldy % 8 == 0, MLORA_ERR_INVALID, "lora_expand: need ldy >= N and ldy %% 8 == 0 (ldy=%d N=%d)", ldy, N);
  MLORA_CHECK(y && v_part && B && tok_adapter, MLORA_ERR_INVALID, "lora_expand: null pointer");
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "lora_expand: bad y_dtype %d", y_dtype);
  if (T == 0) return MLORA_OK;
  hipStream_t s = (hipStream_t)stream;
  const float* vp = (const float*)v_part;
  const f16* Bp = (const f16*)B;
#define MLORA_EXPAND(R)                                                                                   \
  if (y_dtype == MLORA_F16) launch_expand<R, f16>((f16*)y, ldy, vp, Bp, tok_adapter, scaling, T, K, N, n_ad, s, bf.bucket_of, bf.bucket); \
  else launch_expand<R, float>((float*)y, ldy, vp, Bp, tok_adapter, scaling, T, K, N, n_ad, s, bf.bucket_of, bf.bucket)
  switch (r) {
    case 8: MLORA_EXPAND(8); break;
    case 16: MLORA_EXPAND(16); break;
    case 32: MLORA_EXPAND(32); break;
    default: MLORA_EXPAND(64); break;
  }
#undef MLORA_EXPAND
  return mlora_launch_status("lora_expand");
}

extern "C" int mlora_lora_expand(void* y, int y_dtype, int ldy, const void* v_part, const void* B,
                                 const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                                 void* stream) {
  return expand_impl(y, y_dtype, ldy, v_part, B, tok_adapter, scaling, T, K, N, r, n_ad, BucketFilter{nullptr, 0}, stream);
}

// The one-launch kernel applies when the table fits one wave (T <= 64) and the partials fit LDS.
static bool gmm_one_launch_fits(int T, int K, int r) {
  return T > 0 && T <= 64 && (size_t)(lora_k_split(K).kc + 1) * T * r * sizeof(float) <= 48 * 1024;
}

template <int R>
static void gmm_launch_r(const GmmSet& one, const GmmSet* sets, dim3 grid, size_t lds, int y_dtype, const int32_t* ids,
                         float scaling, int T, int K, int N, int n_ad, int ldy, int frag_tt, int P, LoraKSplit ks, hipStream_t s,
                         BucketFilter bf, const GmmBuckets* mb) {
  const dim3 block(GMM_THREADS);
  if (mb != nullptr) {     // adapters of several ranks: R is the largest, bf.bucket_of the per-token bucket
#define MLORA_GMM_MULTI(YT)                                                                                                      \
  hipLaunchKernelGGL((gather_mm_decode_kernel<R, YT, 16, true>), grid, block, lds, s, one, sets, ids, scaling, T, K, N, n_ad, ldy, \
                     frag_tt, P, ks.ci, ks.kc, bf.bucket_of, 0, *mb)
    if (y_dtype == MLORA_F16) MLORA_GMM_MULTI(f16);
    else MLORA_GMM_MULTI(float);
#undef MLORA_GMM_MULTI
    return;
  }
#define MLORA_GMM_LAUNCH(YT, GR)                                                                                              \
  hipLaunchKernelGGL((gather_mm_decode_kernel<R, YT, GR>), grid, block, lds, s, one, sets, ids, scaling, T, K, N, n_ad, ldy, \
                     frag_tt, P, ks.ci, ks.kc, bf.bucket_of, bf.bucket, GmmBuckets())
  const bool many = grid.y > 1;
  if (y_dtype == MLORA_F16) {
    if (many) MLORA_GMM_LAUNCH(f16, 8);
    else MLORA_GMM_LAUNCH(f16, 16);
  } else {
    if (many) MLORA_GMM_LAUNCH(float, 8);
    else MLORA_GMM_LAUNCH(float, 16);
  }
#undef MLORA_GMM_LAUNCH
}

static int gmm_one_launch(const GmmSet& one, const GmmSet* sets, int n_sets, int y_dtype, int ldy, int x_layout,
                          const int32_t* ids, float scaling, int T, int K, int N, int r, int n_ad, hipStream_t s,
                          BucketFilter bf = BucketFilter{nullptr, 0}, const GmmBuckets* mb = nullptr) {
  const LoraKSplit ks = lora_k_split(K);
  const int groups = ceil_div(n_ad, 8);                 // adapters are dealt to the 8 XCDs in groups of 8
  // Output-row slices per adapter: enough workgroups to cover the chip when the launch holds one problem, one slice
  // (no repeated shrink) once the problems themselves supply the parallelism.
  int P = 256 / (groups * 8 * n_sets);
  const int pmax = ceil_div(N, GMM_THREADS);
  if (P > pmax) P = pmax;
  if (P < 1) P = 1;
  const size_t lds = (size_t)(ks.kc + 1) * T * r * sizeof(float);
  const int frag_tt = x_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  const dim3 grid(groups * 8 * P, n_sets);
  switch (r) {
    case 8: gmm_launch_r<8>(one, sets, grid, lds, y_dtype, ids, scaling, T, K, N, n_ad, ldy, frag_tt, P, ks, s, bf, mb); break;
    case 16: gmm_launch_r<16>(one, sets, grid, lds, y_dtype, ids, scaling, T, K, N, n_ad, ldy, frag_tt, P, ks, s, bf, mb); break;
    case 32: gmm_launch_r<32>(one, sets, grid, lds, y_dtype, ids, scaling, T, K, N, n_ad, ldy, frag_tt, P, ks, s, bf, mb); break;
    default: gmm_launch_r<64>(one, sets, grid, lds, y_dtype, ids, scaling, T, K, N, n_ad, ldy, frag_tt, P, ks, s, bf, mb); break;
  }
  return mlora_launch_status("gather_mm");
}

// Problems in a launch from which the two streaming passes pay off (a launch boundary costs a few microseconds; below
// this the single launch with its LDS hand-over is shorter).
constexpr int GMM_STREAM_MIN_SETS = 8;

extern "C" int mlora_gather_mm_batch(const void* const* sets, int n_sets, int y_dtype, int ldy, int x_layout,
                                     const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_lora_shape(T, K, N, r, n_ad)) return e;
  MLORA_CHECK(sets && tok_adapter && n_sets >= 0 && n_sets <= 65535, MLORA_ERR_INVALID, "gather_mm_batch: null pointer or bad n_sets=%d", n_sets);
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "gather_mm_batch: bad y_dtype %d", y_dtype);
  MLORA_CHECK(ldy >= N, MLORA_ERR_INVALID, "gather_mm_batch: need ldy >= N (ldy=%d N=%d)", ldy, N);
  MLORA_CHECK(x_layout == MLORA_ROWMAJOR || (x_layout == MLORA_FRAG && K % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "gather_mm_batch: fragment-ordered x needs K %% 32 == 0");
  if (T == 0 || n_sets == 0) return MLORA_OK;
  MLORA_CHECK(gmm_one_launch_fits(T, K, r), MLORA_ERR_UNSUPPORTED,
              "gather_mm_batch: decode shapes only (T <= 64 and (kc + 1) * T * r * 4 <= 48 KiB; T=%d K=%d r=%d)", T, K, r);
  if (workspace != nullptr && n_sets >= GMM_STREAM_MIN_SETS) {
    const size_t need = (size_t)n_sets * mlora_gather_mm_workspace_bytes(T, K, r);
    MLORA_CHECK(workspace_bytes >= need, MLORA_ERR_WORKSPACE, "gather_mm_batch: workspace of %zu bytes given, %zu needed for %d sets",
                workspace_bytes, need, n_sets);
    return gmm_batch_stream((const GmmSet*)sets, n_sets, y_dtype, ldy, x_layout, tok_adapter, scaling, T, K, N, r, n_ad,
                            (float*)workspace, (hipStream_t)stream);
  }
  return gmm_one_launch(GmmSet(), (const GmmSet*)sets, n_sets, y_dtype, ldy, x_layout, tok_adapter, scaling, T, K, N, r, n_ad,
                        (hipStream_t)stream);
}

// Shrink of pj.n projections on the matrix cores into v [pj.n][splits][T][R] fp32; returns the number of K ranges
// (`splits`) whose partial sums a reader adds in range order.
template <int R>
static int gmm_segments_shrink_r(const SegProjs& pj, const f16* x, int frag_tt, const int32_t* ids, int T, int K, int n_ad, float* v,
                                 BucketFilter bf, hipStream_t s) {
  const int tiles = ceil_div(T, 16);
  // few token tiles: split K over workgroups so that the shrink still covers the chip (partials fit the workspace,
  // which holds lora_k_split(K).kc slices of [T, r] per projection); the same split whatever the number of
  // projections, so that a projection's sums do not depend on what shares its launch
  int splits = 512 / tiles;
  const int kc = lora_k_split(K).kc;
  if (splits > kc) splits = kc;
  if (splits > K / 128) splits = K / 128;
  if (splits < 1) splits = 1;
  // Up to 1024 tokens the call is taken to be a decode batch (one token per sequence, tiles that mix many adapters);
  // beyond that a prefill whose tokens come in adapter segments: four token tiles per shrink workgroup, two per expand
  // workgroup, about two workgroups per compute unit.  Either set of kernels is correct for either input.
  if (T <= 1024) {
    constexpr int NG = 16 / (8 / ((R + 15) / 16));   // adapter groups of a tile, each with its own workgroup
    hipLaunchKernelGGL((lora_shrink_mfma_kernel<R>), dim3(tiles, splits, pj.n * NG), dim3(SEG_WAVES * WAVE), 0, s, v, x, frag_tt, pj, ids, T, K,
                       n_ad, bf.bucket_of, bf.bucket);
  } else {
    const int quads = ceil_div(tiles, 4);
    splits = 256 / quads;                        // few K ranges: the expand adds the ranges' partial sums per token
    if (splits > kc) splits = kc;
    if (splits > K / 128) splits = K / 128;
    if (splits < 1) splits = 1;
    hipLaunchKernelGGL((lora_shrink_quad_mfma_kernel<R>), dim3(quads, splits, pj.n), dim3(SEG_WAVES * WAVE), 0, s, v, x, frag_tt, pj, ids, T,
                       K, n_ad, bf.bucket_of, bf.bucket);
  }
  return splits;
}

template <int R>
static void gmm_segments_r(const SegProjs& pj, int y_dtype, int ldy, const f16* x, int frag_tt, const int32_t* ids, float scaling, int T, int K,
                           int n_ad, float* v, BucketFilter bf, hipStream_t s) {
  const int tiles = ceil_div(T, 16);
  int N = 0;
  for (int i = 0; i < pj.n; ++i) N = pj.N[i] > N ? pj.N[i] : N;
  const bool mixed = T <= 1024;
  const int splits = gmm_segments_shrink_r<R>(pj, x, frag_tt, ids, T, K, n_ad, v, bf, s);
  // column blocks per workgroup: as many as leave about a thousand workgroups (per-workgroup set-up amortised)
  int nit = (int)(((long)tiles * pj.n * ceil_div(N, SEG_WAVES * 64)) / 1024);
  nit = nit < 1 ? 1 : (nit > 8 ? 8 : nit);
  if (!mixed) {
    const int pairs = ceil_div(tiles, 2);
    nit = (int)(((long)pairs * pj.n * ceil_div(N, SEG_WAVES * 64)) / 512);
    nit = nit < 1 ? 1 : (nit > 8 ? 8 : nit);
  }
  const dim3 grid(mixed ? tiles : ceil_div(tiles, 2), ceil_div(N, SEG_WAVES * 64 * nit), pj.n);
#define MLORA_EXPAND_MFMA(KERNEL, YT)                                                                                       \
  hipLaunchKernelGGL((KERNEL<R, YT>), grid, dim3(SEG_WAVES * WAVE), 0, s, pj, v, ids, scaling, T, ldy, n_ad, \
                     bf.bucket_of, bf.bucket, splits, nit)
  if (y_dtype == MLORA_F16) {
    if (mixed) MLORA_EXPAND_MFMA(lora_expand_mixed_mfma_kernel, f16);
    else MLORA_EXPAND_MFMA(lora_expand_pair_mfma_kernel, f16);
  } else {
    if (mixed) MLORA_EXPAND_MFMA(lora_expand_mixed_mfma_kernel, float);
    else MLORA_EXPAND_MFMA(lora_expand_pair_mfma_kernel, float);
  }
#undef MLORA_EXPAND_MFMA
}

// ---------------------------------------------------------------------------------------------
// Pieces of the prefill linear that carries its LoRA delta as extra k-steps of the base GEMM (gemm.hip): the adapter a
// 256-token block agrees on, and the shrink results as fp16 hi + lo halves.
// ---------------------------------------------------------------------------------------------
constexpr int FUSE_BLOCK = 256;            // token block of the persistent GEMM

// blk[b] = the adapter every valid token of block b names (-1: tokens without adapter or of several adapters);
// rest[t] = -1 where the block's delta rides in the GEMM, else ids[t] (what a separate gather-matmul still has to do)
__global__ __launch_bounds__(FUSE_BLOCK) void lora_block_adapters_kernel(int32_t* __restrict__ blk, int32_t* __restrict__ rest,
                                                                       const int32_t* __restrict__ ids, int T, int n_ad) {
  __shared__ int s_first, s_bad;
  const int t = blockIdx.x * FUSE_BLOCK + threadIdx.x;
  if (threadIdx.x == 0) {
    const int raw = ids[blockIdx.x * FUSE_BLOCK];        // the block's first token exists
    s_first = (raw >= 0 && raw < n_ad) ? raw : -1;
    s_bad = 0;
  }
  __syncthreads();
  const int raw = t < T ? ids[t] : s_first;
  const int id = (raw >= 0 && raw < n_ad) ? raw : -1;
  if (id != s_first) s_bad = 1;                            // benign race: every writer stores 1
  __syncthreads();
  const int a = (s_bad || s_first < 0) ? -1 : s_first;
  if (threadIdx.x == 0) blk[blockIdx.x] = a;
  if (t < T) rest[t] = a >= 0 ? -1 : id;
}

// vh, vl [T][R] fp16: hi and lo halves of scaling * (sum of the K-range partials of the shrink, in range order) - the
// values and the split the expand kernels use.  blockIdx.y = projection; v = [n_proj][splits][T, R] fp32.
struct VSplitOut {
  f16* vh[SEG_MAX_PROJ];
  f16* vl[SEG_MAX_PROJ];
};
template <int R>
__global__ __launch_bounds__(256) void lora_v_split_kernel(VSplitOut o, const float* __restrict__ v, int splits, float scaling, int T,
                                                           const int32_t* __restrict__ ids, int n_ad) {
  const int e = blockIdx.x * 256 + threadIdx.x;              // four rank entries of one token
  const int t = e / (R / 4), j = (e % (R / 4)) * 4;
  if (t >= T) return;
  const int pj = blockIdx.y;
  v += (size_t)pj * splits * T * R;
  // the shrink writes rows of adapted tokens only: a token without adapter gets zeros here (what the workspace holds
  // in its row is left over from earlier calls), so that its delta in a block of the extra-k-step linear is zero
  const int id = ids[t];
  const bool adapted = id >= 0 && id < n_ad;
  f16x4 h = f16x4{0, 0, 0, 0}, l = h;
  if (adapted) {
    const f32x4 sum = sum_ranges(v + (size_t)t * R + j, splits, (size_t)T * R);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float f = sum[q] * scaling;
      h[q] = (f16)f;
      l[q] = (f16)(f - (float)h[q]);
    }
  }
  *reinterpret_cast<f16x4*>(o.vh[pj] + (size_t)t * R + j) = h;
  *reinterpret_cast<f16x4*>(o.vl[pj] + (size_t)t * R + j) = l;
}

// shrink + expand on the matrix cores for pj.n projections; v = workspace viewed as [pj.n][splits][T, r] fp32
static int gmm_segments(const SegProjs& pj, int y_dtype, int ldy, const f16* x, int x_layout, const int32_t* ids, float scaling, int T, int K,
                        int r, int n_ad, float* v, BucketFilter bf, hipStream_t s) {
  const int frag_tt = x_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  switch (r) {
    case 8: gmm_segments_r<8>(pj, y_dtype, ldy, x, frag_tt, ids, scaling, T, K, n_ad, v, bf, s); break;
    case 16: gmm_segments_r<16>(pj, y_dtype, ldy, x, frag_tt, ids, scaling, T, K, n_ad, v, bf, s); break;
    case 32: gmm_segments_r<32>(pj, y_dtype, ldy, x, frag_tt, ids, scaling, T, K, n_ad, v, bf, s); break;
    default: gmm_segments_r<64>(pj, y_dtype, ldy, x, frag_tt, ids, scaling, T, K, n_ad, v, bf, s); break;
  }
  return mlora_launch_status("gather_mm");
}

// the matrix-core kernels need 16-byte aligned rows of y and whole 16-column tiles
static bool gmm_segments_fit(const void* y, int ldy, int x_layout, int T, int K, int N) {
  return (x_layout == MLORA_ROWMAJOR || x_layout == MLORA_FRAG) && T > 64 && K % 32 == 0 && N % 16 == 0 && ldy % 8 == 0 && (uintptr_t)y % 16 == 0;
}

static int gather_mm_impl(void* y, int y_dtype, int ldy, const void* x, int x_layout, const void* A, const void* B,
                          const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                          void* workspace, size_t workspace_bytes, BucketFilter bf, void* stream) {
  if (int e = check_lora_shape(T, K, N, r, n_ad)) return e;
  // the workspace is part of the contract whichever kernel runs (the one-launch kernel keeps its partials in LDS)
  MLORA_CHECK(workspace && workspace_bytes >= mlora_gather_mm_workspace_bytes(T, K, r) || T == 0, MLORA_ERR_WORKSPACE,
              "gather_mm: workspace of %zu bytes given, %zu needed", workspace_bytes,
              mlora_gather_mm_workspace_bytes(T, K, r));
  if (gmm_one_launch_fits(T, K, r)) {
    MLORA_CHECK(y && x && A && B && tok_adapter, MLORA_ERR_INVALID, "gather_mm: null pointer");
    MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "gather_mm: bad y_dtype %d", y_dtype);
    MLORA_CHECK(ldy >= N, MLORA_ERR_INVALID, "gather_mm: need ldy >= N (ldy=%d N=%d)", ldy, N);
    MLORA_CHECK(x_layout == MLORA_ROWMAJOR || (x_layout == MLORA_FRAG && K % 32 == 0), MLORA_ERR_UNSUPPORTED,
                "gather_mm: fragment-ordered x needs K %% 32 == 0 (layout=%d K=%d)", x_layout, K);
    const GmmSet one = {y, (const f16*)x, (const f16*)A, (const f16*)B};
    return gmm_one_launch(one, nullptr, 1, y_dtype, ldy, x_layout, tok_adapter, scaling, T, K, N, r, n_ad, (hipStream_t)stream, bf);
  }
  if (gmm_segments_fit(y, ldy, x_layout, T, K, N)) {
    MLORA_CHECK(y && x && A && B && tok_adapter, MLORA_ERR_INVALID, "gather_mm: null pointer");
    MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "gather_mm: bad y_dtype %d", y_dtype);
    MLORA_CHECK(ldy >= N, MLORA_ERR_INVALID, "gather_mm: need ldy >= N (ldy=%d N=%d)", ldy, N);
    SegProjs pj = {};
    pj.A[0] = (const f16*)A; pj.B[0] = (const f16*)B; pj.y[0] = y; pj.N[0] = N; pj.n = 1;
    return gmm_segments(pj, y_dtype, ldy, (const f16*)x, x_layout, tok_adapter, scaling, T, K, r, n_ad, (float*)workspace, bf,
                        (hipStream_t)stream);
  }
  if (int e = shrink_impl(workspace, x, x_layout, A, tok_adapter, T, K, r, n_ad, bf, stream)) return e;
  return expand_impl(y, y_dtype, ldy, workspace, B, tok_adapter, scaling, T, K, N, r, n_ad, bf, stream);
}

extern "C" int mlora_gather_mm(void* y, int y_dtype, int ldy, const void* x, int x_layout, const void* A, const void* B,
                               const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                               void* workspace, size_t workspace_bytes, void* stream) {
  return gather_mm_impl(y, y_dtype, ldy, x, x_layout, A, B, tok_adapter, scaling, T, K, N, r, n_ad, workspace, workspace_bytes,
                        BucketFilter{nullptr, 0}, stream);
}

// ---------------------------------------------------------------------------------------------
// mlora_gather_mm without a caller workspace and without any allocation: the shrink results of the T > 64 kernels
// (and the K-slice partials of the odd-shape pair) live in a file-scope device array.  Every device the library runs
// on holds its own copy of the array at its own address until the process ends; the address is looked up once per
// device, with that device current, and host code uses that address - never the array's name - from then on.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[MLORA_GATHER_MM_STATIC_BYTES];

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[STATIC_MAX_DEVICES] = {};

// Device address of `scratch` on the current device (nullptr after setting the error message).
void* static_scratch_ptr() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) {
    mlora_set_error(MLORA_ERR_LAUNCH, "gather_mm_static: cannot name the current device (%d)", dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      mlora_set_error(MLORA_ERR_LAUNCH, "gather_mm_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" size_t mlora_gather_mm_static_max_bytes(void) { return MLORA_GATHER_MM_STATIC_BYTES; }

extern "C" int mlora_gather_mm_static(void* y, int y_dtype, int ldy, const void* x, int x_layout, const void* A, const void* B,
                                      const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                                      void* stream) {
  if (int e = check_lora_shape(T, K, N, r, n_ad)) return e;
  const size_t need = mlora_gather_mm_workspace_bytes(T, K, r);
  MLORA_CHECK(need <= (size_t)MLORA_GATHER_MM_STATIC_BYTES, MLORA_ERR_WORKSPACE,
              "gather_mm_static: T=%d K=%d r=%d needs %zu bytes of scratch, the built-in buffer holds %zu (use mlora_gather_mm "
              "with a workspace)", T, K, r, need, (size_t)MLORA_GATHER_MM_STATIC_BYTES);
  if (T == 0) return MLORA_OK;
  void* ws = static_scratch_ptr();
  if (ws == nullptr) return MLORA_ERR_LAUNCH;
  return gather_mm_impl(y, y_dtype, ldy, x, x_layout, A, B, tok_adapter, scaling, T, K, N, r, n_ad, ws,
                        (size_t)MLORA_GATHER_MM_STATIC_BYTES, BucketFilter{nullptr, 0}, stream);
}

// One launch for n_proj projections that share x (columns col_offset[p] .. + n_cols[p] of y) and n_buckets rank buckets
// each; buckets is [n_proj][n_buckets].  Returns 1 when the launch was made, 0 when the shapes do not allow it (the
// caller then falls back to a launch sequence per bucket), < 0 on an argument error.
static int gmm_multi_one_launch(void* y, int y_dtype, int ldy, const void* x, int x_layout, const mlora_lora_bucket* buckets,
                                int n_buckets, int n_proj, const int32_t* col_offset, const int32_t* n_cols,
                                const int32_t* tok_bucket, const int32_t* tok_adapter, int T, int K, hipStream_t stream) {
  int rmax = 0, total = 0, live = 0, nmax = 0;
  for (int e = 0; e < n_proj * n_buckets; ++e) {
    if (!buckets[e].A) continue;
    ++live;
    total += buckets[e].n_ad;
    if (buckets[e].r > rmax) rmax = buckets[e].r;
    if (n_cols[e / n_buckets] > nmax) nmax = n_cols[e / n_buckets];
  }
  if (live < 2 || live > GMM_MAX_BUCKETS || !gmm_one_launch_fits(T, K, rmax)) return 0;
  MLORA_CHECK(y && x, MLORA_ERR_INVALID, "gather_mm_multi: null pointer");
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "gather_mm_multi: bad y_dtype %d", y_dtype);
  MLORA_CHECK(x_layout == MLORA_ROWMAJOR || (x_layout == MLORA_FRAG && K % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "gather_mm_multi: fragment-ordered x needs K %% 32 == 0");
  GmmBuckets mb = {};
  int first = 0, n = 0;
  for (int e = 0; e < n_proj * n_buckets; ++e) {
    if (!buckets[e].A) continue;           // absent entries take no workgroups
    const int p = e / n_buckets;
    MLORA_CHECK(col_offset[p] >= 0 && n_cols[p] > 0 && col_offset[p] + n_cols[p] <= ldy, MLORA_ERR_INVALID,
                "gather_mm_multi: columns %d..%d of projection %d outside a row of %d", col_offset[p], col_offset[p] + n_cols[p], p, ldy);
    mb.A[n] = (const f16*)buckets[e].A;
    mb.B[n] = (const f16*)buckets[e].B;
    mb.r[n] = buckets[e].r;
    mb.scaling[n] = buckets[e].scaling;
    mb.tok_bucket[n] = e % n_buckets;
    mb.ycol[n] = col_offset[p];
    mb.ncols[n] = n_cols[p];
    mb.first[n] = first;
    first += buckets[e].n_ad;
    ++n;
  }
  for (int e = n; e <= GMM_MAX_BUCKETS; ++e) mb.first[e] = first;
  mb.n = n;
  GmmSet one = {y, (const f16*)x, nullptr, nullptr};
  if (int rc = gmm_one_launch(one, nullptr, 1, y_dtype, ldy, x_layout, tok_adapter, 1.f, T, K, nmax, rmax, total, stream,
                              BucketFilter{tok_bucket, 0}, &mb))
    return rc;
  return 1;
}

extern "C" int mlora_gather_mm_multi(void* y, int y_dtype, int ldy, const void* x, int x_layout,
                                     const mlora_lora_bucket* buckets, int n_buckets, const int32_t* tok_bucket,
                                     const int32_t* tok_adapter, int T, int K, int N, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  MLORA_CHECK(buckets && n_buckets > 0 && n_buckets <= 64, MLORA_ERR_INVALID, "gather_mm_multi: bad bucket list (n_buckets=%d)", n_buckets);
  MLORA_CHECK((tok_bucket || n_buckets == 1) && tok_adapter, MLORA_ERR_INVALID, "gather_mm_multi: null id array");
  // validate every bucket before the first launch, so that an error leaves y untouched
  for (int b = 0; b < n_buckets; ++b) {
    if (!buckets[b].A && !buckets[b].B) continue;       // this bucket's adapters do not target the projection
    if (int e = check_lora_shape(T, K, N, buckets[b].r, buckets[b].n_ad)) return e;
    MLORA_CHECK(buckets[b].A && buckets[b].B, MLORA_ERR_INVALID, "gather_mm_multi: bucket %d has one null table", b);
    MLORA_CHECK(T == 0 || (workspace && workspace_bytes >= mlora_gather_mm_workspace_bytes(T, K, buckets[b].r)), MLORA_ERR_WORKSPACE,
                "gather_mm_multi: workspace of %zu bytes given, %zu needed for bucket %d (rank %d)", workspace_bytes,
                mlora_gather_mm_workspace_bytes(T, K, buckets[b].r), b, buckets[b].r);
  }
  // Decode-sized batches with up to GMM_MAX_BUCKETS buckets: ONE launch serves all ranks (same bits as a launch per bucket)
  const int32_t zero = 0;
  if (int rc = gmm_multi_one_launch(y, y_dtype, ldy, x, x_layout, buckets, n_buckets, 1, &zero, &N, tok_bucket, tok_adapter, T, K,
                                    (hipStream_t)stream))
    return rc < 0 ? rc : MLORA_OK;   // > 0: launched
  for (int b = 0; b < n_buckets; ++b) {
    if (!buckets[b].A) continue;
    if (int e = gather_mm_impl(y, y_dtype, ldy, x, x_layout, buckets[b].A, buckets[b].B, tok_adapter, buckets[b].scaling, T, K, N,
                               buckets[b].r, buckets[b].n_ad, workspace, workspace_bytes, BucketFilter{tok_bucket, b}, stream))
      return e;
  }
  return MLORA_OK;
}

extern "C" int mlora_gather_mm_multi_proj(void* y, int y_dtype, int ldy, const void* x, int x_layout,
                                          const mlora_lora_bucket* buckets, int n_buckets, int n_proj,
                                          const int32_t* col_offset, const int32_t* n_cols, const int32_t* tok_bucket,
                                          const int32_t* tok_adapter, int T, int K, void* workspace, size_t workspace_bytes,
                                          void* stream) {
  MLORA_CHECK(buckets && n_buckets > 0 && n_buckets <= 64 && n_proj > 0 && n_proj <= 8, MLORA_ERR_INVALID,
              "gather_mm_multi_proj: bad bucket list (n_buckets=%d n_proj=%d)", n_buckets, n_proj);
  MLORA_CHECK(y && x && col_offset && n_cols && (tok_bucket || n_buckets == 1) && tok_adapter, MLORA_ERR_INVALID,
              "gather_mm_multi_proj: null pointer");
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "gather_mm_multi_proj: bad y_dtype %d", y_dtype);
  // validate everything before the first launch, so that an error leaves y untouched
  for (int p = 0; p < n_proj; ++p) {
    MLORA_CHECK(col_offset[p] >= 0 && col_offset[p] % 8 == 0 && n_cols[p] > 0 && col_offset[p] + n_cols[p] <= ldy, MLORA_ERR_INVALID,
                "gather_mm_multi_proj: projection %d: columns %d..%d (offset must be a multiple of 8, row of %d)", p, col_offset[p],
                col_offset[p] + n_cols[p], ldy);
    for (int b = 0; b < n_buckets; ++b) {
      const mlora_lora_bucket& bk = buckets[p * n_buckets + b];
      if (!bk.A && !bk.B) continue;
      if (int e = check_lora_shape(T, K, n_cols[p], bk.r, bk.n_ad)) return e;
      MLORA_CHECK(bk.A && bk.B, MLORA_ERR_INVALID, "gather_mm_multi_proj: projection %d bucket %d has one null table", p, b);
      MLORA_CHECK(T == 0 || (workspace && workspace_bytes >= mlora_gather_mm_workspace_bytes(T, K, bk.r)), MLORA_ERR_WORKSPACE,
                  "gather_mm_multi_proj: workspace of %zu bytes given, %zu needed (rank %d)", workspace_bytes,
                  mlora_gather_mm_workspace_bytes(T, K, bk.r), bk.r);
    }
  }
  if (int rc = gmm_multi_one_launch(y, y_dtype, ldy, x, x_layout, buckets, n_buckets, n_proj, col_offset, n_cols, tok_bucket,
                                    tok_adapter, T, K, (hipStream_t)stream))
    return rc < 0 ? rc : MLORA_OK;
  const size_t esz = y_dtype == MLORA_F16 ? 2 : 4;
  if (T == 0) return MLORA_OK;
  // Larger batches: per rank bucket, the projections that carry it (same rank, table size and scaling) share one
  // shrink launch and one expand launch on the matrix cores when the workspace holds a slice for each of them.
  bool done[8 * 64] = {};
  for (int b = 0; b < n_buckets; ++b) {
    SegProjs pj = {};
    int members[SEG_MAX_PROJ];
    const mlora_lora_bucket* lead = nullptr;
    for (int p = 0; p < n_proj && pj.n < SEG_MAX_PROJ; ++p) {
      const mlora_lora_bucket& bk = buckets[p * n_buckets + b];
      void* yp = (char*)y + (size_t)col_offset[p] * esz;
      if (!bk.A || !gmm_segments_fit(yp, ldy, x_layout, T, K, n_cols[p])) continue;
      if (lead && (bk.r != lead->r || bk.n_ad != lead->n_ad || bk.scaling != lead->scaling)) continue;
      if (!lead) lead = &bk;
      pj.A[pj.n] = (const f16*)bk.A; pj.B[pj.n] = (const f16*)bk.B; pj.y[pj.n] = yp; pj.N[pj.n] = n_cols[p];
      members[pj.n++] = p;
    }
    if (pj.n >= 2 && workspace_bytes >= (size_t)pj.n * mlora_gather_mm_workspace_bytes(T, K, lead->r)) {
      if (int e = gmm_segments(pj, y_dtype, ldy, (const f16*)x, x_layout, tok_adapter, lead->scaling, T, K, lead->r, lead->n_ad,
                               (float*)workspace, BucketFilter{tok_bucket, b}, (hipStream_t)stream))
        return e;
      for (int i = 0; i < pj.n; ++i) done[members[i] * n_buckets + b] = true;
    }
  }
  for (int p = 0; p < n_proj; ++p)
    for (int b = 0; b < n_buckets; ++b) {
      const mlora_lora_bucket& bk = buckets[p * n_buckets + b];
      if (!bk.A || done[p * n_buckets + b]) continue;
      if (int e = gather_mm_impl((char*)y + (size_t)col_offset[p] * esz, y_dtype, ldy, x, x_layout, bk.A, bk.B, tok_adapter, bk.scaling,
                                 T, K, n_cols[p], bk.r, bk.n_ad, workspace, workspace_bytes, BucketFilter{tok_bucket, b}, stream))
        return e;
    }
  return MLORA_OK;
}

extern "C" int mlora_lora_block_adapters(int32_t* blk_adapter, int32_t* tok_rest, const int32_t* tok_adapter, int T, int n_ad,
                                         void* stream) {
  MLORA_CHECK(blk_adapter && tok_rest && tok_adapter, MLORA_ERR_INVALID, "lora_block_adapters: null pointer");
  MLORA_CHECK(T >= 0 && n_ad > 0, MLORA_ERR_INVALID, "lora_block_adapters: bad T=%d n_ad=%d", T, n_ad);
  if (T == 0) return MLORA_OK;
  hipLaunchKernelGGL(lora_block_adapters_kernel, dim3(ceil_div(T, FUSE_BLOCK)), dim3(FUSE_BLOCK), 0, (hipStream_t)stream, blk_adapter, tok_rest,
                     tok_adapter, T, n_ad);
  return mlora_launch_status("lora_block_adapters");
}

extern "C" int mlora_lora_shrink_split(void* const* v_hi, void* const* v_lo, const void* x, int x_layout, const void* const* A, int n_proj,
                                       const int32_t* tok_adapter, float scaling, int T, int K, int r, int n_ad, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  MLORA_CHECK(v_hi && v_lo && x && A && tok_adapter && n_proj >= 1 && n_proj <= SEG_MAX_PROJ, MLORA_ERR_INVALID,
              "lora_shrink_split: null pointer or n_proj outside 1..%d", SEG_MAX_PROJ);
  MLORA_CHECK((r == 32 || r == 64) && n_ad > 0 && n_ad <= 65535, MLORA_ERR_UNSUPPORTED, "lora_shrink_split: rank %d not in {32, 64} or bad n_ad %d", r, n_ad);
  MLORA_CHECK(T > 64 && K > 0 && K % 32 == 0 && (x_layout == MLORA_ROWMAJOR || x_layout == MLORA_FRAG), MLORA_ERR_UNSUPPORTED,
              "lora_shrink_split: needs T > 64, K %% 32 == 0 (T=%d K=%d layout=%d)", T, K, x_layout);
  MLORA_CHECK(workspace && workspace_bytes >= (size_t)n_proj * mlora_gather_mm_workspace_bytes(T, K, r), MLORA_ERR_WORKSPACE,
              "lora_shrink_split: workspace of %zu bytes given, %zu needed", workspace_bytes, (size_t)n_proj * mlora_gather_mm_workspace_bytes(T, K, r));
  SegProjs pj = {};
  for (int i = 0; i < n_proj; ++i) {
    MLORA_CHECK(A[i] && v_hi[i] && v_lo[i], MLORA_ERR_INVALID, "lora_shrink_split: null table or output of projection %d", i);
    pj.A[i] = (const f16*)A[i];
  }
  pj.n = n_proj;
  hipStream_t s = (hipStream_t)stream;
  const int frag_tt = x_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  float* v = (float*)workspace;
  const BucketFilter bf{nullptr, 0};
  int splits;
  if (r == 32) splits = gmm_segments_shrink_r<32>(pj, (const f16*)x, frag_tt, tok_adapter, T, K, n_ad, v, bf, s);
  else splits = gmm_segments_shrink_r<64>(pj, (const f16*)x, frag_tt, tok_adapter, T, K, n_ad, v, bf, s);
  VSplitOut vo = {};
  for (int i = 0; i < n_proj; ++i) {
    vo.vh[i] = (f16*)v_hi[i];
    vo.vl[i] = (f16*)v_lo[i];
  }
  const dim3 grid(ceil_div(T * (r / 4), 256), n_proj);
  if (r == 32) hipLaunchKernelGGL((lora_v_split_kernel<32>), grid, dim3(256), 0, s, vo, v, splits, scaling, T, tok_adapter, n_ad);
  else hipLaunchKernelGGL((lora_v_split_kernel<64>), grid, dim3(256), 0, s, vo, v, splits, scaling, T, tok_adapter, n_ad);
  return mlora_launch_status("lora_shrink_split");
}

extern "C" int mlora_write_tensor_part(void* Z, const void* X, const void* Y, const int32_t* ids, int B, int A, int PH,
                                       void* stream) {
  MLORA_CHECK(B >= 0 && A >= 0 && PH > 0 && PH % 8 == 0, MLORA_ERR_INVALID, "write_tensor_part: bad shape B=%d A=%d PH=%d", B, A, PH);
  MLORA_CHECK(Z && X && (A == 0 || (Y && ids)), MLORA_ERR_INVALID, "write_tensor_part: null pointer");
  const int rows = B > A ? B : A;
  if (rows == 0) return MLORA_OK;
  // copy then scatter are ordered by two launches on the same stream
  hipStream_t s = (hipStream_t)stream;
  if (Z != X && B > 0)
    hipLaunchKernelGGL(write_tensor_part_kernel, dim3(B, 1), dim3(256), 0, s, (f16*)Z, (const f16*)X, (const f16*)Y, ids, B, A, PH);
  if (A > 0) {
    // blockIdx.y == 1 selects the scatter phase
    hipLaunchKernelGGL(write_tensor_part_kernel, dim3(A, 2), dim3(256), 0, s, (f16*)Z, (const f16*)Z, (const f16*)Y, ids, B, A, PH);
  }
  return mlora_launch_status("write_tensor_part");
}
