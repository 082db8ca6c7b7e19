// Many decode-shaped gather-matmul problems of one shape and one token->adapter table as two streaming passes:
//     pass 1 (shrink)  v[set][t][:] = scaling * sum_c A_set[id_t][:, K-slice c] . x_set[t, K-slice c]
//     pass 2 (expand)  y_set[t, :] += B_set[id_t] . v[set][t][:]
// A launch that holds hundreds of problems is bound by what a compute unit can take in per second, not by the latency
// of one problem.  What that wants is independent requests and no byte fetched twice: in pass 1 a wave needs nothing
// but the table row before it can request its whole slice of A[a] and the x rows of a's tokens, and the workgroup
// (one per set and adapter, a wave per K-slice) finishes v in LDS, so that 64 bytes per token cross to pass 2; in
// pass 2 a wave owns 256 rows of B[a] (8 KiB, read as they lie in memory), requests them, the y elements under them
// and v at once, and never waits for another wave.  The one-launch kernel, whose workgroups shrink and then expand, is
// what a single problem wants (one launch instead of two); over 128 problems of the benchmark shape it reaches 3.4
// TB/s where the two passes reach 5.1.
// The arithmetic is that of lora_shrink_unit / the one-launch kernel, sum for sum, so the result bits are the same.
#include "gather_mm_batch.h"

namespace {

struct BatchArgs {
  const GmmSet* sets;
  const int32_t* ids;
  float* ws;             // v [n_sets][T][r] fp32: shrink results, summed over the K-slices and scaled
  size_t ws_stride;      // floats per set
  int T, K, N, r, n_ad, ci, kc, frag_tt, ldy;
  float scaling;
};

__device__ __forceinline__ f16x8 x_slice(const f16* __restrict__ x, int t, int k, int K, int frag_tt) {
  return ld8(x + (frag_tt ? frag_offset(t, k, frag_tt) : (size_t)t * K + k));
}

// Pass 1.  One workgroup per (set, adapter), wave c = K-slice c.  The waves leave their fp32 partials in LDS; the
// workgroup then adds them in slice order and scales (lora_v), so that what crosses to pass 2 is one finished
// v[t][0..r) per token: 64 bytes at rank 16, instead of kc partial rows that every pass-2 wave would have to fetch again.
// With the whole slice in registers (rank <= 16, one 512-wide chunk per slice) the x rows of the next token pair are
// requested before the current pair is reduced.
template <bool RESIDENT>   // the wave's whole slice of A[a] fits its registers (rank <= 16, one 512-wide chunk per slice)
__global__ __launch_bounds__(LORA_MAX_KC* WAVE, (RESIDENT ? 4 : 2)) void gmm_batch_shrink_kernel(BatchArgs a, int speculate) {
  extern __shared__ float part[];              // [kc][T][r]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int ad = blockIdx.x;
  const GmmSet s = a.sets[blockIdx.y];
  const int r = a.r, K = a.K, T = a.T;
  const int id = lane < T ? a.ids[lane] : -1;
  constexpr int G = 16;
  const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  constexpr bool resident = RESIDENT;
  const f16* __restrict__ A = s.A + (size_t)ad * r * K;
  const int kbase = wave * LORA_KCHUNK + lane * 8;
  const bool in = kbase < K;
  f16x8 areg[G];
  if (resident && speculate) {
#pragma unroll
    for (int j = 0; j < G; ++j) areg[j] = (j < r && in) ? ld8(A + (size_t)j * K + kbase) : zero8;
  }
  const unsigned long long mine = __ballot(id == ad);
  if (!mine) return;                           // workgroup-uniform
  if constexpr (!resident) {
    LoraShrinkBatch b = {};
    b.A[0] = s.A;
    b.n_proj = 1;
    b.vpart = part;
    b.x = s.x;
    b.ids = a.ids;
    b.T = T; b.K = K; b.r = r; b.n_ad = a.n_ad; b.ci = a.ci; b.kc = a.kc; b.frag_tt = a.frag_tt;
    b.speculate = 0;
    b.bucket_of = nullptr;
    b.bucket = 0;
    lora_shrink_unit(b, ad * a.kc + wave, lane);
  } else {
    float* __restrict__ vp = part + (size_t)wave * T * r;
    unsigned long long m = mine;
    int t0 = __builtin_ctzll(m);
    m &= m - 1;
    int t1 = -1;
    if (m) {
      t1 = __builtin_ctzll(m);
      m &= m - 1;
    }
    // x ahead of A: loads come back in request order, so the products of row j can start as soon as row j is in
    f16x8 x0 = in ? x_slice(s.x, t0, kbase, K, a.frag_tt) : zero8;
    f16x8 x1 = in ? x_slice(s.x, t1 >= 0 ? t1 : t0, kbase, K, a.frag_tt) : zero8;
    if (!speculate) {
#pragma unroll
      for (int j = 0; j < G; ++j) areg[j] = (j < r && in) ? ld8(A + (size_t)j * K + kbase) : zero8;
    }
    while (true) {
      int n0 = -1, n1 = -1;                    // the next pair: requested now, used in the next round
      f16x8 y0 = zero8, y1 = zero8;
      if (m) {
        n0 = __builtin_ctzll(m);
        m &= m - 1;
        if (m) {
          n1 = __builtin_ctzll(m);
          m &= m - 1;
        }
        if (in) {
          y0 = x_slice(s.x, n0, kbase, K, a.frag_tt);
          y1 = x_slice(s.x, n1 >= 0 ? n1 : n0, kbase, K, a.frag_tt);
        }
      }
      float p0[G], p1[G];
#pragma unroll
      for (int j = 0; j < G; ++j) {
        p0[j] = dot8(areg[j], x0, 0.f);
        p1[j] = dot8(areg[j], x1, 0.f);
      }
      const int j0 = reduce_transpose<G>(p0, lane);
      if (j0 < r && (lane & (WAVE / G - 1)) == 0) vp[(size_t)t0 * r + j0] = p0[0];
      const int j1 = reduce_transpose<G>(p1, lane);
      if (t1 >= 0 && j1 < r && (lane & (WAVE / G - 1)) == 0) vp[(size_t)t1 * r + j1] = p1[0];
      if (n0 < 0) break;
      t0 = n0; t1 = n1; x0 = y0; x1 = y1;
    }
  }
  __syncthreads();
  float* __restrict__ vout = a.ws + (size_t)blockIdx.y * a.ws_stride;
  for (int e = threadIdx.x; e < T * r; e += blockDim.x) {
    const int t = e / r, j = e % r;
    if ((mine >> t) & 1) vout[e] = lora_v(part, a.kc, T, r, t, j, a.scaling);
  }
}

// Pass 1 as a persistent launch: one workgroup per compute unit walks (set, adapter in use) pairs, and the whole of pair
// i + 1 - the wave's slice of A[a], 16 rows, and the x rows of a's first four tokens - is requested before pair i is
// reduced.  As one short-lived workgroup per pair, every pair paid its own memory round trips with an empty pipeline
// (table row, set pointers, then A and x); here a workgroup pays them once per launch: the token->adapter table is
// the same for all sets, so the adapters in use and their token masks are found once, the set pointers of a
// workgroup's pairs are fetched 64 pairs at a time, one pair per lane, and handed out by lane reads, and adapters
// without a token cost nothing.  Every load of the pipeline is unconditional (addresses are clamped into the tables
// and what a lane must not use is zeroed where it is used): only then can the waits be counted per register, and a
// wait for pair i leaves the requests of pair i + 1 in flight.  The arithmetic of a pair is that of
// gmm_batch_shrink_kernel<true>: the same bits.
// (pointers that were put together from lane reads are plain integers to the compiler: they are declared as pointers
// into global memory, or every load through them would be a flat load, whose completion cannot be counted per register)
typedef const __attribute__((address_space(1))) f16* gf16p;
__device__ __forceinline__ f16x8 gld8(gf16p p) { return *reinterpret_cast<const __attribute__((address_space(1))) f16x8*>(p); }
__device__ __forceinline__ f16x8 gx_slice(gf16p x, int t, int k, int K, int frag_tt) {
  return gld8(x + (frag_tt ? frag_offset(t, k, frag_tt) : (size_t)t * K + k));
}

struct ShrinkPair {
  f16x8 a[16];           // the wave's K-slice of the adapter's 16 rows of A (rows past the rank repeat the last row)
  f16x8 x[4];            // the slice of the x rows of the adapter's first four tokens (fewer: the last one repeated)
  gf16p xs;              // x of the pair's set
  unsigned long long mask;
  int set;
};

__global__ __launch_bounds__(LORA_MAX_KC* WAVE, 1) void gmm_batch_shrink_pers_kernel(BatchArgs a, int n_sets) {
  extern __shared__ float part_all[];           // [2][kc][T][r]: the partials of a pair, double buffered
  __shared__ unsigned long long s_mask[WAVE];
  __shared__ int s_used[WAVE];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = a.r, K = a.K, T = a.T, kc = a.kc;
  constexpr int G = 16;
  const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  const int raw = lane < T ? a.ids[lane] : -1;
  const int id = (raw >= 0 && raw < a.n_ad) ? raw : -1;
  // the adapters in use, in the order of their first token, with the tokens of each (every wave finds the same list)
  int n_used = 0;
  for (unsigned long long todo = __ballot(id >= 0); todo;) {
    const int ad = __builtin_amdgcn_readlane(id, __builtin_ctzll(todo));
    const unsigned long long m = __ballot(id == ad);
    if (threadIdx.x == 0) {
      s_used[n_used] = ad;
      s_mask[n_used] = m;
    }
    ++n_used;
    todo &= ~m;
  }
  __syncthreads();
  const int total = n_sets * n_used;
  const int n_wg = gridDim.x, wg = blockIdx.x;
  // pairs wg, wg + n_wg, ...: the adapters of one set are worked on by neighbouring workgroups at the same time (a
  // contiguous range of pairs per workgroup measured 6 % slower)
  const int my_pairs = wg < total ? (total - wg + n_wg - 1) / n_wg : 0;
  const int kbase = wave * LORA_KCHUNK + lane * 8;
  const bool in = kbase < K;
  const int kld = in ? kbase : 0;               // where this lane reads; what it reads past K is multiplied by zeros
  const int rlast = r - 1;
  const size_t part_sz = (size_t)kc * T * r;

  for (int c0 = 0; c0 < my_pairs; c0 += WAVE) {
    // lane l holds where pair c0 + l of this workgroup lives
    const int qi = c0 + lane;
    unsigned long long pA = 0, px = 0;
    int pu = 0, pset = 0;
    if (qi < my_pairs) {
      const int q = wg + qi * n_wg;
      pset = q / n_used;
      pu = q - pset * n_used;
      const GmmSet* sp = a.sets + pset;
      pA = (unsigned long long)sp->A;
      px = (unsigned long long)sp->x;
    }
    const int nchunk = my_pairs - c0 < WAVE ? my_pairs - c0 : WAVE;
    auto lane_u64 = [](unsigned long long v, int l) -> unsigned long long {
      const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)v, l);
      const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(v >> 32), l);
      return ((unsigned long long)hi << 32) | lo;
    };
    auto fetch = [&](int i, ShrinkPair& P) {
      const int u = __builtin_amdgcn_readlane(pu, i);
      P.set = __builtin_amdgcn_readlane(pset, i);
      P.xs = (gf16p)lane_u64(px, i);
      P.mask = s_mask[u];
      const gf16p A = (gf16p)lane_u64(pA, i) + (size_t)s_used[u] * r * K;
      unsigned long long m = P.mask;
      int t = __builtin_ctzll(m);
      // x ahead of A: loads come back in request order, so the products of row j can start as soon as row j is in
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        P.x[q] = gx_slice(P.xs, t, kld, K, a.frag_tt);
        m &= m - 1;
        if (m) t = __builtin_ctzll(m);
      }
#pragma unroll
      for (int j = 0; j < G; ++j) P.a[j] = gld8(A + (size_t)(j < r ? j : rlast) * K + kld);
    };
    auto reduce = [&](ShrinkPair& P, int buf) {
      float* __restrict__ pb = part_all + (size_t)buf * part_sz;
      float* __restrict__ vp = pb + (size_t)wave * T * r;
      unsigned long long m = P.mask;
      // one token pair: the products of the 16 rows with both tokens, reduced over the lanes, into the wave's partials
      auto token_pair = [&](f16x8 x0, f16x8 x1, int t0, int t1) {
        if (!in) {
          x0 = zero8;
          x1 = zero8;
        }
        float p0[G], p1[G];
#pragma unroll
        for (int j = 0; j < G; ++j) {
          p0[j] = dot8(P.a[j], x0, 0.f);
          p1[j] = dot8(P.a[j], x1, 0.f);
        }
        const int j0 = reduce_transpose<G>(p0, lane);
        if (j0 < r && (lane & (WAVE / G - 1)) == 0) vp[(size_t)t0 * r + j0] = p0[0];
        const int j1 = reduce_transpose<G>(p1, lane);
        if (t1 >= 0 && j1 < r && (lane & (WAVE / G - 1)) == 0) vp[(size_t)t1 * r + j1] = p1[0];
      };
      auto next_token = [&]() -> int {
        if (!m) return -1;
        const int t = __builtin_ctzll(m);
        m &= m - 1;
        return t;
      };
      int t0 = next_token(), t1 = next_token();
      token_pair(P.x[0], P.x[1], t0, t1);
      t0 = next_token();
      if (t0 >= 0) {                             // a third and fourth token: their rows came with the pair
        t1 = next_token();
        token_pair(P.x[2], P.x[3], t0, t1);
        t0 = next_token();
        while (t0 >= 0) {                        // more than four tokens of one adapter: fetched now (this drains the pipeline)
          t1 = next_token();
          const f16x8 x0 = gx_slice(P.xs, t0, kld, K, a.frag_tt);
          const f16x8 x1 = gx_slice(P.xs, t1 >= 0 ? t1 : t0, kld, K, a.frag_tt);
          token_pair(x0, x1, t0, t1);
          t0 = next_token();
        }
      }
      // the partials are in LDS; the bare barrier: __syncthreads() would first wait for the next pair's requests as well
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      bare_barrier();
      // the slices' partials, added in slice order and scaled; the other buffer is free for the next pair meanwhile
      float* __restrict__ vout = a.ws + (size_t)P.set * a.ws_stride;
      for (int e = threadIdx.x; e < T * r; e += blockDim.x) {
        const int t = e / r, j = e % r;
        if ((P.mask >> t) & 1) vout[e] = lora_v(pb, kc, T, r, t, j, a.scaling);
      }
    };
    if (c0 > 0) {                                // the previous chunk's last pair may still be read from its buffer
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      bare_barrier();
    }
    // Two pairs in turn, each in registers of its own; no request sits behind a condition inside the loop, and the last
    // one or two pairs of the chunk are worked off after it.
    ShrinkPair P0, P1;
    fetch(0, P0);
    int i = 0;
    for (; i + 2 < nchunk; i += 2) {
      fetch(i + 1, P1);
      reduce(P0, 0);
      fetch(i + 2, P0);
      reduce(P1, 1);
    }
    if (i + 1 < nchunk) {
      fetch(i + 1, P1);
      reduce(P0, 0);
      reduce(P1, 1);
    } else {
      reduce(P0, 0);
    }
  }
}

template <typename YT, int N>
struct YRow;
template <> struct YRow<f16, 8> { typedef f16x8 type; };
template <> struct YRow<f16, 4> { typedef f16x4 type; };
template <> struct YRow<f16, 2> { typedef f16x2 type; };
template <> struct YRow<float, 4> { typedef f32x4 type; };
template <> struct YRow<float, 2> { typedef f32x2 type; };

// RPL consecutive y elements as fp32, in pieces of at most 16 bytes (vec: the pieces are aligned)
template <typename YT, int RPL>
__device__ __forceinline__ void y_load(const YT* __restrict__ p, float (&out)[RPL], bool vec) {
  constexpr int PIECE = RPL * sizeof(YT) > 16 ? 16 / sizeof(YT) : RPL;
  if constexpr (PIECE == 1) {
    out[0] = (float)p[0];
  } else {
    if (vec) {
      typedef typename YRow<YT, PIECE>::type V;
#pragma unroll
      for (int c = 0; c < RPL / PIECE; ++c) {
        const V v = *reinterpret_cast<const V*>(p + c * PIECE);
#pragma unroll
        for (int q = 0; q < PIECE; ++q) out[c * PIECE + q] = (float)v[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < RPL; ++q) out[q] = (float)p[q];
    }
  }
}

template <typename YT, int RPL>
__device__ __forceinline__ void y_store(YT* __restrict__ p, const YT (&in)[RPL], bool vec) {
  constexpr int PIECE = RPL * sizeof(YT) > 16 ? 16 / sizeof(YT) : RPL;
  if constexpr (PIECE == 1) {
    p[0] = in[0];
  } else {
    if (vec) {
      typedef typename YRow<YT, PIECE>::type V;
#pragma unroll
      for (int c = 0; c < RPL / PIECE; ++c) {
        V v;
#pragma unroll
        for (int q = 0; q < PIECE; ++q) v[q] = in[c * PIECE + q];
        *reinterpret_cast<V*>(p + c * PIECE) = v;
      }
    } else {
#pragma unroll
      for (int q = 0; q < RPL; ++q) p[q] = in[q];
    }
  }
}

// s + (s of the lane whose index differs in bit log2(O)), inside groups of 8 lanes, by data-parallel-primitive moves
// (no LDS traffic).  For O = 4 the partner is lane ^ 7: any lane of the other half of the group holds the same value.
template <int O>
__device__ __forceinline__ float xor_add(float s) {
  constexpr int ctrl = O == 1 ? 0xB1 : (O == 2 ? 0x4E : 0x141);   // quad_perm [1,0,3,2] / [2,3,0,1] / row_half_mirror
  const int other = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), ctrl, 0xF, 0xF, false);
  return s + __builtin_bit_cast(float, other);
}

// Pass 2.  One wave per workgroup; it owns (adapter, CH consecutive output rows) and never waits for another wave.
// B[a] is read as it lies in memory: the block of rows is CH * R * 2 contiguous bytes, fetched by NI load instructions
// of 1 KiB, in which LPR = R / 8 neighbouring lanes hold one row.  A lane multiplies its 8 rank entries, the row's lanes
// add up by butterfly, the row sums cross the wave's LDS buffer, and every lane updates RPL = CH / 64 consecutive y
// elements of a token with one load and one store.  All loads of the block - B (before the table row is back, when
// `speculate` says that most adapters have a token), the y elements of the adapter's first TY tokens, the shrink
// partials - are in flight together.  Summation order = lora_expand_kernel's = row_dot's.
template <int R, typename YT>
__global__ __launch_bounds__(WAVE) void gmm_batch_expand_kernel(BatchArgs a, int blocks_per_adapter, int speculate) {
  constexpr int LPR = R / 8;                   // lanes sharing one row of B
  constexpr int RPI = WAVE / LPR;              // rows per load instruction
  constexpr int NI = 8;                        // load instructions per block
  constexpr int CH = NI * RPI;                 // rows per block
  constexpr int RPL = CH / WAVE;               // consecutive y elements per lane
  constexpr int TY = 4;                        // tokens whose y elements are in flight together
  constexpr int PIECE = RPL * sizeof(YT) > 16 ? 16 / sizeof(YT) : RPL;          // elements per y access
  __shared__ float stage[TY][CH];
  const int ad = blockIdx.x / blocks_per_adapter, blk = blockIdx.x % blocks_per_adapter;
  const int lane = threadIdx.x;
  const int sub = lane % LPR, rloc = lane / LPR;
  const int T = a.T, N = a.N, ldy = a.ldy;
  const int id = lane < T ? a.ids[lane] : -1;
  const GmmSet s = a.sets[blockIdx.y];
  const f16* __restrict__ B = s.B + (size_t)ad * N * R;
  const int n0 = blk * CH;                     // first row of this block
  const f16x8 zero8 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  f16x8 bv[NI];
  if (speculate) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int row = n0 + i * RPI + rloc;
      bv[i] = row < N ? ld8(B + (size_t)row * R + sub * 8) : zero8;
    }
  }
  const unsigned long long mine = __ballot(id == ad);
  if (!mine) return;
  if (!speculate) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int row = n0 + i * RPI + rloc;
      bv[i] = row < N ? ld8(B + (size_t)row * R + sub * 8) : zero8;
    }
  }
  YT* __restrict__ y = (YT*)s.y;
  const float* __restrict__ vset = a.ws + (size_t)blockIdx.y * a.ws_stride;
  const bool vec_ok = (ldy % PIECE == 0) && (((uintptr_t)y) % (PIECE * sizeof(YT)) == 0);
  const int ny = n0 + lane * RPL;              // this lane's y elements ny .. ny + RPL - 1 (N % 8 == 0, RPL | 8: all in or all out)
  unsigned long long todo = mine;
  while (todo) {                               // TY tokens per round; one round unless the adapter has more than TY tokens
    int tok[TY];
#pragma unroll
    for (int u = 0; u < TY; ++u) {
      tok[u] = -1;
      if (todo) {
        tok[u] = __builtin_ctzll(todo);
        todo &= todo - 1;
      }
    }
    float yv[TY][RPL];
#pragma unroll
    for (int u = 0; u < TY; ++u) {
      if (tok[u] >= 0 && ny < N) y_load<YT, RPL>(y + (size_t)tok[u] * ldy + ny, yv[u], vec_ok);
    }
    // v of these tokens, finished by pass 1: a lane takes the 8 rank entries that meet its 8 entries of a row of B
    f32x4 vlo[TY], vhi[TY];
#pragma unroll
    for (int u = 0; u < TY; ++u) {
      if (tok[u] >= 0) {                       // uniform
        const f32x4* vp = reinterpret_cast<const f32x4*>(vset + (size_t)tok[u] * R + sub * 8);
        vlo[u] = vp[0];
        vhi[u] = vp[1];
      }
    }
#pragma unroll
    for (int u = 0; u < TY; ++u) {
      if (tok[u] >= 0) {                       // uniform
        const float v[8] = {vlo[u][0], vlo[u][1], vlo[u][2], vlo[u][3], vhi[u][0], vhi[u][1], vhi[u][2], vhi[u][3]};
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          float sum = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) sum = fmaf((float)bv[i][e], v[e], sum);
          if constexpr (LPR >= 2) sum = xor_add<1>(sum);   // neighbouring groups of 8 first
          if constexpr (LPR >= 4) sum = xor_add<2>(sum);
          if constexpr (LPR >= 8) sum = xor_add<4>(sum);
          if (sub == 0) stage[u][i * RPI + rloc] = sum;
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int u = 0; u < TY; ++u) {
      if (tok[u] >= 0 && ny < N) {
        YT out[RPL];
#pragma unroll
        for (int q = 0; q < RPL; ++q) out[q] = (YT)(yv[u][q] + stage[u][lane * RPL + q]);
        y_store<YT, RPL>(y + (size_t)tok[u] * ldy + ny, out, vec_ok);
      }
    }
    __builtin_amdgcn_wave_barrier();           // the next round overwrites stage
  }
}

template <int R>
void launch_expand(const BatchArgs& a, int n_sets, int y_dtype, int speculate, hipStream_t s) {
  constexpr int CH = 8 * (WAVE / (R / 8));                     // rows per workgroup (see the kernel)
  const int bpa = ceil_div(a.N, CH);                           // workgroups per adapter
  const dim3 grid(a.n_ad * bpa, n_sets);
  if (y_dtype == MLORA_F16) hipLaunchKernelGGL((gmm_batch_expand_kernel<R, f16>), grid, dim3(WAVE), 0, s, a, bpa, speculate);
  else hipLaunchKernelGGL((gmm_batch_expand_kernel<R, float>), grid, dim3(WAVE), 0, s, a, bpa, speculate);
}

}  // namespace

int gmm_batch_stream(const GmmSet* sets, int n_sets, int y_dtype, int ldy, int x_layout, const int32_t* ids, float scaling,
                     int T, int K, int N, int r, int n_ad, float* ws, hipStream_t s) {
  const LoraKSplit ks = lora_k_split(K);
  BatchArgs a = {};
  a.sets = sets;
  a.ids = ids;
  a.ws = ws;
  a.ws_stride = (size_t)T * r;
  a.T = T; a.K = K; a.N = N; a.r = r; a.n_ad = n_ad; a.ci = ks.ci; a.kc = ks.kc;
  a.frag_tt = x_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  a.ldy = ldy;
  a.scaling = scaling;
  // A is requested before the table row has come back when most adapters have a token (one memory round fewer);
  // otherwise only the adapters in use are read.
  int speculate = n_ad <= T / 2;
  const size_t lds = (size_t)ks.kc * T * r * sizeof(float);
  // enough pairs for two or more per compute unit: the persistent form (two partial buffers; its LDS is reserved once)
  static const int n_cu = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cu = 0;
    return cu;
  }();
  static const hipError_t pers_lds =
      hipFuncSetAttribute((const void*)gmm_batch_shrink_pers_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * LORA_MAX_KC * WAVE * 16 * (int)sizeof(float));
  const int pairs_est = n_sets * (n_ad < T ? n_ad : T);
  if (r <= 16 && ks.ci == 1 && n_cu > 0 && pers_lds == hipSuccess && pairs_est >= 2 * n_cu)
    hipLaunchKernelGGL(gmm_batch_shrink_pers_kernel, dim3(n_cu), dim3(ks.kc * WAVE), 2 * lds, s, a, n_sets);
  else if (r <= 16 && ks.ci == 1) hipLaunchKernelGGL(gmm_batch_shrink_kernel<true>, dim3(n_ad, n_sets), dim3(ks.kc * WAVE), lds, s, a, speculate);
  else hipLaunchKernelGGL(gmm_batch_shrink_kernel<false>, dim3(n_ad, n_sets), dim3(ks.kc * WAVE), lds, s, a, 0);
  switch (r) {
    case 8: launch_expand<8>(a, n_sets, y_dtype, speculate, s); break;
    case 16: launch_expand<16>(a, n_sets, y_dtype, speculate, s); break;
    case 32: launch_expand<32>(a, n_sets, y_dtype, speculate, s); break;
    default: launch_expand<64>(a, n_sets, y_dtype, speculate, s); break;
  }
  return mlora_launch_status("gather_mm_batch");
}
