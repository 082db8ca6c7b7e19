// Decode-time base linear for gfx950:  y[T, N] (=|+=) x[T, K] . W[N, K]^T  with T <= 64.
//
// The weight matrix is read exactly once, straight from HBM into MFMA operand registers: for
// v_mfma_f32_16x16x32_f16 a lane holds 8 consecutive k of one row.  The token block x (T x K fp16,
// L2-resident) is the other operand, so one weight fragment is applied to 16 tokens per MFMA and the
// kernel stays HBM-bound (32 tokens need 64 flop per weight element - beyond the vector ALUs, well
// inside the matrix cores).  A workgroup of 8 waves owns 16*NT rows of W and splits K eight ways;
// partial tiles are summed in a fixed order through LDS, so results do not depend on scheduling.
//
// Two weight layouts:
//   row-major W[N, K]  - a wave-wide 16-byte load covers 16 rows x 64 bytes (one DRAM page each);
//   packed (mlora_pack_weight) - fragments are stored in operand order,
//       Wp[n/16][k/32][(k%32)/8][n%16][k%8],
//     so the fragment of (16 rows, 32 k) is one contiguous 1 KiB block and a wave streams consecutive
//     blocks: every load is a full DRAM page and consecutive k-steps are consecutive addresses.
#include "lora_device.h"

namespace {

constexpr int GEMV_WAVES = 8;
constexpr int KSTEP = 32;   // k per MFMA

enum { OUT_F16 = 0, OUT_F32 = 1, OUT_ACC_F32 = 2, OUT_SILU_FRAG = 3 };

// v / d for a uniform divisor 1..4 (the slice counts of a launch): shifts and one multiply instead of the division
// sequences - a hundred scalar instructions each, three times over - that stood before a workgroup's first load
__device__ __forceinline__ int udiv_le4(int v, int d) {
  const unsigned u = (unsigned)v;
  return (int)(d == 4 ? u >> 2 : d == 3 ? u / 3u : d == 2 ? u >> 1 : u);
}

// The expand of a LoRA delta by workgroups that ride at the front of an accumulating GEMV launch.  The shrink results
// come as `n_vpart` shares per (token, rank entry) - vpart [n_vpart, T, r] fp32, e.g. one share per attention head from
// the kernel that produced the launch's token block - which rider (t, part) adds in a fixed order before it writes
// delta[t][c] = scaling * B[id_t][c] . v for its share of the N columns into `out` [T, N] fp32 (zeros for a token
// without adapter): a row block that the reader of y adds like a K-slice partial.  The GEMV's own rows stay the base
// weight (no appended adapter rows), and the norm that follows has no table to stream - its B rows arrive here, a few
// KiB per rider, under the shadow of the weight stream.
struct LoraDeltaRide {
  const float* vpart;   // [n_vpart, T, r]
  const f16* B;         // [n_ad, N, r]
  const int32_t* ids;   // [T]
  float* out;           // [T, N]
  float scaling;
  int n_vpart, T, N, r, n_ad, per_token;
  int accumulate;       // out[t, :] += delta for the tokens that have an adapter, others untouched (the stand-alone launch)
};

constexpr int RIDE_BQ = 2;     // 16-byte chunks of B per rider thread: a rider is short, and there are many of them
constexpr int SOLO_BQ = 8;     // ... and per thread of the stand-alone launch: one round of fewer, larger workgroups

template <int BQ>
__device__ __forceinline__ void lora_delta_ride(const LoraDeltaRide& d, int unit, float* __restrict__ lds) {
  constexpr int NTH = GEMV_WAVES * WAVE;
  const int tid = threadIdx.x;
  const int t = unit / d.per_token, part = unit - t * d.per_token;
  const int ncol = d.N / d.per_token, c0 = part * ncol;
  float* __restrict__ out = d.out + (size_t)t * d.N + c0;
  const int id = d.ids[t];                                   // uniform
  if (id < 0 || id >= d.n_ad) {
    if (!d.accumulate)
      for (int c = tid * 4; c < ncol; c += NTH * 4) *reinterpret_cast<f32x4*>(out + c) = f32x4{0.f, 0.f, 0.f, 0.f};
    return;
  }
  const int r = d.r, lpr = r >> 3;                           // 16-byte chunks per row of B
  const int nq = ncol * lpr;                                 // chunks of this rider's rows of B: at most BQ per thread
  // one round of requests: the rider's rows of B (uniform base + 32-bit lane offset) and the shares of v
  f16x8 bv[BQ];
  const f16* __restrict__ Bp = d.B + ((size_t)id * d.N + c0) * r;
#pragma unroll
  for (int u = 0; u < BQ; ++u) {
    const int q = u * NTH + tid;
    bv[u] = ld8(Bp + (unsigned)((q < nq ? q : 0) * 8));
  }
  // the row's old values, where the deltas are added in place: requested with everything else
  const int csub = tid % lpr;                                // a thread's chunks all cover ranks 8 csub .. (512 % lpr == 0)
  float yold[BQ];
#pragma unroll
  for (int u = 0; u < BQ; ++u) {
    const int q = u * NTH + tid;
    yold[u] = d.accumulate && csub == 0 && q < nq ? out[q / lpr] : 0.f;
  }
  // v[j] = scaling * sum of the shares: thread e = h r + j takes the shares h, h + 512 / r, ... of entry j (512 % r == 0),
  // the lanes of a wave that hold the same j add up by shuffles, the eight waves' sums meet in LDS - a fixed order
  float* __restrict__ wsum = lds;                            // [8][r], then v [r]
  float* __restrict__ lv = lds + GEMV_WAVES * r;
  float a = 0.f;
  for (int e = tid; e < d.n_vpart * r; e += NTH) {
    const int h = e / r, jj = e - h * r;
    a += d.vpart[((size_t)h * d.T + t) * r + jj];
  }
  for (int o = r; o < WAVE; o <<= 1) a += __shfl_xor(a, o, WAVE);
  if ((tid & (WAVE - 1)) < r) wsum[(tid >> 6) * r + (tid & (WAVE - 1))] = a;
  __syncthreads();
  if (tid < r) {
    float sum = wsum[tid];
#pragma unroll
    for (int w = 1; w < GEMV_WAVES; ++w) sum += wsum[w * r + tid];
    lv[tid] = sum * d.scaling;
  }
  __syncthreads();
  float lvr[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) lvr[e] = lv[csub * 8 + e];
#pragma unroll
  for (int u = 0; u < BQ; ++u) {
    const int q = u * NTH + tid;
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) sum = fmaf((float)bv[u][e], lvr[e], sum);
    for (int o = 1; o < lpr; o <<= 1) sum += __shfl_xor(sum, o, WAVE);
    if (csub == 0 && q < nq) out[q / lpr] = yold[u] + sum;
  }
}

// the riders as a launch of their own (token blocks beyond what the decode GEMV serves): y[t, :] += delta
__global__ __launch_bounds__(GEMV_WAVES* WAVE) void lora_expand_shares_kernel(LoraDeltaRide d) {
  __shared__ float lds[(GEMV_WAVES + 1) * 64];
  lora_delta_ride<SOLO_BQ>(d, blockIdx.x, lds);
}

// With SHRINK the first `shrink_blocks` workgroups of the launch do LoRA shrink units (one per wave) on the same
// x instead of a GEMV tile: the adapter work rides in the GEMV launch and finishes long before it does.
// An accumulating launch without shrink units may instead carry `ride_blocks` delta riders (lora_delta_ride).
template <int NT, int TT, int OUT, bool PACKED, bool XFRAG, bool SHRINK, int PIPE = 4>   // PIPE: k-steps in flight per wave
__global__ __launch_bounds__(GEMV_WAVES* WAVE, (NT * TT > 8 ? 2 : 4)) void gemv_kernel(void* __restrict__ yv, const f16* __restrict__ x, int ldx,
                                                                const f16* __restrict__ W, int T, int K, int N,
                                                                LoraShrinkBatch sb, int shrink_blocks, int n_main,
                                                                float* __restrict__ y2, int ksplit, float* __restrict__ part,
                                                                LoraDeltaRide dr, int ride_blocks) {
  constexpr int TILES = NT * TT;
  constexpr int HT = TILES > 8 ? TILES / 2 : TILES;   // accumulator tiles summed per pass through LDS (64 KiB holds 8)
  constexpr bool RIDE = OUT == OUT_ACC_F32 && PACKED && XFRAG && !SHRINK;   // the launches that may carry delta riders
  __shared__ f32x4 red[GEMV_WAVES][HT][WAVE];
  // all arguments in one round of scalar loads, ahead of the first weight request (the compiler would fetch each
  // group at its first use, a dependent round each time)
  asm volatile("" ::"s"(yv), "s"(x), "s"(ldx), "s"(W), "s"(T), "s"(K), "s"(N), "s"(shrink_blocks), "s"(n_main), "s"(y2), "s"(ksplit), "s"(part));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: keeps the k-loop control scalar
  const int lane = threadIdx.x & 63;
  int bid = blockIdx.x;
  if constexpr (RIDE) {
    if (bid < ride_blocks) {                       // uniform
      lora_delta_ride<RIDE_BQ>(dr, bid, reinterpret_cast<float*>(&red[0][0][0]));
      return;
    }
    bid -= ride_blocks;
  }
  if constexpr (SHRINK) {
    if (bid < shrink_blocks) {
      const int unit = bid * GEMV_WAVES + wave;
      if (unit < sb.n_proj * sb.n_ad * sb.kc) lora_shrink_unit(sb, unit, lane);
      return;
    }
    bid -= shrink_blocks;
  }
  // K split over `ksplit` consecutive workgroups: slice 0 runs the normal epilogue, slice s > 0 stores its fp32
  // partial tile to part[s - 1][t][n]; whoever reads y next adds the partials in slice order.
  int slice = 0;
  if (ksplit > 1) {
    const int q = udiv_le4(bid, ksplit);
    slice = bid - q * ksplit;
    bid = q;
  }
  const int r16 = lane & 15;
  const int kg = lane >> 4;
  const int n0 = bid * (16 * NT);
  const int KB = K / KSTEP;
  constexpr int WSTEP = PACKED ? 512 : KSTEP;   // elements between consecutive k-steps of one fragment stream

  const f16* wp[PACKED ? 1 : NT];
  int woff[NT];                                    // packed: element offset of tile i from the block's first tile (uniform)
  const f16* xp[TT];
  if constexpr (PACKED) wp[0] = W + ((size_t)bid * NT * KB) * 512 + lane * 8;
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    if constexpr (PACKED) {
      // a tile past the end repeats the block's first tile and is not stored
      woff[i] = ((bid * NT + i) * 16 < N ? i : 0) * KB * 512;
    } else {
      woff[i] = 0;
      int n = n0 + i * 16 + r16;
      n = n < N ? n : N - 1;
      wp[i] = W + (size_t)n * K + kg * 8;
    }
  }
  constexpr int XSTEP = XFRAG ? TT * 512 : KSTEP;   // elements between consecutive k-steps of the x fragments
#pragma unroll
  for (int j = 0; j < TT; ++j) {
    if constexpr (XFRAG) {
      xp[j] = x + j * 512 + lane * 8;
    } else {
      int t = j * 16 + r16;
      t = t < T ? t : T - 1;
      xp[j] = x + (size_t)t * ldx + kg * 8;
    }
  }

  f32x4 acc[NT][TT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // wave w takes k-steps w, w + 8, w + 16, ...; stage s of this wave is k-step w + 8 s.
  // PIPE stages are always in flight: each buffer is refilled right after it is consumed.
  const int kb0 = ksplit > 1 ? udiv_le4(slice * KB, ksplit) : 0;
  const int kb1 = ksplit > 1 ? udiv_le4((slice + 1) * KB, ksplit) : KB;
  const int S = (kb1 - kb0 - wave + GEMV_WAVES - 1) / GEMV_WAVES;
  f16x8 a[PIPE][NT], b[PIPE][TT];
  auto load_stage = [&](int u, int s) {
    const bool in = s < S;
    const int ks = in ? kb0 + wave + GEMV_WAVES * s : 0;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      a[u][i] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(wp[PACKED ? 0 : i] + (woff[i] + ks * WSTEP)));
      if (!in) a[u][i] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < TT; ++j) b[u][j] = ld8(xp[j] + (size_t)ks * XSTEP);
  };
#pragma unroll
  for (int u = 0; u < PIPE; ++u) load_stage(u, u);
  for (int s0 = 0; s0 < S; s0 += PIPE) {
#pragma unroll
    for (int u = 0; u < PIPE; ++u) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
      load_stage(u, s0 + u + PIPE);
    }
  }

  if constexpr (OUT == OUT_SILU_FRAG) {
    // The weight interleaves 16-row tiles of gate and up, so this block's two tiles are gate rows c..c+15 and up
    // rows c..c+15 of the same channels: out[t, c + ..] = silu(f16(gate)) * f16(up), written in fragment order.
    static_assert(NT % 2 == 0 && TILES <= 8, "the SiLU epilogue pairs a gate tile with an up tile and sums all tiles in one pass");
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int j = 0; j < TT; ++j) red[wave][i * TT + j][lane] = acc[i][j];
    __syncthreads();
    for (int e = threadIdx.x; e < (NT / 2) * TT * WAVE; e += GEMV_WAVES * WAVE) {
      const int pj = e >> 6, sl = e & 63;
      const int p = pj / TT, j = pj % TT;         // tile pair (gate tile 2p, up tile 2p + 1), token tile j
      f32x4 sg = red[0][2 * p * TT + j][sl], su = red[0][(2 * p + 1) * TT + j][sl];
#pragma unroll
      for (int w = 1; w < GEMV_WAVES; ++w) {
        sg += red[w][2 * p * TT + j][sl];
        su += red[w][(2 * p + 1) * TT + j][sl];
      }
      const int c = (bid * (NT / 2) + p) * 16 + (sl >> 4) * 4;   // output channel of the first of this lane's 4 rows
      const int t = j * 16 + (sl & 15);
      if (t < T && c < N / 2) {
        f16x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float gf = (float)(f16)sg[q];
          o[q] = (f16)(gf / (1.f + expf(-gf)) * (float)(f16)su[q]);
        }
        *reinterpret_cast<f16x4*>((f16*)yv + frag_offset(t, c, TT)) = o;
      }
    }
    return;
  }
  // The waves' partial tiles are summed through LDS, in wave order, HT tiles per pass: thread e sums tile h0 + e / 64,
  // lane slot e % 64.
  for (int h0 = 0; h0 < TILES; h0 += HT) {
    if (h0 > 0) __syncthreads();
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int j = 0; j < TT; ++j) {
        const int tile = i * TT + j;               // compile-time
        if (tile >= h0 && tile < h0 + HT) red[wave][tile - h0][lane] = acc[i][j];
      }
    __syncthreads();
    for (int e = threadIdx.x; e < HT * WAVE; e += GEMV_WAVES * WAVE) {
      const int lt = e >> 6, sl = e & 63;
      f32x4 s = red[0][lt][sl];
#pragma unroll
      for (int w = 1; w < GEMV_WAVES; ++w) s += red[w][lt][sl];
      const int tile = h0 + lt;
      const int i = tile / TT, j = tile % TT;
      const int n = n0 + i * 16 + (sl >> 4) * 4;   // D[n][t]: lane holds rows 4*(lane/16)..+3, column lane%16
      const int t = j * 16 + (sl & 15);
      if (slice > 0) {                             // a K slice other than the first: fp32 partial, summed by the reader of y
        if (t < T && n < N) *reinterpret_cast<f32x4*>(part + ((size_t)(slice - 1) * T + t) * N + n) = s;
      } else if (t < T && n >= n_main && n < N) {
        // rows past n_main are a second result block (adapter shrink rows appended to the weight): fp32, own buffer
        *reinterpret_cast<f32x4*>(y2 + (size_t)t * (N - n_main) + (n - n_main)) = s;
      } else if (t < T && n < N) {                 // N % 4 == 0: the 4 rows are inside together
        const size_t o = (size_t)t * n_main + n;
        if constexpr (OUT == OUT_F16) {
          *reinterpret_cast<f16x4*>((f16*)yv + o) = f16x4{(f16)s[0], (f16)s[1], (f16)s[2], (f16)s[3]};
        } else if constexpr (OUT == OUT_F32) {
          *reinterpret_cast<f32x4*>((float*)yv + o) = s;
        } else if constexpr (OUT == OUT_ACC_F32) {
          f32x4* p = reinterpret_cast<f32x4*>((float*)yv + o);
          *p = *p + s;
        }
      }
    }
  }
}

// Gate/up GEMV with the SiLU epilogue as ONE workgroup per compute unit.  A unit takes in first-level-cache fills at a
// bounded rate, weights and token block together, so a launch is as fast as its most loaded unit: here every unit gets
// an equal share of the (gate tile, up tile) pairs - NP or NP - 1 of them - and reads the token block once for all of
// them, instead of once per pair.  Same k-split over the 8 waves and the same fixed-order reduction as gemv_kernel, so
// the result bits are the same.  The reduction goes through LDS one pair at a time.
template <int NP, int TT, int PIPE>
__global__ __launch_bounds__(GEMV_WAVES* WAVE, 2) void gemv_silu_cu_kernel(f16* __restrict__ act, const f16* __restrict__ x,
                                                                        const f16* __restrict__ W, int T, int K, int I,
                                                                        int base, int rem) {
  constexpr int NT = 2 * NP;
  __shared__ f32x4 red[GEMV_WAVES][2 * TT][WAVE];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int wg = blockIdx.x;
  const int p0 = wg * base + (wg < rem ? wg : rem);    // first pair of this workgroup
  const int np = base + (wg < rem ? 1 : 0);            // and how many it has
  const int KB = K / KSTEP;
  const f16* wp = W + ((size_t)(2 * p0) * KB) * 512 + lane * 8;
  int woff[NT];                                        // a missing last pair repeats the first tile (cache hits) and is not stored
#pragma unroll
  for (int i = 0; i < NT; ++i) woff[i] = (i < 2 * np ? i : 0) * KB * 512;
  const f16* xp = x + lane * 8;
  constexpr int XSTEP = TT * 512;

  f32x4 acc[NT][TT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int S = (KB - wave + GEMV_WAVES - 1) / GEMV_WAVES;
  f16x8 a[PIPE][NT], b[PIPE][TT];
  auto load_stage = [&](int u, int s) {
    const bool in = s < S;
    const int ks = in ? wave + GEMV_WAVES * s : 0;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      a[u][i] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(wp + (woff[i] + ks * 512)));
      if (!in) a[u][i] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < TT; ++j) b[u][j] = ld8(xp + j * 512 + (size_t)ks * XSTEP);
  };
#pragma unroll
  for (int u = 0; u < PIPE; ++u) load_stage(u, u);
  for (int s0 = 0; s0 < S; s0 += PIPE) {
#pragma unroll
    for (int u = 0; u < PIPE; ++u) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
      load_stage(u, s0 + u + PIPE);
    }
  }
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    if (p < np) {                                      // workgroup-uniform
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < TT; ++j) red[wave][h * TT + j][lane] = acc[2 * p + h][j];
      __syncthreads();
      for (int e = threadIdx.x; e < TT * WAVE; e += GEMV_WAVES * WAVE) {
        const int j = e >> 6, sl = e & 63;
        f32x4 sg = red[0][j][sl], su = red[0][TT + j][sl];
#pragma unroll
        for (int w = 1; w < GEMV_WAVES; ++w) {
          sg += red[w][j][sl];
          su += red[w][TT + j][sl];
        }
        const int c = (p0 + p) * 16 + (sl >> 4) * 4;   // output channel of the first of this lane's 4 rows
        const int t = j * 16 + (sl & 15);
        if (t < T && c < I) {
          f16x4 o;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float gf = (float)(f16)sg[q];
            o[q] = (f16)(gf / (1.f + expf(-gf)) * (float)(f16)su[q]);
          }
          *reinterpret_cast<f16x4*>(act + frag_offset(t, c, TT)) = o;
        }
      }
      __syncthreads();
    }
  }
}

// GEMV over a weight with appended shrink rows (q/k/v + the stacked A tables) as ONE workgroup per compute unit.
// The main row tiles are dealt out evenly (NM or NM - 1 per unit); the few appended tiles are cut into kq ranges of K
// and every (tile, range) piece goes to a unit of its own, starting with the units that got one main tile fewer, so
// that no unit takes in more than NM tiles plus a 1/kq piece - with whole appended tiles in the deal, the units that
// drew one would set the time of the launch.  A piece's fp32 partial goes to block `range` of y2 [kq][T][n_ext];
// whoever reads the shrink results adds the blocks in range order.  Main rows: f16 store, the k order and the wave
// reduction of gemv_kernel, hence its bits.
template <int NM, int TT, int PIPE>
__global__ __launch_bounds__(GEMV_WAVES* WAVE, 2) void gemv_split_cu_kernel(f16* __restrict__ y, float* __restrict__ y2,
                                                                         const f16* __restrict__ x, const f16* __restrict__ W,
                                                                         int T, int K, int n_main, int n_ext, int base, int rem,
                                                                         int kq, int n_wg) {   // n_wg: the grid size, as an argument (gridDim comes from a later scalar load)
  constexpr int NT = NM + 1;                           // register tile NM is the piece of an appended tile
  __shared__ f32x4 red[GEMV_WAVES][TT][WAVE];
  asm volatile("" ::"s"(y), "s"(y2), "s"(x), "s"(W), "s"(T), "s"(K), "s"(n_main), "s"(n_ext), "s"(base), "s"(rem), "s"(kq), "s"(n_wg));   // all arguments (and the grid size) in one round of scalar loads
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int wg = blockIdx.x;
  const int m0 = wg * base + (wg < rem ? wg : rem);    // first main tile of this workgroup
  const int nm = base + (wg < rem ? 1 : 0);            // and how many it has
  const int KB = K / KSTEP;
  const int piece = n_wg - 1 - wg;                     // pieces are dealt from the last unit backwards
  const bool has_ext = piece < (n_ext / 16) * kq;
  const int et = has_ext ? udiv_le4(piece, kq) : 0, eq = has_ext ? piece - et * kq : 0;
  const int ekb0 = has_ext ? udiv_le4(eq * KB, kq) : 0, ekb1 = has_ext ? udiv_le4((eq + 1) * KB, kq) : 0;
  const f16* wp = W + lane * 8;
  size_t woff[NT];                                     // a missing main tile repeats the first one (cache hits) and is not stored
#pragma unroll
  for (int i = 0; i < NM; ++i) woff[i] = (size_t)(m0 + (i < nm ? i : 0)) * KB * 512;
  woff[NM] = (size_t)(n_main / 16 + et) * KB * 512;
  const f16* xp = x + lane * 8;
  constexpr int XSTEP = TT * 512;

  f32x4 acc[NT][TT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int S = (KB - wave + GEMV_WAVES - 1) / GEMV_WAVES;
  f16x8 a[PIPE][NT], b[PIPE][TT];
  auto load_stage = [&](int u, int s) {
    const bool in = s < S;
    const int ks = in ? wave + GEMV_WAVES * s : 0;
#pragma unroll
    for (int i = 0; i < NM; ++i) {
      a[u][i] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(wp + (woff[i] + (size_t)ks * 512)));
      if (!in) a[u][i] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
    a[u][NM] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (in && ks >= ekb0 && ks < ekb1)                 // wave-uniform: the piece covers only its range of K
      a[u][NM] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(wp + (woff[NM] + (size_t)ks * 512)));
#pragma unroll
    for (int j = 0; j < TT; ++j) b[u][j] = ld8(xp + j * 512 + (size_t)ks * XSTEP);
  };
#pragma unroll
  for (int u = 0; u < PIPE; ++u) load_stage(u, u);
  for (int s0 = 0; s0 < S; s0 += PIPE) {
#pragma unroll
    for (int u = 0; u < PIPE; ++u) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
      load_stage(u, s0 + u + PIPE);
    }
  }
  // the waves' sums, one register tile at a time, added in wave order
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const bool live = i < NM ? i < nm : has_ext;       // workgroup-uniform
    if (live) {
#pragma unroll
      for (int j = 0; j < TT; ++j) red[wave][j][lane] = acc[i][j];
      __syncthreads();
      for (int e = threadIdx.x; e < TT * WAVE; e += GEMV_WAVES * WAVE) {
        const int j = e >> 6, sl = e & 63;
        f32x4 s = red[0][j][sl];
#pragma unroll
        for (int w = 1; w < GEMV_WAVES; ++w) s += red[w][j][sl];
        const int t = j * 16 + (sl & 15);
        if (t < T) {
          if (i < NM) {
            const int n = (m0 + i) * 16 + (sl >> 4) * 4;
            *reinterpret_cast<f16x4*>(y + (size_t)t * n_main + n) = f16x4{(f16)s[0], (f16)s[1], (f16)s[2], (f16)s[3]};
          } else {
            const int n = et * 16 + (sl >> 4) * 4;
            *reinterpret_cast<f32x4*>(y2 + ((size_t)eq * T + t) * n_ext + n) = s;
          }
        }
      }
      __syncthreads();
    }
  }
}

// one thread per 16-byte chunk of the packed array
__global__ __launch_bounds__(256) void pack_weight_kernel(f16* __restrict__ dst, const f16* __restrict__ src, int N, int K,
                                                          size_t chunks) {
  const size_t c = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= chunks) return;
  const int KB = K / KSTEP;
  const int row = c & 15;
  const int g = (c >> 4) & 3;
  const size_t blk = c >> 6;
  const int ks = blk % KB;
  const size_t nt = blk / KB;
  const size_t n = nt * 16 + row;
  f16x8 v = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  if (n < (size_t)N) v = ld8(src + n * K + ks * KSTEP + g * 8);
  st8(dst + c * 8, v);
}

// one thread per 16-byte chunk of the fragment-ordered activation block
__global__ __launch_bounds__(256) void pack_activation_kernel(f16* __restrict__ dst, const f16* __restrict__ src, int ldsrc,
                                                              int T, int K, int TT, int chunks) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= chunks) return;
  const int t16 = c & 15, kg = (c >> 4) & 3, blk = c >> 6;
  const int tt = blk % TT, ks = blk / TT;
  const int t = tt * 16 + t16;
  f16x8 v = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  if (t < T) v = ld8(src + (size_t)t * ldsrc + ks * KSTEP + kg * 8);
  st8(dst + (size_t)c * 8, v);
}

template <int NT, int TT, bool PACKED, bool XFRAG, bool SHRINK, int PIPE = 4>
void launch_gemv(void* y, int out, const f16* x, int ldx, const f16* W, int T, int K, int N, hipStream_t s,
                 const LoraShrinkBatch& sb, int n_main, float* y2, int ksplit = 1, float* part = nullptr,
                 const LoraDeltaRide& dr = LoraDeltaRide(), int rblocks = 0) {
  const int sblocks = SHRINK ? ceil_div(lora_shrink_units(sb), GEMV_WAVES) : 0;
  const dim3 grid(ceil_div(N, 16 * NT) * ksplit + sblocks + rblocks), block(GEMV_WAVES * WAVE);
  if (out == OUT_F16) hipLaunchKernelGGL((gemv_kernel<NT, TT, OUT_F16, PACKED, XFRAG, SHRINK, PIPE>), grid, block, 0, s, y, x, ldx, W, T, K, N, sb, sblocks, n_main, y2, ksplit, part, dr, 0);
  else if (out == OUT_F32) hipLaunchKernelGGL((gemv_kernel<NT, TT, OUT_F32, PACKED, XFRAG, SHRINK, PIPE>), grid, block, 0, s, y, x, ldx, W, T, K, N, sb, sblocks, n_main, y2, ksplit, part, dr, 0);
  else hipLaunchKernelGGL((gemv_kernel<NT, TT, OUT_ACC_F32, PACKED, XFRAG, SHRINK, PIPE>), grid, block, 0, s, y, x, ldx, W, T, K, N, sb, sblocks, n_main, y2, ksplit, part, dr, rblocks);
}

// Rows per workgroup.  Every workgroup reads the whole token block, so its L2 traffic is T / (16 NT) of the weight
// traffic and the time of a launch follows the most loaded compute unit: wide matrices (>= 768 tiles) take four tiles
// per wave, which keeps one or two equal workgroups on every unit; narrow ones one tile (or, with a partials buffer,
// four tiles and a K split - see mlora_gemv_ksplit).
// compute units of the current device (0 if it cannot be asked), read once
int gemv_n_cu() {
  static const int n_cu = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cu = 0;
    return cu;
  }();
  return n_cu;
}

template <bool PACKED, bool XFRAG, bool SHRINK = false>
int gemv_dispatch(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W, int T, int K, int N, void* stream,
                  const LoraShrinkBatch& sb = LoraShrinkBatch(), int n_main = -1, float* y2 = nullptr, int ksplit = 1,
                  float* part = nullptr, const LoraDeltaRide& dr = LoraDeltaRide(), int rblocks = 0) {
  if (n_main < 0) n_main = N;
  const int out = mode == MLORA_ACCUMULATE ? OUT_ACC_F32 : (y_dtype == MLORA_F32 ? OUT_F32 : OUT_F16);
  hipStream_t s = (hipStream_t)stream;
  const f16* xp = (const f16*)x;
  const f16* Wp = (const f16*)W;
  const int tiles = ceil_div(N, 16);
  if constexpr (PACKED && XFRAG) {
    if (T <= 32 && (ksplit > 1 || tiles >= 768)) {
      // three tiles per workgroup where that gives every compute unit exactly one workgroup's worth or less (768 tiles on
      // 256 units: with four tiles a quarter of the units would stay idle and the others set the time); same bits
      const int n_cu = gemv_n_cu();
      if (ksplit == 1 && n_cu > 0 && tiles % 3 == 0 && tiles / 3 <= n_cu && ceil_div(tiles, 4) < tiles / 3) {
        if (T <= 16) launch_gemv<3, 1, PACKED, XFRAG, SHRINK, 4>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2, ksplit, part);
        else launch_gemv<3, 2, PACKED, XFRAG, SHRINK, 4>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2, ksplit, part);
        return mlora_launch_status("gemv");
      }
      if (T <= 16) launch_gemv<4, 1, PACKED, XFRAG, SHRINK, 4>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2, ksplit, part, dr, rblocks);
      else launch_gemv<4, 2, PACKED, XFRAG, SHRINK, 3>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2, ksplit, part, dr, rblocks);
      return mlora_launch_status("gemv");
    }
  }
  // two 16-row tiles per wave once there are enough rows to give every CU a workgroup; the packed
  // layout pads N to a multiple of 16, so an odd tile count keeps one tile per wave
  // (just above 256 tiles, one tile per workgroup would leave a second, nearly empty round of workgroups)
  const bool wide = (tiles >= 512 && (!PACKED || tiles % 2 == 0)) || (PACKED && tiles > 256 && tiles < 512);
  if (T <= 16) {
    if (wide) launch_gemv<2, 1, PACKED, XFRAG, SHRINK>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2);
    else launch_gemv<1, 1, PACKED, XFRAG, SHRINK>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2);
  } else if (T <= 32) {
    if (wide) launch_gemv<2, 2, PACKED, XFRAG, SHRINK>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2);
    else launch_gemv<1, 2, PACKED, XFRAG, SHRINK>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2);
  } else {
    // 33..64 tokens: four token tiles leave registers for two row tiles per wave (x traffic is then twice the weight
    // traffic instead of four times): 5.3 -> 4.4 ms of GEMV per decode step at T = 64
    if constexpr (PACKED && XFRAG) {
      if (ksplit > 1 || tiles >= 768) {           // one workgroup per unit with four row tiles: the token block is read once per unit
        launch_gemv<4, 4, PACKED, XFRAG, SHRINK, 2>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2, ksplit, part, dr, rblocks);
        return mlora_launch_status("gemv");
      }
      if (tiles > 256) {                          // 257..511 tiles as one-tile workgroups would need a second, thin round
        launch_gemv<2, 4, PACKED, XFRAG, SHRINK, 2>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2, ksplit, part);
        return mlora_launch_status("gemv");
      }
    }
    launch_gemv<1, 4, PACKED, XFRAG, SHRINK>(y, out, xp, ldx, Wp, T, K, N, s, sb, n_main, y2);
  }
  return mlora_launch_status("gemv");
}

}  // namespace

int mlora_check_linear(const char* who, const void* y, int y_dtype, int mode, const void* x, int ldx, const void* W,
                       int T, int K, int N) {
  MLORA_CHECK(y && x && W, MLORA_ERR_INVALID, "%s: null pointer", who);
  MLORA_CHECK(T >= 0 && K > 0 && N > 0 && ldx >= K, MLORA_ERR_INVALID, "%s: bad shape T=%d K=%d N=%d ldx=%d", who, T, K, N, ldx);
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "%s: bad y_dtype %d", who, y_dtype);
  MLORA_CHECK(mode == MLORA_STORE || mode == MLORA_ACCUMULATE, MLORA_ERR_INVALID, "%s: bad mode %d", who, mode);
  MLORA_CHECK(mode == MLORA_STORE || y_dtype == MLORA_F32, MLORA_ERR_UNSUPPORTED, "%s: accumulate needs an fp32 y", who);
  MLORA_CHECK(K % 32 == 0 && N % 4 == 0 && ldx % 8 == 0, MLORA_ERR_UNSUPPORTED,
              "%s: need K %% 32 == 0, N %% 4 == 0, ldx %% 8 == 0 (K=%d N=%d ldx=%d)", who, K, N, ldx);
  return MLORA_OK;
}

extern "C" int mlora_gemv(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W, int T, int K, int N,
                          void* stream) {
  if (int e = mlora_check_linear("gemv", y, y_dtype, mode, x, ldx, W, T, K, N)) return e;
  MLORA_CHECK(T <= 64, MLORA_ERR_UNSUPPORTED, "gemv: T=%d exceeds 64 (use mlora_gemm)", T);
  if (T == 0) return MLORA_OK;
  return gemv_dispatch<false, false>(y, y_dtype, mode, x, ldx, W, T, K, N, stream);
}

extern "C" int mlora_gemv_packed(void* y, int y_dtype, int mode, const void* x, int ldx, const void* Wp, int T, int K,
                                 int N, void* stream) {
  if (int e = mlora_check_linear("gemv_packed", y, y_dtype, mode, x, ldx, Wp, T, K, N)) return e;
  MLORA_CHECK(T <= 64, MLORA_ERR_UNSUPPORTED, "gemv_packed: T=%d exceeds 64 (use mlora_gemm_packed)", T);
  if (T == 0) return MLORA_OK;
  return gemv_dispatch<true, false>(y, y_dtype, mode, x, ldx, Wp, T, K, N, stream);
}

extern "C" int mlora_gemv_frag(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N,
                               void* stream) {
  if (int e = mlora_check_linear("gemv_frag", y, y_dtype, mode, xf, K, Wp, T, K, N)) return e;
  MLORA_CHECK(T <= 64, MLORA_ERR_UNSUPPORTED, "gemv_frag: T=%d exceeds 64", T);
  if (T == 0) return MLORA_OK;
  return gemv_dispatch<true, true>(y, y_dtype, mode, xf, K, Wp, T, K, N, stream);
}

static int check_shrink_args(const char* who, const void* v_part, const void* const* A, int n_proj, const int32_t* tok_adapter,
                             int r, int n_ad) {
  MLORA_CHECK(n_proj >= 1 && n_proj <= LORA_MAX_PROJ && v_part && A && tok_adapter, MLORA_ERR_INVALID,
              "%s: need 1..%d projections and non-null LoRA arguments", who, LORA_MAX_PROJ);
  MLORA_CHECK((r == 8 || r == 16 || r == 32 || r == 64) && n_ad > 0 && n_ad <= 65535, MLORA_ERR_UNSUPPORTED,
              "%s: rank %d not in {8,16,32,64} or bad n_ad %d", who, r, n_ad);
  return MLORA_OK;
}

static LoraShrinkBatch shrink_batch(const void* xf, void* v_part, const void* const* A, int n_proj, const int32_t* tok_adapter,
                                    int T, int K, int r, int n_ad) {
  const LoraKSplit ks = lora_k_split(K);
  LoraShrinkBatch b = {};
  for (int i = 0; i < n_proj; ++i) b.A[i] = (const f16*)A[i];   // a null slot is skipped
  b.n_proj = n_proj;
  b.vpart = (float*)v_part;
  b.x = (const f16*)xf;
  b.ids = tok_adapter;
  b.T = T; b.K = K; b.r = r; b.n_ad = n_ad; b.ci = ks.ci; b.kc = ks.kc;
  b.frag_tt = mlora_frag_tiles(T);
  b.speculate = n_ad <= 2 * T;
  return b;
}

extern "C" int mlora_gemv_frag_lora(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N,
                                    void* v_part, const void* const* A, int n_proj, const int32_t* tok_adapter, int r,
                                    int n_ad, void* stream) {
  if (int e = mlora_check_linear("gemv_frag_lora", y, y_dtype, mode, xf, K, Wp, T, K, N)) return e;
  MLORA_CHECK(T <= 64, MLORA_ERR_UNSUPPORTED, "gemv_frag_lora: T=%d exceeds 64", T);
  if (int e = check_shrink_args("gemv_frag_lora", v_part, A, n_proj, tok_adapter, r, n_ad)) return e;
  if (T == 0) return MLORA_OK;
  return gemv_dispatch<true, true, true>(y, y_dtype, mode, xf, K, Wp, T, K, N, stream,
                                         shrink_batch(xf, v_part, A, n_proj, tok_adapter, T, K, r, n_ad));
}

// A narrow weight (fewer than 512 row tiles) gives too few workgroups for four tiles each; splitting K over up to four
// workgroups restores one equal workgroup per compute unit.  At least 24 k-steps per slice keep every wave's pipeline full.
int mlora_gemm_mid_ksplit(int T, int K, int N, int ks_max);
int mlora_gemm_mid_acc(float* resid, float* part, int ld_part, int ks, const void* xf, const void* Wp, int T, int K, int N, void* stream);

extern "C" int mlora_gemv_ksplit(int T, int K, int N_total) {
  if (T <= 0 || K <= 0 || K % 32 || N_total <= 0) return 1;
  if (T > 64) return mlora_gemm_mid_ksplit(T, K, N_total, 4);      // the matrix-core kernel for mid-size token blocks
  const int tiles = ceil_div(N_total, 16);
  if (tiles >= 512) return 1;
  const int groups = ceil_div(tiles, 4);      // row tiles per workgroup of the split kernel (see gemv_dispatch)
  int ks = 256 / groups;
  const int by_k = (K / KSTEP) / 24;
  if (ks > by_k) ks = by_k;
  if (ks > 4) ks = 4;
  return ks < 1 ? 1 : ks;
}

// What the shrink units that ride in a launch weigh in the K-split rule: sixteen workgroups' worth of rows, whatever
// the number of adapters - the slice count (and with it the order in which a row's partial sums are added) must not
// depend on which adapters a batch happens to hold.  Sixteen adapters of rank 16 over K = 4096 are exactly that many
// workgroups of units; with more, the launch exceeds the compute units by the difference.
extern "C" int mlora_gemv_shrink_rows(int K, int n_proj, int n_ad) {
  if (K <= 0 || n_proj <= 0 || n_ad <= 0) return 0;
  return 256;
}

extern "C" size_t mlora_gemv_ksplit_bytes(int T, int N_total, int ks) {
  if (T <= 0 || N_total <= 0 || ks <= 1) return 0;
  return (size_t)(ks - 1) * T * N_total * sizeof(float);
}

extern "C" int mlora_gemv_frag_acc_ksplit(float* y, float* y2, float* part, int ks, const void* xf, const void* Wp, int T, int K,
                                          int N_main, int N_ext, void* v_part, const void* const* A, int n_proj,
                                          const int32_t* tok_adapter, int r, int n_ad, void* stream) {
  if (int e = mlora_check_linear("gemv_frag_acc_ksplit", y, MLORA_F32, MLORA_ACCUMULATE, xf, K, Wp, T, K, N_main)) return e;
  if (T > 64) {      // the matrix-core kernel for mid-size token blocks: K slices only, nothing rides along
    MLORA_CHECK(N_ext == 0 && A == nullptr, MLORA_ERR_UNSUPPORTED, "gemv_frag_acc_ksplit: appended rows and shrink units need T <= 64 (T=%d)", T);
    MLORA_CHECK(ks >= 1 && ks <= 4 && (ks == 1 || part), MLORA_ERR_INVALID, "gemv_frag_acc_ksplit: ks=%d outside 1..4, or no partials buffer", ks);
    return mlora_gemm_mid_acc(y, part, N_main, ks, xf, Wp, T, K, N_main, stream);
  }
  MLORA_CHECK(N_ext >= 0 && N_ext % 4 == 0 && (N_ext == 0 || (y2 && N_main % 16 == 0)), MLORA_ERR_INVALID,
              "gemv_frag_acc_ksplit: appended rows need y2, N_ext %% 4 == 0 and N_main %% 16 == 0 (N_main=%d N_ext=%d)", N_main, N_ext);
  MLORA_CHECK(!(A && N_ext), MLORA_ERR_INVALID, "gemv_frag_acc_ksplit: shrink units and appended rows are exclusive");
  MLORA_CHECK(ks >= 1 && ks <= 4 && (ks == 1 || (part && (K / KSTEP) / ks >= 8)), MLORA_ERR_INVALID,
              "gemv_frag_acc_ksplit: ks=%d outside 1..4, too many slices for K=%d, or no partials buffer", ks, K);
  if (A)
    if (int e = check_shrink_args("gemv_frag_acc_ksplit", v_part, A, n_proj, tok_adapter, r, n_ad)) return e;
  if (T == 0) return MLORA_OK;
  const int N = N_main + N_ext;
  if (A)
    return gemv_dispatch<true, true, true>(y, MLORA_F32, MLORA_ACCUMULATE, xf, K, Wp, T, K, N, stream,
                                           shrink_batch(xf, v_part, A, n_proj, tok_adapter, T, K, r, n_ad), N_main, y2, ks, part);
  return gemv_dispatch<true, true, false>(y, MLORA_F32, MLORA_ACCUMULATE, xf, K, Wp, T, K, N, stream, LoraShrinkBatch(), N_main, y2,
                                          ks, part);
}

// Riders per token of the delta-carrying launch below (0: the shape is not served): a rider thread keeps at most
// RIDE_BQ 16-byte chunks of B, the launch must be K-split (it is the split form of the kernel that carries riders),
// and with riders the slices are chosen as if the matrix had 256 more rows (sixteen workgroups' worth, as for the
// riding shrink units: a constant, so that the slice count does not depend on the batch).
static int delta_ride_per_token(int T, int K, int N, int r) {
  if (T <= 0 || T > 64 || K <= 0 || K % 32 || N <= 0 || N % 16) return 0;
  if (r != 8 && r != 16 && r != 32 && r != 64) return 0;
  const int per_thread = ceil_div(N * (r / 8), GEMV_WAVES * WAVE);
  const int per_token = ceil_div(per_thread, RIDE_BQ);
  if (N % per_token || (N / per_token) % 4) return 0;
  if (mlora_gemv_ksplit(T, K, N + 256) < 2) return 0;
  return per_token;
}

// at most three slices: with the delta rows the reader then adds three slots, the most the RMSNorm takes
extern "C" int mlora_gemv_delta_ride_ksplit(int T, int K, int N, int r) {
  if (delta_ride_per_token(T, K, N, r) <= 0) return 0;
  const int ks = mlora_gemv_ksplit(T, K, N + 256);
  return ks > 3 ? 3 : ks;
}

extern "C" int mlora_gemv_frag_acc_ksplit_delta(float* y, float* part, int ks, const void* xf, const void* Wp, int T, int K, int N,
                                                const float* vpart, int n_vpart, const void* B, const int32_t* tok_adapter,
                                                float scaling, int r, int n_ad, void* stream) {
  if (int e = mlora_check_linear("gemv_frag_acc_ksplit_delta", y, MLORA_F32, MLORA_ACCUMULATE, xf, K, Wp, T, K, N)) return e;
  MLORA_CHECK(part && vpart && B && tok_adapter && n_ad > 0, MLORA_ERR_INVALID, "gemv_frag_acc_ksplit_delta: null pointer or no adapters");
  const int per_token = delta_ride_per_token(T, K, N, r);
  MLORA_CHECK(per_token > 0 && ks == mlora_gemv_delta_ride_ksplit(T, K, N, r) && (K / KSTEP) / ks >= 8, MLORA_ERR_UNSUPPORTED,
              "gemv_frag_acc_ksplit_delta: T=%d K=%d N=%d r=%d ks=%d not served (mlora_gemv_delta_ride_ksplit gives %d)", T, K, N, r, ks,
              mlora_gemv_delta_ride_ksplit(T, K, N, r));
  MLORA_CHECK(n_vpart >= 1, MLORA_ERR_INVALID, "gemv_frag_acc_ksplit_delta: no shares");
  LoraDeltaRide dr;
  dr.vpart = vpart;
  dr.B = (const f16*)B;
  dr.ids = tok_adapter;
  dr.out = part + (size_t)(ks - 1) * T * N;       // the slot behind the K-slice partials
  dr.scaling = scaling;
  dr.n_vpart = n_vpart; dr.T = T; dr.N = N; dr.r = r; dr.n_ad = n_ad;
  dr.per_token = per_token;
  dr.accumulate = 0;
  return gemv_dispatch<true, true, false>(y, MLORA_F32, MLORA_ACCUMULATE, xf, K, Wp, T, K, N, stream, LoraShrinkBatch(), N, nullptr, ks,
                                          part, dr, T * per_token);
}

extern "C" int mlora_lora_expand_shares_ok(int N, int r) {
  if (N <= 0 || N % 16 || (r != 8 && r != 16 && r != 32 && r != 64)) return 0;
  const int per_token = ceil_div(ceil_div(N * (r / 8), GEMV_WAVES * WAVE), SOLO_BQ);
  return N % per_token == 0 && (N / per_token) % 4 == 0 ? 1 : 0;
}

extern "C" int mlora_lora_expand_shares(float* y, const float* vpart, int n_vpart, const void* B, const int32_t* tok_adapter, float scaling,
                                        int T, int N, int r, int n_ad, void* stream) {
  MLORA_CHECK(y && vpart && B && tok_adapter && n_ad > 0, MLORA_ERR_INVALID, "lora_expand_shares: null pointer or no adapters");
  MLORA_CHECK(T >= 0 && mlora_lora_expand_shares_ok(N, r), MLORA_ERR_UNSUPPORTED,
              "lora_expand_shares: need N %% 16 == 0, rank 8, 16, 32 or 64 and N dividing over the workgroups of a token (N=%d r=%d)", N, r);
  MLORA_CHECK(n_vpart >= 1, MLORA_ERR_INVALID, "lora_expand_shares: no shares");
  const int per_token = ceil_div(ceil_div(N * (r / 8), GEMV_WAVES * WAVE), SOLO_BQ);
  MLORA_CHECK((long)T * per_token <= 0x7fffffffL, MLORA_ERR_UNSUPPORTED, "lora_expand_shares: T=%d is too many tokens", T);
  if (T == 0) return MLORA_OK;
  LoraDeltaRide dr;
  dr.vpart = vpart;
  dr.B = (const f16*)B;
  dr.ids = tok_adapter;
  dr.out = y;
  dr.scaling = scaling;
  dr.n_vpart = n_vpart; dr.T = T; dr.N = N; dr.r = r; dr.n_ad = n_ad;
  dr.per_token = per_token;
  dr.accumulate = 1;
  hipLaunchKernelGGL(lora_expand_shares_kernel, dim3(T * per_token), dim3(GEMV_WAVES * WAVE), 0, (hipStream_t)stream, dr);
  return mlora_launch_status("lora_expand_shares");
}

extern "C" int mlora_gemv_frag_silu(void* act, const void* xf, const void* Wil_p, int T, int K, int I, void* stream) {
  MLORA_CHECK(act && xf && Wil_p, MLORA_ERR_INVALID, "gemv_frag_silu: null pointer");
  MLORA_CHECK(T > 0 && T <= 64 && K > 0 && K % 32 == 0 && I > 0 && I % 32 == 0, MLORA_ERR_UNSUPPORTED,
              "gemv_frag_silu: need 0 < T <= 64, K %% 32 == 0, I %% 32 == 0 (T=%d K=%d I=%d)", T, K, I);
  const f16* xp = (const f16*)xf;
  const f16* Wp = (const f16*)Wil_p;
  hipStream_t s = (hipStream_t)stream;
  const LoraShrinkBatch sb = LoraShrinkBatch();
  const dim3 grid(I / 16), block(GEMV_WAVES * WAVE);
  // enough pairs for two or more per compute unit: one workgroup per unit with an equal share of the pairs
  const int n_cu = gemv_n_cu();
  const int pairs = I / 16;
  const int per = n_cu > 0 ? ceil_div(pairs, n_cu) : 0;
  if ((T <= 32 || per <= 3) && n_cu > 0 && pairs >= 2 * n_cu && per <= 4) {
    const int base = pairs / n_cu, rem = pairs % n_cu;
    const dim3 g(n_cu);
#define MLORA_SILU_CU(NP, TT, PIPE) \
  hipLaunchKernelGGL((gemv_silu_cu_kernel<NP, TT, PIPE>), g, block, 0, s, (f16*)act, xp, Wp, T, K, I, base, rem)
    if (T <= 16) {
      if (per <= 2) MLORA_SILU_CU(2, 1, 4);
      else if (per == 3) MLORA_SILU_CU(3, 1, 4);
      else MLORA_SILU_CU(4, 1, 3);
    } else if (T <= 32) {
      if (per <= 2) MLORA_SILU_CU(2, 2, 4);
      else if (per == 3) MLORA_SILU_CU(3, 2, 3);
      else MLORA_SILU_CU(4, 2, 2);
    } else {                                   // 33..64 tokens: four token tiles, at most three pairs fit the registers
      if (per <= 2) MLORA_SILU_CU(2, 4, 2);
      else MLORA_SILU_CU(3, 4, 2);
    }
#undef MLORA_SILU_CU
    return mlora_launch_status("gemv_frag_silu");
  }
  if (T <= 16) hipLaunchKernelGGL((gemv_kernel<2, 1, OUT_SILU_FRAG, true, true, false>), grid, block, 0, s, act, xp, K, Wp, T, K, 2 * I, sb, 0, 2 * I, nullptr, 1, nullptr, LoraDeltaRide(), 0);
  else if (T <= 32) hipLaunchKernelGGL((gemv_kernel<2, 2, OUT_SILU_FRAG, true, true, false>), grid, block, 0, s, act, xp, K, Wp, T, K, 2 * I, sb, 0, 2 * I, nullptr, 1, nullptr, LoraDeltaRide(), 0);
  else hipLaunchKernelGGL((gemv_kernel<2, 4, OUT_SILU_FRAG, true, true, false, 2>), grid, block, 0, s, act, xp, K, Wp, T, K, 2 * I, sb, 0, 2 * I, nullptr, 1, nullptr, LoraDeltaRide(), 0);
  return mlora_launch_status("gemv_frag_silu");
}

extern "C" int mlora_gemv_frag_split(void* y, int y_dtype, int mode, float* y2, const void* xf, const void* Wp, int T, int K,
                                     int N_main, int N_ext, void* stream) {
  if (int e = mlora_check_linear("gemv_frag_split", y, y_dtype, mode, xf, K, Wp, T, K, N_main)) return e;
  MLORA_CHECK(T <= 64, MLORA_ERR_UNSUPPORTED, "gemv_frag_split: T=%d exceeds 64", T);
  MLORA_CHECK(y2 && N_ext > 0 && N_ext % 4 == 0 && N_main % 16 == 0, MLORA_ERR_INVALID,
              "gemv_frag_split: need y2, N_ext %% 4 == 0 and N_main %% 16 == 0 (N_main=%d N_ext=%d)", N_main, N_ext);
  if (T == 0) return MLORA_OK;
  return gemv_dispatch<true, true, false>(y, y_dtype, mode, xf, K, Wp, T, K, N_main + N_ext, stream, LoraShrinkBatch(), N_main, y2);
}

// K ranges of the appended rows in the one-workgroup-per-unit form of the split GEMV (1: that form does not apply)
extern "C" int mlora_gemv_split_kq(int T, int K, int N_main, int N_ext) {
  const int n_cu = gemv_n_cu();
  if (T <= 0 || T > 32 || K <= 0 || K % 32 || N_main <= 0 || N_main % 16 || N_ext <= 0 || N_ext % 16 || n_cu <= 0) return 1;
  const int main_tiles = N_main / 16, ext_tiles = N_ext / 16;
  const int per = ceil_div(main_tiles, n_cu);
  const int kq = LORA_MAX_KQ;
  if (main_tiles < 2 * n_cu || per > 3 || (K / 32) / kq < 8 || ext_tiles * kq > n_cu) return 1;
  return kq;
}

extern "C" int mlora_gemv_frag_split_kq(void* y, float* y2, int kq, const void* xf, const void* Wp, int T, int K, int N_main,
                                        int N_ext, void* stream) {
  if (int e = mlora_check_linear("gemv_frag_split_kq", y, MLORA_F16, MLORA_STORE, xf, K, Wp, T, K, N_main)) return e;
  MLORA_CHECK(T <= 64, MLORA_ERR_UNSUPPORTED, "gemv_frag_split_kq: T=%d exceeds 64", T);
  MLORA_CHECK(y2 && N_ext > 0 && N_ext % 4 == 0 && N_main % 16 == 0, MLORA_ERR_INVALID,
              "gemv_frag_split_kq: need y2, N_ext %% 4 == 0 and N_main %% 16 == 0 (N_main=%d N_ext=%d)", N_main, N_ext);
  MLORA_CHECK(kq == 1 || kq == mlora_gemv_split_kq(T, K, N_main, N_ext), MLORA_ERR_INVALID,
              "gemv_frag_split_kq: kq=%d, mlora_gemv_split_kq gives %d", kq, mlora_gemv_split_kq(T, K, N_main, N_ext));
  if (T == 0) return MLORA_OK;
  if (kq == 1)
    return gemv_dispatch<true, true, false>(y, MLORA_F16, MLORA_STORE, xf, K, Wp, T, K, N_main + N_ext, stream, LoraShrinkBatch(), N_main, y2);
  const int n_cu = gemv_n_cu();
  const int main_tiles = N_main / 16;
  const int base = main_tiles / n_cu, rem = main_tiles % n_cu;
  const int per = ceil_div(main_tiles, n_cu);
  const dim3 g(n_cu), block(GEMV_WAVES * WAVE);
  hipStream_t s = (hipStream_t)stream;
#define MLORA_SPLIT_CU(NM, TT, PIPE)                                                                                       \
  hipLaunchKernelGGL((gemv_split_cu_kernel<NM, TT, PIPE>), g, block, 0, s, (f16*)y, y2, (const f16*)xf, (const f16*)Wp, T, K, \
                     N_main, N_ext, base, rem, kq, n_cu)
  if (T <= 16) {
    if (per <= 2) MLORA_SPLIT_CU(2, 1, 4);
    else MLORA_SPLIT_CU(3, 1, 4);
  } else {
    if (per <= 2) MLORA_SPLIT_CU(2, 2, 4);
    else MLORA_SPLIT_CU(3, 2, 3);
  }
#undef MLORA_SPLIT_CU
  return mlora_launch_status("gemv_frag_split_kq");
}

extern "C" size_t mlora_frag_activation_elems(int T, int K) {
  if (T <= 0 || K <= 0) return 0;
  return (size_t)mlora_frag_tiles(T) * 16 * (size_t)K;
}

extern "C" int mlora_pack_activation(void* dst, const void* src, int ldsrc, int T, int K, void* stream) {
  MLORA_CHECK(dst && src && dst != src, MLORA_ERR_INVALID, "pack_activation: null or aliasing pointers");
  MLORA_CHECK(T > 0 && K > 0 && K % 32 == 0 && ldsrc >= K && ldsrc % 8 == 0 && (size_t)mlora_frag_tiles(T) * 2 * K < 0x7fffffffULL,
              MLORA_ERR_UNSUPPORTED, "pack_activation: need T > 0, K %% 32 == 0, ldsrc >= K (T=%d K=%d ldsrc=%d)", T, K, ldsrc);
  const int chunks = mlora_frag_tiles(T) * 16 * (K / 8);
  hipLaunchKernelGGL(pack_activation_kernel, dim3(ceil_div(chunks, 256)), dim3(256), 0, (hipStream_t)stream, (f16*)dst,
                     (const f16*)src, ldsrc, T, K, mlora_frag_tiles(T), chunks);
  return mlora_launch_status("pack_activation");
}

extern "C" size_t mlora_packed_weight_elems(int N, int K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)ceil_div(N, 16) * 16 * (size_t)K;
}

extern "C" int mlora_pack_weight(void* dst, const void* src, int N, int K, void* stream) {
  MLORA_CHECK(dst && src && dst != src, MLORA_ERR_INVALID, "pack_weight: null or aliasing pointers");
  MLORA_CHECK(N > 0 && K > 0 && K % 32 == 0, MLORA_ERR_UNSUPPORTED, "pack_weight: need K %% 32 == 0 (N=%d K=%d)", N, K);
  const size_t chunks = mlora_packed_weight_elems(N, K) / 8;
  MLORA_CHECK(chunks / 256 + 1 < 0x7fffffffULL, MLORA_ERR_UNSUPPORTED, "pack_weight: matrix too large");
  hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (f16*)dst,
                     (const f16*)src, N, K, chunks);
  return mlora_launch_status("pack_weight");
}
