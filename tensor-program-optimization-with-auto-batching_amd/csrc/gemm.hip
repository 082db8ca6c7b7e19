// Prefill-time base linear for gfx950:  y[T, N] (=|+=) x[T, K] . W[N, K]^T  for any T (MFMA-bound).
//
// Three kernels, by operand layout and problem size:
//   gemm_kernel      row-major or fragment-ordered W, fragments loaded straight from global memory into registers
//                    (both operands are K-contiguous, which is what v_mfma_f32_16x16x32_f16 wants: a lane holds 8
//                    consecutive k of one row); a wave owns 64 x 64 outputs.  Any shape; the small-T workhorse.
//   gemm_lds_kernel  fragment-ordered W, register-staged LDS double buffer; 256 x 64 or 256 x 256 blocks.
//   gemm_pp_kernel   fragment-ordered W and row-major or fragment-ordered x, both copied from global memory straight
//                    into a four-stage LDS ring; persistent 256 x 256 blocks, eight waves.  The large-T kernel.
// All three add the 32-k MFMA steps of an output in ascending k into one accumulator, so their results are the same
// bits.
#include <type_traits>

#include "common.h"

int mlora_check_linear(const char* who, const void* y, int y_dtype, int mode, const void* x, int ldx, const void* W,
                       int T, int K, int N);

namespace {

enum { OUT_F16 = 0, OUT_F32 = 1, OUT_ACC_F32 = 2, OUT_SILU = 3 };

// compute units of the current device (0 if it cannot be asked), read once
int gemm_n_cu() {
  static const int n_cu = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cu = 0;
    return cu;
  }();
  return n_cu;
}

constexpr int WT = 4;   // 16-wide MFMA tiles per wave along N and along T

template <int OUT, bool PACKED>
__global__ __launch_bounds__(256) void gemm_kernel(void* __restrict__ yv, const f16* __restrict__ x, int ldx,
                                                   const f16* __restrict__ W, int T, int K, int N) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, kg = lane >> 4;
  const int n0 = blockIdx.x * 128 + (wave & 1) * 64;
  const int t0 = blockIdx.y * 128 + (wave >> 1) * 64;
  if (n0 >= N || t0 >= T) return;

  constexpr int WSTEP = PACKED ? 512 : 32;   // elements between consecutive k-steps of one fragment stream
  const int tiles = (N + 15) / 16;
  const f16* wp[WT];
  const f16* xp[WT];
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    if constexpr (PACKED) {
      int nt = n0 / 16 + i;
      nt = nt < tiles ? nt : tiles - 1;
      wp[i] = W + ((size_t)nt * (K / 32)) * 512 + lane * 8;
    } else {
      int n = n0 + i * 16 + r16;
      n = n < N ? n : N - 1;
      wp[i] = W + (size_t)n * K + kg * 8;
    }
    int t = t0 + i * 16 + r16;
    t = t < T ? t : T - 1;
    xp[i] = x + (size_t)t * ldx + kg * 8;
  }
  f32x4 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  f16x8 a[WT], b[WT];
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    a[i] = ld8(wp[i]);
    b[i] = ld8(xp[i]);
  }
  const int KB = K / 32;
  for (int ks = 1; ks <= KB; ++ks) {
    f16x8 an[WT], bn[WT];
    const int kc = ks < KB ? ks : 0;   // the last prefetch wraps to a valid address and is discarded
#pragma unroll
    for (int i = 0; i < WT; ++i) {
      an[i] = ld8(wp[i] + (size_t)kc * WSTEP);
      bn[i] = ld8(xp[i] + kc * 32);
    }
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
      for (int j = 0; j < WT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], acc[i][j], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < WT; ++i) {
      a[i] = an[i];
      b[i] = bn[i];
    }
  }

  const int g = lane >> 4;
#pragma unroll
  for (int j = 0; j < WT; ++j) {
    const int t = t0 + j * 16 + r16;
    if (t >= T) continue;
#pragma unroll
    for (int i = 0; i < WT; ++i) {
      const int n = n0 + i * 16 + g * 4;
      if (n >= N) continue;
      const size_t o = (size_t)t * N + n;
      const f32x4 s = acc[i][j];
      if constexpr (OUT == OUT_F16) {
        *reinterpret_cast<f16x4*>((f16*)yv + o) = f16x4{(f16)s[0], (f16)s[1], (f16)s[2], (f16)s[3]};
      } else if constexpr (OUT == OUT_F32) {
        *reinterpret_cast<f32x4*>((float*)yv + o) = s;
      } else {
        f32x4* p = reinterpret_cast<f32x4*>((float*)yv + o);
        *p = *p + s;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// LDS-staged variant for fragment-ordered weights.  In its large shape a workgroup of 4 waves owns a 256-token x
// 256-column output block, a wave 128 x 128 of it (8 x 8 MFMA tiles; the 256 accumulator registers live in the
// accumulation half of the register file at one wave per SIMD).  A stage is 64 k of both operands (2 x 32 KiB) staged through LDS in
// fragment order, double buffered: while the matrix cores work on one buffer, the next stage's global loads are in
// flight and are written to the other buffer, one barrier per stage.  Weight fragments are copied as they lie in
// memory (contiguous 1 KiB); the token rows are read 64 contiguous bytes at a time and transposed into fragment
// order by the LDS write (with an XOR on the token slot that keeps every quarter-wave write conflict-free).
// Per stage and CU: 64 KiB from L2 for 2 x 64 x 4 MFMAs (2048 MFMA cycles per SIMD): 32 B/clk, half the L1 rate;
// LDS traffic 64 KiB written + 128 KiB read.
// ---------------------------------------------------------------------------------------------
constexpr int LBK = 64;              // k per stage

// FT x FN: 16-row fragments of tokens / of weight rows per block; WT x WN: MFMA tiles of a wave (FT/WT * FN/WN == 4 waves)
template <int OUT, int FT, int FN, int WT_, int WN_>
__global__ __launch_bounds__(256) void gemm_lds_kernel(void* __restrict__ yv, const f16* __restrict__ x, int ldx,
                                                       const f16* __restrict__ Wp, int T, int K, int N) {
  static_assert((FT / WT_) * (FN / WN_) == 4, "four waves cover the block");
  constexpr int KS = LBK / 32;                      // 32-k steps per stage
  constexpr int WELEMS = KS * FN * 512, XELEMS = KS * FT * 512;   // fp16 elements of a stage: W, then x
  constexpr int STAGE = WELEMS + XELEMS;
  constexpr int WCH = KS * FN * WAVE / 256, XCH = KS * FT * WAVE / 256;   // 16-byte chunks per thread and stage
  static_assert(WCH >= 1 && XCH >= 1, "a stage gives every thread at least one chunk of each operand");
  extern __shared__ __align__(16) f16 smem[];       // [2][STAGE]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n0 = blockIdx.x * FN * 16, t0 = blockIdx.y * FT * 16;
  constexpr int WAVES_N = FN / WN_;
  const int wn = wave % WAVES_N, wt = wave / WAVES_N;
  const int KB = K / 32;
  const int tiles = (N + 15) / 16;

  // chunk c = threadIdx.x + 256 j of an operand's stage: fragment f = c / 64 = ks * F + tile, lane slot l = c % 64
  const f16* wsrc[WCH];
  const f16* xsrc[XCH];
#pragma unroll
  for (int j = 0; j < WCH; ++j) {
    const int c = threadIdx.x + 256 * j;
    const int f = c >> 6, l = c & 63;
    const int ks = f / FN, tile = f % FN;
    int nt = n0 / 16 + tile;
    nt = nt < tiles ? nt : tiles - 1;               // columns past N: a valid fragment, results dropped
    wsrc[j] = Wp + ((size_t)nt * KB + ks) * 512 + l * 8;
  }
  // x chunks: 4 consecutive lanes read the 64 contiguous bytes (one 32-k step) of one token row, so a quarter-wave
  // covers 4 rows x 4 lane groups g.  The LDS slot of a token inside its 16-token fragment is XORed with 4 g: the 16
  // lanes of a quarter-wave then write 16 different slots (no bank conflict), and a read of a fragment stays a
  // permutation inside each 16-lane group.
  int xdst[XCH];
#pragma unroll
  for (int j = 0; j < XCH; ++j) {
    const int c2 = threadIdx.x + 256 * j;
    const int ks = c2 / (FT * 64), c = c2 % (FT * 64);
    const int row = c >> 2, gq = c & 3;
    int t = t0 + row;
    t = t < T ? t : T - 1;
    xsrc[j] = x + (size_t)t * ldx + ks * 32 + gq * 8;
    xdst[j] = ((ks * FT + (row >> 4)) * 64 + gq * 16 + ((row & 15) ^ (gq << 2))) * 8;
  }
  f16x8 wst[WCH], xst[XCH];
  auto load_stage = [&](int s) {                    // s: stage index; k-steps KS*s .. (the last may be past K)
#pragma unroll
    for (int j = 0; j < WCH; ++j) {
      const int ks = (threadIdx.x + 256 * j) / (64 * FN);
      const int kb = s * KS + ks;
      const int kc = kb < KB ? kb : KB - 1;         // past K: a valid address; that step is not multiplied
      wst[j] = ld8(wsrc[j] + (size_t)(kc - ks) * 512);
    }
#pragma unroll
    for (int j = 0; j < XCH; ++j) {
      const int ks = (threadIdx.x + 256 * j) / (FT * 64);
      const int kb = s * KS + ks;
      const int kc = kb < KB ? kb : KB - 1;
      xst[j] = ld8(xsrc[j] + (kc - ks) * 32);
    }
  };
  auto store_stage = [&](int buf) {
    f16* dst = smem + buf * STAGE;
#pragma unroll
    for (int j = 0; j < WCH; ++j) st8(dst + (threadIdx.x + 256 * j) * 8, wst[j]);
#pragma unroll
    for (int j = 0; j < XCH; ++j) st8(dst + WELEMS + xdst[j], xst[j]);
  };

  f32x4 acc[WN_][WT_];
#pragma unroll
  for (int i = 0; i < WN_; ++i)
#pragma unroll
    for (int j = 0; j < WT_; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int xslot = (lane & 48) + ((lane & 15) ^ ((lane >> 4) << 2));   // lane's token slot after the write-side XOR
  const int S = (KB + KS - 1) / KS;
  load_stage(0);
  store_stage(0);
  __syncthreads();
  for (int s = 0; s < S; ++s) {
    if (s + 1 < S) load_stage(s + 1);
    const f16* ws = smem + (s & 1) * STAGE;
    const f16* xs = ws + WELEMS;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (s * KS + ks < KB) {                        // workgroup-uniform
        f16x8 a[WN_], b[WT_];
#pragma unroll
        for (int i = 0; i < WN_; ++i) a[i] = ld8(ws + (ks * FN + wn * WN_ + i) * 512 + lane * 8);
#pragma unroll
        for (int j = 0; j < WT_; ++j) b[j] = ld8(xs + (ks * FT + wt * WT_ + j) * 512 + xslot * 8);
#pragma unroll
        for (int i = 0; i < WN_; ++i)
#pragma unroll
          for (int j = 0; j < WT_; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], acc[i][j], 0, 0, 0);
      }
    }
    if (s + 1 < S) store_stage((s + 1) & 1);
    __syncthreads();
  }

  const int r16 = lane & 15, g = lane >> 4;
#pragma unroll
  for (int j = 0; j < WT_; ++j) {
    const int t = t0 + (wt * WT_ + j) * 16 + r16;
    if (t >= T) continue;
#pragma unroll
    for (int i = 0; i < WN_; ++i) {
      const int n = n0 + (wn * WN_ + i) * 16 + g * 4;
      if (n >= N) continue;
      const size_t o = (size_t)t * N + n;
      const f32x4 sacc = acc[i][j];
      if constexpr (OUT == OUT_F16) {
        *reinterpret_cast<f16x4*>((f16*)yv + o) = f16x4{(f16)sacc[0], (f16)sacc[1], (f16)sacc[2], (f16)sacc[3]};
      } else if constexpr (OUT == OUT_F32) {
        *reinterpret_cast<f32x4*>((float*)yv + o) = sacc;
      } else {
        f32x4* p = reinterpret_cast<f32x4*>((float*)yv + o);
        *p = *p + sacc;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Eight-wave persistent variant for large token counts.  A workgroup owns 256 tokens x 256 weight rows at a time, a
// wave 64 tokens x 128 rows of it (4 x 8 MFMA tiles, 128 accumulator registers), two waves per SIMD, one workgroup
// per compute unit, which walks through its share of the output blocks.
//   * Both operands go from global memory straight into LDS (global_load_lds_dwordx4: no register staging, no LDS
//     store instructions) in fragment order, through a ring of four 32-k stages with three stages in flight ahead of
//     the one being multiplied.  A weight fragment is copied as it lies in memory.  A token fragment likewise when the
//     activations come in fragment order (x_tt > 0: Xf[k/32][t/16][4][16][8], one contiguous 1 KiB block per
//     fragment); from row-major activations it is gathered 16 rows x 64 bytes by the load's per-lane addresses - half
//     cache lines, which costs the load path a third of its speed.
//   * The ring runs on across block boundaries: while the last stages of a block are multiplied and its results are
//     stored, the first stages of the workgroup's next block are already in flight.
//   * Fragment registers are double-buffered: the LDS reads of stage g + 1 are issued right before the MFMAs of stage
//     g and complete under them.
//   * fp16 results cross a small LDS buffer so that a store instruction writes whole 128-byte lines of a token row.
// Blocks are numbered so that an XCD (workgroup id mod 8) works through a contiguous range of weight-row blocks, all
// token blocks of one weight block next to each other: every XCD streams its own share of W through its L2 once.
// ---------------------------------------------------------------------------------------------
constexpr int PP_WAVES = 8;
constexpr int PP_STAGES = 4;
constexpr int PP_F = 16;                       // 16-row fragments per block side (256 tokens, 256 weight rows)
constexpr int PP_STAGE_ELEMS = 2 * PP_F * 512; // fp16 elements of one 32-k stage: 16 weight fragments, then 16 token fragments
constexpr int PP_OUT_LD = 64 + 4;              // fp16 elements per token row of a wave's output staging (padded: conflict-free writes)
constexpr int PP_OUT_ELEMS = 16 * PP_OUT_LD;   // per wave: 16 tokens x 64 columns

// LoRA deltas that ride in the GEMM as extra k-steps: y = [x | v_hi | v_lo] . [W | B[a] | B[a]]^T for a 256-token block
// whose tokens all name adapter a (blk_adapter[block] >= 0), v = scaling * x . A[a]^T as fp16 hi + lo halves [T][r].
// Projections are row ranges of the fused weight, each with its own B table [n_ad][rows][r] (row-major, r in {32, 64})
// and its own v; a 256-row block lies inside one range (checked by the launcher).  n_proj == 0: a plain GEMM.
struct PPLora {
  const f16* B[3];
  const f16* vh[3];
  const f16* vl[3];
  int n_begin[3], n_rows[3];
  int n_proj, r;
  const int32_t* blk_adapter;
};

__device__ __forceinline__ unsigned long long uniform64(unsigned long long v) {
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// OUT_SILU: Wp is the fused [2 I, K] gate / up matrix (N = 2 I, gate rows first) and the output is
// act = silu(f16(gate)) * f16(up) [T, I] in fragment order (tiles per 32-k step: x_tt).  A block is 256 tokens x 128
// channels: the ring slots of a stage hold, for each of the two row groups of waves, four gate tiles and then the four
// up tiles of the same channels, so that a lane ends up with both halves of its channels and the product never leaves
// the registers.  LoRA deltas: slot 0 of `lo` is the gate projection, slot 1 the up projection (B == nullptr: not
// adapted); each rides as its own extra k-steps, in which only that half of a wave's tiles is multiplied.
// LORA = false is the plain GEMM (lo is ignored)
template <int OUT, bool LORA>
__global__ __launch_bounds__(PP_WAVES* WAVE, 2) void gemm_pp_kernel(void* __restrict__ yv, const f16* __restrict__ x, int ldx, int x_tt,
                                                                   const f16* __restrict__ Wp, int T, int K, int N, int gx, int gy,
                                                                   PPLora lo) {
  extern __shared__ __align__(16) f16 smem[];  // [PP_STAGES][PP_STAGE_ELEMS], then [PP_WAVES][PP_OUT_ELEMS]
  constexpr int NW = PP_WAVES;
  constexpr int LQ = 2 * PP_F / NW;            // fragments a wave fetches per stage (4)
  constexpr int WTF = 4;                       // token fragments of a wave's tile (64 tokens)
  constexpr bool SILU = OUT == OUT_SILU;
  constexpr int BN = SILU ? PP_F * 8 : PP_F * 16;   // output columns of a block (SILU: channels, each a gate and an up row)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nb = gx * gy;
  const int KB = K / 32;
  const int tiles = (N + 15) / 16;
  const int I = N / 2, itiles = I / 16;        // SILU: channels and their 16-row tiles
  const int G = gridDim.x;

  // block number -> (weight-row block, token block)
  auto block_of = [&](int L, int& n0, int& t0) {
    int idx = L;
    if ((nb & 7) == 0 && (G & 7) == 0) idx = (L & 7) * (nb >> 3) + (L >> 3);
    n0 = (idx / gy) * BN;
    t0 = (idx % gy) * (PP_F * 16);
  };
  // the LoRA part of a block: projection slot and adapter (-1: none), everything uniform
  auto lora_of = [&](int n0, int t0, int& slot) -> int {
    if constexpr (SILU) {
      slot = 0;
      return lo.blk_adapter[t0 / (PP_F * 16)];
    }
    slot = -1;
#pragma unroll
    for (int i = 0; i < 3; ++i)
      if (i < lo.n_proj && n0 >= lo.n_begin[i] && n0 < lo.n_begin[i] + lo.n_rows[i]) slot = i;
    if (slot < 0) return -1;
    return lo.blk_adapter[t0 / (PP_F * 16)];
  };
  const int EP = LORA ? 2 * (lo.r / 32) : 0;    // extra k-steps per projection of a block with a delta: hi halves, then lo halves
  const bool has_gate = SILU && LORA && lo.B[0] != nullptr;
  const int E = SILU ? EP * ((lo.B[0] != nullptr) + (lo.B[1] != nullptr)) : EP;

  // ---- loader role: wave w fetches fragments 4 w .. 4 w + 3 of every stage (waves 0-3: weights, waves 4-7: tokens)
  const f16* src[LQ];
  int step = 0;                                // elements between consecutive k-steps of this wave's sources
  int load_L = blockIdx.x, load_kb = 0;        // the stage the loader issues next
  int load_nst = KB;                           // stages of the block being loaded (KB, or KB + E with a delta)
  const f16* l_src = nullptr;                  // LoRA stages of that block (all uniform): row 0 of the block in B[a] (weight waves) or in v_hi (token waves) ...
  long l_lo = 0;                               // ... the distance from v_hi to v_lo (token waves; 0 for weight waves) ...
  int l_rows = 1;                              // ... and the rows that exist from there on (rows past them repeat the last one; their results are dropped)
  int l_a = -1, l_n0 = 0, l_t0 = 0;            // SILU: adapter, first channel and first token of that block (the stages' addresses are formed per stage)
  auto load_block = [&](int L) {
    int n0, t0;
    block_of(L < nb ? L : blockIdx.x, n0, t0); // past the last block: valid addresses, the data is never multiplied
    load_nst = KB;
    if constexpr (LORA) {
      int slot;
      const int a = L < nb ? lora_of(n0, t0, slot) : -1;
      if (a >= 0) load_nst = __builtin_amdgcn_readfirstlane(KB + E);
      if (SILU) {
        l_a = a;
        l_n0 = n0;
        l_t0 = t0;
      } else if (a >= 0) {
        const f16* Bt = lo.B[0];
        const f16* vh = lo.vh[0];
        const f16* vl = lo.vl[0];
        int nbeg = lo.n_begin[0], nrows = lo.n_rows[0];
#pragma unroll
        for (int i = 1; i < 3; ++i)
          if (i == slot) {                     // uniform select: the struct is never indexed dynamically
            Bt = lo.B[i]; vh = lo.vh[i]; vl = lo.vl[i]; nbeg = lo.n_begin[i]; nrows = lo.n_rows[i];
          }
        if (wave < NW / 2) {
          l_src = Bt + ((size_t)a * nrows + (n0 - nbeg)) * lo.r;
          l_lo = 0;
          l_rows = nrows - (n0 - nbeg);
        } else {
          l_src = vh + (size_t)t0 * lo.r;
          l_lo = vl - vh;
          l_rows = T - t0;
        }
        // all of this is the same in every lane: say so, it lives in scalar registers across the K loop
        l_src = (const f16*)uniform64((unsigned long long)l_src);
        l_lo = (long)uniform64((unsigned long long)l_lo);
        l_rows = __builtin_amdgcn_readfirstlane(l_rows);
      }
    }
    if (wave < NW / 2) {
#pragma unroll
      for (int q = 0; q < LQ; ++q) {
        int nt;
        if constexpr (SILU) {                  // slots 8 wn + 0..3: gate tiles of channels n0 + 64 wn .., slots 8 wn + 4..7: their up tiles
          int it = n0 / 16 + (wave >> 1) * LQ + q;
          it = it < itiles ? it : itiles - 1;
          nt = it + (wave & 1) * itiles;
        } else {
          nt = n0 / 16 + wave * LQ + q;
          nt = nt < tiles ? nt : tiles - 1;    // rows past N: a valid fragment, results dropped
        }
        src[q] = Wp + (size_t)nt * KB * 512 + lane * 8;
      }
      step = 512;
    } else if (x_tt > 0) {
#pragma unroll
      for (int q = 0; q < LQ; ++q) {
        int tt = t0 / 16 + (wave - NW / 2) * LQ + q;
        tt = tt < x_tt ? tt : x_tt - 1;
        src[q] = x + (size_t)tt * 512 + lane * 8;
      }
      step = x_tt * 512;
    } else {
#pragma unroll
      for (int q = 0; q < LQ; ++q) {
        int t = t0 + ((wave - NW / 2) * LQ + q) * 16 + (lane & 15);
        t = t < T ? t : T - 1;
        src[q] = x + (size_t)t * ldx + (lane >> 4) * 8;
      }
      step = 32;
    }
  };
  int ring = 0;                                // ring slot of the stage issued next
  // PLAIN: the caller knows that this stage is an ordinary k-step and not the last of its block (no tests at all)
  auto issue = [&](auto PLAIN) {
    constexpr bool plain = decltype(PLAIN)::value;
    f16* dst = smem + ring * PP_STAGE_ELEMS + wave * LQ * 512;
    if (plain || !LORA || load_kb < KB) {
#pragma unroll
      for (int q = 0; q < LQ; ++q)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[q] + (size_t)load_kb * step),
                                         (__attribute__((address_space(3))) void*)(dst + q * 512), 16, 0, 0);
    } else if constexpr (SILU) {               // a LoRA stage of the gate or of the up projection
      const int j = load_kb - KB, RB = lo.r / 32;
      const bool up = !(has_gate && j < EP);   // uniform
      const int jj = has_gate && up ? j - EP : j;
      const bool lo_half = jj >= RB;
      const int ks = (lo_half ? jj - RB : jj) * 32;
      const f16* base;
      int row0, rows;
      if (wave < NW / 2) {                     // rows of the projection's table for this wave's channels (used by the waves of that half only)
        base = (up ? lo.B[1] : lo.B[0]) + (size_t)l_a * I * lo.r;
        row0 = l_n0 + (wave >> 1) * (LQ * 16);
        rows = I;
      } else {
        base = up ? (lo_half ? lo.vl[1] : lo.vh[1]) : (lo_half ? lo.vl[0] : lo.vh[0]);
        row0 = l_t0 + (wave & 3) * (LQ * 16);
        rows = T;
      }
#pragma unroll
      for (int q = 0; q < LQ; ++q) {
        int row = row0 + q * 16 + (lane & 15);
        row = row < rows ? row : rows - 1;
        const f16* p = base + ((size_t)row * lo.r + ks + (lane >> 4) * 8);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p,
                                         (__attribute__((address_space(3))) void*)(dst + q * 512), 16, 0, 0);
      }
    } else {                                   // a LoRA stage: 16 rows x 64 bytes per fragment, gathered by the lanes' addresses
      const int j = load_kb - KB, RB = lo.r / 32;
      const int ks = (j < RB ? j : j - RB) * 32;
#pragma unroll
      for (int q = 0; q < LQ; ++q) {
        int row = ((wave & 3) * LQ + q) * 16 + (lane & 15);
        row = row < l_rows ? row : l_rows - 1;
        const f16* p = l_src + (j < RB ? 0 : l_lo) + ((size_t)row * lo.r + ks + (lane >> 4) * 8);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)p,
                                         (__attribute__((address_space(3))) void*)(dst + q * 512), 16, 0, 0);
      }
    }
    ring = (ring + 1) & (PP_STAGES - 1);
    ++load_kb;
    if constexpr (!plain) {
      if (load_kb == load_nst) {               // uniform
        load_kb = 0;
        load_L += G;
        load_block(load_L);
      }
    }
  };

  // ---- compute role: rows wn * 128 .., tokens wt * 64 ..
  const int wn = wave & 1, wt = wave >> 1;
  f32x4 acc[8][WTF];
  f16x8 a[2][8], b[2][WTF];
  int rd = 0;                                  // ring slot of the stage whose fragments are read next
  auto read_frags = [&](auto U) {
    constexpr int u = decltype(U)::value;
    const f16* st = smem + rd * PP_STAGE_ELEMS + lane * 8;
#pragma unroll
    for (int j = 0; j < WTF; ++j) b[u][j] = ld8(st + (PP_F + wt * WTF + j) * 512);
#pragma unroll
    for (int i = 0; i < 8; ++i) a[u][i] = ld8(st + (wn * 8 + i) * 512);
    rd = (rd + 1) & (PP_STAGES - 1);
  };
  // half (uniform): -1 all eight row tiles, 0 / 1 the first / last four (a LoRA stage of the gate / up projection)
  auto multiply = [&](auto U, int half) {
    constexpr int u = decltype(U)::value;
    if (half != 1) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < WTF; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
    }
    if (half != 0) {
#pragma unroll
      for (int i = 4; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < WTF; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
    }
  };
  // One stage: its successor must be in LDS (this wave's share: at most the two stages issued after it still in flight;
  // everybody's: the barrier).  The wait also covers this wave's fragment reads of the stage about to be multiplied,
  // so after the barrier nobody reads that ring slot any more and it is refilled; then the reads of the successor go
  // out, then the MFMAs.
  auto stage = [&](auto U, auto PLAIN, int half) {
    constexpr int u = decltype(U)::value;
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    issue(PLAIN);
    read_frags(std::integral_constant<int, 1 - u>());
    __builtin_amdgcn_sched_barrier(0);
    multiply(U, half);
    __builtin_amdgcn_sched_barrier(0);
  };

  load_block(load_L);
  issue(std::false_type());
  issue(std::false_type());
  issue(std::false_type());
  asm volatile("s_waitcnt vmcnt(8)" ::: "memory");     // the first stage of this wave has landed
  __syncthreads();
  issue(std::false_type());
  read_frags(std::integral_constant<int, 0>());
  f16* ostage = smem + PP_STAGES * PP_STAGE_ELEMS + wave * PP_OUT_ELEMS;
  const int r16 = lane & 15, g = lane >> 4;
  for (int L = blockIdx.x; L < nb; L += G) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < WTF; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    int n0, t0;
    block_of(L, n0, t0);
    int nst = KB;                                      // KB and E are even (checked by the launcher): the register sets alternate
    if constexpr (LORA) {
      int slot;
      if (lora_of(n0, t0, slot) >= 0) nst += E;
      nst = __builtin_amdgcn_readfirstlane(nst);
    }
    for (int kb = 0; kb < nst; kb += 2) {
      // (the plain GEMM keeps one copy of the pair: with two, the compiler's register allocation of this loop falls apart)
      if constexpr (SILU && LORA) {
        // one copy of the pair; a pair of LoRA stages belongs to one projection and multiplies that half of the tiles only
        const int half = kb < KB ? -1 : (has_gate && kb - KB < EP ? 0 : 1);   // uniform
        stage(std::integral_constant<int, 0>(), std::false_type(), half);
        stage(std::integral_constant<int, 1>(), std::false_type(), half);
      } else if (LORA && load_kb + 2 < KB) {             // uniform: the two stages fetched next are ordinary k-steps inside their block
        stage(std::integral_constant<int, 0>(), std::true_type(), -1);
        stage(std::integral_constant<int, 1>(), std::true_type(), -1);
      } else {
        stage(std::integral_constant<int, 0>(), std::false_type(), -1);
        stage(std::integral_constant<int, 1>(), std::false_type(), -1);
      }
    }
    if constexpr (SILU) {
      // acc[i] and acc[4 + i] are the gate and the up half of channels n0 + wn * 64 + i * 16 + 4 g .. + 3 for token r16 of
      // token fragment j: four products = one 8-byte piece of the output fragment; the pieces of a store instruction
      // are 512 contiguous bytes
#pragma unroll
      for (int j = 0; j < WTF; ++j) {
        const int t = t0 + (wt * WTF + j) * 16 + r16;
        if ((t >> 4) >= x_tt) continue;                  // the token tile does not exist
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c = n0 + (wn * 4 + i) * 16 + g * 4;
          if (c >= I) continue;
          f16x4 o = f16x4{0, 0, 0, 0};                   // rows past T inside the last tile: zeros, as the separate kernel writes them
          if (t < T) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float gf = (float)(f16)acc[i][j][r];
              o[r] = (f16)(gf / (1.f + expf(-gf)) * (float)(f16)acc[4 + i][j][r]);
            }
          }
          *reinterpret_cast<f16x4*>((f16*)yv + ((size_t)(c >> 5) * x_tt + (t >> 4)) * 512 + ((c & 31) >> 3) * 128 + (t & 15) * 8 + (c & 7)) = o;
        }
      }
    } else if constexpr (OUT == OUT_F16) {
      // 16 tokens x 64 columns at a time through the wave's staging buffer: D[n][t] fragments in, token rows out
#pragma unroll
      for (int j = 0; j < WTF; ++j) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const f32x4 sacc = acc[h * 4 + i][j];
            *reinterpret_cast<f16x4*>(ostage + r16 * PP_OUT_LD + i * 16 + g * 4) = f16x4{(f16)sacc[0], (f16)sacc[1], (f16)sacc[2], (f16)sacc[3]};
          }
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int c = q * 64 + lane;           // 16-byte chunk: token row c / 8, columns (c % 8) * 8 ..
            const int tr = c >> 3, cc = (c & 7) * 8;
            const int t = t0 + (wt * WTF + j) * 16 + tr;
            const int n = n0 + (wn * 8 + h * 4) * 16 + cc;
            const f16x4 lo = *reinterpret_cast<const f16x4*>(ostage + tr * PP_OUT_LD + cc);
            const f16x4 hi = *reinterpret_cast<const f16x4*>(ostage + tr * PP_OUT_LD + cc + 4);
            if (t < T && n + 8 <= N) {
              st8((f16*)yv + (size_t)t * N + n, f16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
            } else if (t < T) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if (n + e < N) ((f16*)yv)[(size_t)t * N + n + e] = lo[e];
                if (n + 4 + e < N) ((f16*)yv)[(size_t)t * N + n + 4 + e] = hi[e];
              }
            }
          }
          __builtin_amdgcn_wave_barrier();
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < WTF; ++j) {
        const int t = t0 + (wt * WTF + j) * 16 + r16;
        if (t >= T) continue;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int n = n0 + (wn * 8 + i) * 16 + g * 4;
          if (n >= N) continue;
          const size_t o = (size_t)t * N + n;
          if constexpr (OUT == OUT_F32) {
            *reinterpret_cast<f32x4*>((float*)yv + o) = acc[i][j];
          } else {
            f32x4* p = reinterpret_cast<f32x4*>((float*)yv + o);
            *p = *p + acc[i][j];
          }
        }
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // the loads issued past the last block must not outlive the workgroup's LDS
}

template <int OUT>
int launch_gemm_pp(void* y, const f16* x, int ldx, int x_tt, const f16* Wp, int T, int K, int N, hipStream_t s,
                   const PPLora& lo = PPLora()) {
  constexpr size_t lds = ((size_t)PP_STAGES * PP_STAGE_ELEMS + (size_t)PP_WAVES * PP_OUT_ELEMS) * sizeof(f16);
  // the attribute is per kernel, set once per process (the initialiser of a local static runs once, also when several
  // host threads make their first call together)
  static const hipError_t configured = [] {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_pp_kernel<OUT, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)gemm_pp_kernel<OUT, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    return e;
  }();
  if (configured != hipSuccess)
    return mlora_set_error(MLORA_ERR_LAUNCH, "gemm_packed: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(configured));
  const int gx = OUT == OUT_SILU ? ceil_div(N / 2, PP_F * 8) : ceil_div(N, PP_F * 16), gy = ceil_div(T, PP_F * 16);
  int n_cu = gemm_n_cu();
  if (n_cu <= 0) n_cu = 256;
  const int grid = gx * gy < n_cu ? gx * gy : n_cu;
  if (lo.n_proj > 0) hipLaunchKernelGGL((gemm_pp_kernel<OUT, true>), dim3(grid), dim3(PP_WAVES * WAVE), lds, s, y, x, ldx, x_tt, Wp, T, K, N, gx, gy, lo);
  else hipLaunchKernelGGL((gemm_pp_kernel<OUT, false>), dim3(grid), dim3(PP_WAVES * WAVE), lds, s, y, x, ldx, x_tt, Wp, T, K, N, gx, gy, lo);
  return MLORA_OK;
}

// ---------------------------------------------------------------------------------------------
// Token blocks between the decode GEMV and the persistent kernel above (65 to a few hundred tokens: a decode step of
// many sequences, a short prefill).  The weights are read once and the matrix cores and the operand loads weigh about
// the same, so the block is as tall as the token block allows and narrow enough to give every compute unit a
// workgroup: FT x FN fragments (128 or 256 tokens x 128, 96 or 64 weight rows), eight waves, both operands in fragment
// order and copied from global memory straight into an LDS ring.  A stage of the ring is TWO 32-k steps: with the
// few MFMAs a wave has per 32-k step here (4 to 16), a barrier and a wait per step cost more than the step itself.
// Four (three) stages, of which three (two) are in flight per compute unit - across the barrier of a stage, which is
// the bare instruction (bare_barrier): behind __syncthreads() the compiler first waits for every request in flight,
// the ring ran as if it had one stage and the launch pulled 2 to 3.4 TB/s of weights whatever its depth.
// What bounds the kernel now is what the second-level caches hand to the compute units: at 256 tokens the counters
// show 417 MB of requests per 100 MB matrix (each weight fragment for two token blocks, the token block once per
// row block), 70 % of them hits, delivered at 8 to 10 TB/s over the chip - every tiling that gives all compute units
// a workgroup has to take in about that much.
// grid = (weight-row blocks, K slices, token blocks).
// With K slices, slice 0 produces the result proper (store or accumulate) and slice s > 0 stores its fp32 partial
// sums to part[s - 1][T][ld_part] - for the two narrow accumulating linears of a layer, whose partials the next
// RMSNorm of the row adds in slice order.
// ---------------------------------------------------------------------------------------------
constexpr int MID_KS = 2;                      // 32-k steps per stage

template <int OUT, int FT, int FN>
__global__ __launch_bounds__(PP_WAVES* WAVE, 2) void gemm_mid_kernel(void* __restrict__ yv, float* __restrict__ part, int ld_part,
                                                                    const f16* __restrict__ xf, int x_tt, const f16* __restrict__ Wp,
                                                                    int T, int K, int N) {
  constexpr int MID_STAGES = FT == 16 ? 3 : 4;
  constexpr int SF = FN + FT;                  // fragments of one 32-k step: weights, then tokens
  constexpr int LF = MID_KS * SF;              // fragments per stage
  constexpr int LQ = (LF + PP_WAVES - 1) / PP_WAVES;   // ... of which a wave fetches LQ (fragment f = wave + 8 q: fragment f % SF of k-step f / SF)
  constexpr int LREM = LF % PP_WAVES;          // ... or, when they do not divide, the waves from LREM on one fewer
  constexpr int STAGE_ELEMS = LF * 512;
  constexpr int WTF = FT / 4;                  // token fragments of a wave's tile
  constexpr int WNF = FN / 2;                  // weight fragments of a wave's tile
  constexpr int VM = (MID_STAGES - 2) * LQ;    // a wave's loads that may still be in flight when the next stage is read
  constexpr int VM1 = (MID_STAGES - 2) * (LQ - 1);   // ... for the waves with one fragment fewer
  static_assert(FT % 4 == 0 && FN % 2 == 0 && WNF <= 4, "the tile divides over the waves");
  static_assert(VM == 5 || VM == 6 || VM == 8, "wait_next has an instruction for each of these");
  static_assert(LREM == 0 || VM1 == 5 || VM1 == 6, "wait_next has an instruction for each of these");
  extern __shared__ __align__(16) f16 smem[];  // [MID_STAGES][STAGE_ELEMS]; the output staging reuses it after the K loop
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int KB = K / 32;
  const int tiles = (N + 15) / 16;
  const int n0 = blockIdx.x * FN * 16, t0 = blockIdx.z * FT * 16;
  const int per = (KB + gridDim.y - 1) / gridDim.y;
  const int kb0 = blockIdx.y * per;
  const int kb1 = kb0 + per < KB ? kb0 + per : KB;
  const int nks = kb1 - kb0;                   // 32-k steps of this slice (>= 1: checked by the launcher)
  const int nst = (nks + MID_KS - 1) / MID_KS; // stages

  const f16* src[LQ];
  int step[LQ], kso[LQ];
#pragma unroll
  for (int q = 0; q < LQ; ++q) {
    const int f = (wave + PP_WAVES * q) % SF;  // uniform (past LF for the last q of a wave with one fewer: set up, never issued)
    kso[q] = (wave + PP_WAVES * q) / SF;
    if (f < FN) {
      int nt = n0 / 16 + f;
      nt = nt < tiles ? nt : tiles - 1;        // rows past N: a valid fragment, results dropped
      src[q] = Wp + (size_t)nt * KB * 512 + lane * 8;
      step[q] = 512;
    } else {
      int tt = t0 / 16 + f - FN;
      tt = tt < x_tt ? tt : x_tt - 1;          // tiles past T: a valid fragment, results dropped
      src[q] = xf + (size_t)tt * 512 + lane * 8;
      step[q] = x_tt * 512;
    }
  }
  int ring = 0, load_kb = kb0;
  auto issue = [&]() {
    f16* dst = smem + ring * STAGE_ELEMS + wave * 512;
#pragma unroll
    for (int q = 0; q < LQ; ++q) {
      if (LREM != 0 && q == LQ - 1 && wave >= LREM) break;      // uniform
      int kb = load_kb + kso[q];
      kb = kb < kb1 ? kb : kb1 - 1;            // past the slice: a valid address; the data is not multiplied
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[q] + (size_t)kb * step[q]),
                                       (__attribute__((address_space(3))) void*)(dst + q * PP_WAVES * 512), 16, 0, 0);
    }
    ring = ring + 1 == MID_STAGES ? 0 : ring + 1;
    load_kb += MID_KS;
  };

  const int wn = wave & 1, wt = wave >> 1;     // weight rows wn * WNF * 16 .., tokens wt * WTF * 16 ..
  f32x4 acc[WNF][WTF];
  f16x8 a[2][MID_KS][WNF], b[2][MID_KS][WTF];  // two register sets: the stage being multiplied and its successor
#pragma unroll
  for (int i = 0; i < WNF; ++i)
#pragma unroll
    for (int j = 0; j < WTF; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  int rd = 0;
  auto read_frags = [&](auto U) {
    constexpr int u = decltype(U)::value;
    const f16* st = smem + rd * STAGE_ELEMS + lane * 8;
#pragma unroll
    for (int ks = 0; ks < MID_KS; ++ks) {
#pragma unroll
      for (int j = 0; j < WTF; ++j) b[u][ks][j] = ld8(st + (ks * SF + FN + wt * WTF + j) * 512);
#pragma unroll
      for (int i = 0; i < WNF; ++i) a[u][ks][i] = ld8(st + (ks * SF + wn * WNF + i) * 512);
    }
    rd = rd + 1 == MID_STAGES ? 0 : rd + 1;
  };
  int done_ks = 0;                             // 32-k steps multiplied so far
  auto multiply = [&](auto U) {
    constexpr int u = decltype(U)::value;
#pragma unroll
    for (int ks = 0; ks < MID_KS; ++ks) {
      if (done_ks + ks < nks) {                // uniform: the last stage of an odd slice holds one step only
#pragma unroll
        for (int i = 0; i < WNF; ++i)
#pragma unroll
          for (int j = 0; j < WTF; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][ks][i], b[u][ks][j], acc[i][j], 0, 0, 0);
      }
    }
    done_ks += MID_KS;
  };
  // the wait: of this wave's loads at most those of the MID_STAGES - 2 youngest stages are still in flight, so the
  // stage multiplied next has landed; with everybody's wait and fragment reads behind the barrier, the slot of the
  // stage just read is refilled
  auto wait_next = [&]() {
    if (LREM != 0 && wave >= LREM) {             // uniform
      if constexpr (VM1 == 5) asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
      return;
    }
    if constexpr (VM == 5) asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory");
    else if constexpr (VM == 6) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
  };
  auto stage = [&](auto U) {
    constexpr int u = decltype(U)::value;
    wait_next();
    bare_barrier();
    issue();
    read_frags(std::integral_constant<int, 1 - u>());
    __builtin_amdgcn_sched_barrier(0);
    multiply(U);
    __builtin_amdgcn_sched_barrier(0);
  };
#pragma unroll
  for (int i = 0; i < MID_STAGES - 1; ++i) issue();
  wait_next();
  bare_barrier();
  issue();
  read_frags(std::integral_constant<int, 0>());
  int g = 0;
  for (; g + 1 < nst; g += 2) {
    stage(std::integral_constant<int, 0>());
    stage(std::integral_constant<int, 1>());
  }
  if (g < nst) stage(std::integral_constant<int, 0>());
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // nothing is in flight into the LDS that the epilogue reuses
  __syncthreads();

  const int r16 = lane & 15, gq = lane >> 4;
  if (blockIdx.y > 0) {                        // a later K slice: fp32 partial sums
    float* pp = part + (size_t)(blockIdx.y - 1) * T * ld_part;
#pragma unroll
    for (int j = 0; j < WTF; ++j) {
      const int t = t0 + (wt * WTF + j) * 16 + r16;
      if (t >= T) continue;
#pragma unroll
      for (int i = 0; i < WNF; ++i) {
        const int n = n0 + (wn * WNF + i) * 16 + gq * 4;
        if (n < N) *reinterpret_cast<f32x4*>(pp + (size_t)t * ld_part + n) = acc[i][j];
      }
    }
    return;
  }
  if constexpr (OUT == OUT_F16) {
    // 16 tokens x (16 WNF) columns at a time through the wave's staging buffer: D[n][t] fragments in, token rows out
    f16* ostage = smem + wave * PP_OUT_ELEMS;
    constexpr int CPR = WNF * 2;               // 16-byte chunks per token row
#pragma unroll
    for (int j = 0; j < WTF; ++j) {
#pragma unroll
      for (int i = 0; i < WNF; ++i) {
        const f32x4 sacc = acc[i][j];
        *reinterpret_cast<f16x4*>(ostage + r16 * PP_OUT_LD + i * 16 + gq * 4) = f16x4{(f16)sacc[0], (f16)sacc[1], (f16)sacc[2], (f16)sacc[3]};
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int q = 0; q < (16 * CPR + WAVE - 1) / WAVE; ++q) {
        const int c = q * 64 + lane;             // 16-byte chunk: token row c / CPR, columns (c % CPR) * 8 ..
        if ((16 * CPR) % WAVE != 0 && c >= 16 * CPR) break;
        const int tr = c / CPR, cc = (c % CPR) * 8;
        const int t = t0 + (wt * WTF + j) * 16 + tr;
        const int n = n0 + wn * WNF * 16 + cc;
        const f16x4 lo = *reinterpret_cast<const f16x4*>(ostage + tr * PP_OUT_LD + cc);
        const f16x4 hi = *reinterpret_cast<const f16x4*>(ostage + tr * PP_OUT_LD + cc + 4);
        if (t < T && n + 8 <= N) {
          st8((f16*)yv + (size_t)t * N + n, f16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
        } else if (t < T) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e < N) ((f16*)yv)[(size_t)t * N + n + e] = lo[e];
            if (n + 4 + e < N) ((f16*)yv)[(size_t)t * N + n + 4 + e] = hi[e];
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  } else {
#pragma unroll
    for (int j = 0; j < WTF; ++j) {
      const int t = t0 + (wt * WTF + j) * 16 + r16;
      if (t >= T) continue;
#pragma unroll
      for (int i = 0; i < WNF; ++i) {
        const int n = n0 + (wn * WNF + i) * 16 + gq * 4;
        if (n >= N) continue;
        const size_t o = (size_t)t * N + n;
        if constexpr (OUT == OUT_F32) {
          *reinterpret_cast<f32x4*>((float*)yv + o) = acc[i][j];
        } else {
          f32x4* p = reinterpret_cast<f32x4*>((float*)yv + o);
          *p = *p + acc[i][j];
        }
      }
    }
  }
}

// Block shape and K slices of the mid-size kernel for a shape: 128-token blocks when 256-token ones would leave most
// compute units without a workgroup, and 64 weight rows per block instead of 128 when that still leaves half of them
// idle (up to 128 tokens: 170 instead of 192 us for the four linears of a 4096 / 11008 layer; with two token blocks
// the narrow form loses, so it is not taken there); 96 rows for the launches without K slices where that fills more
// units in the same number of rounds.
struct MidShape {
  int ft, fn, ksplit;
};
MidShape gemm_mid_shape(int T, int K, int N, int ksplit_max) {
  const int by_k = (K / 32) / 16 < 1 ? 1 : (K / 32) / 16;   // at least 16 k-steps per slice
  const int ks_cap = ksplit_max < by_k ? ksplit_max : by_k;
  MidShape m;
  const int cols8 = ceil_div(N, 128);
  m.ft = (T <= 128 || (long)cols8 * ceil_div(T, 256) * ksplit_max <= 128) ? 8 : 16;
  const int tb = ceil_div(T, m.ft * 16);
  m.fn = (long)cols8 * tb * ks_cap <= 128 ? 4 : 8;
  if (ks_cap == 1 && m.fn == 8) {
    // 96 rows per block where that takes no more rounds of the compute units than 128: more units busy, fewer bytes
    // per workgroup (q/k/v at 256 tokens: 256 workgroups instead of 192, 43.9 -> 41.2 us; gate/up 230 instead of 172,
    // 69.0 -> 63.3 us)
    int n_cu = gemm_n_cu();
    if (n_cu <= 0) n_cu = 256;
    const int w8 = cols8 * tb, w6 = ceil_div(N, 96) * tb;
    if (ceil_div(w6, n_cu) * (m.ft + 6) < ceil_div(w8, n_cu) * (m.ft + 8)) m.fn = 6;
  }
  const int cols = ceil_div(N, m.fn * 16);
  int ks = 256 / (cols * tb);
  if (ks > ks_cap) ks = ks_cap;
  m.ksplit = ks < 1 ? 1 : ks;
  return m;
}

template <int OUT, int FT, int FN>
int launch_gemm_mid_shape(void* y, float* part, int ld_part, int ksplit, const f16* xf, int x_tt, const f16* Wp, int T, int K, int N,
                          hipStream_t s) {
  constexpr size_t lds = (size_t)(FT == 16 ? 3 : 4) * MID_KS * (FN + FT) * 512 * sizeof(f16);
  static_assert(lds >= (size_t)PP_WAVES * PP_OUT_ELEMS * sizeof(f16), "the output staging fits the ring");
  static const hipError_t configured =               // the attribute is per kernel, set once per process, by one thread
      hipFuncSetAttribute((const void*)gemm_mid_kernel<OUT, FT, FN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (configured != hipSuccess)
    return mlora_set_error(MLORA_ERR_LAUNCH, "linear_frag: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(configured));
  const dim3 grid(ceil_div(N, FN * 16), ksplit, ceil_div(T, FT * 16));
  hipLaunchKernelGGL((gemm_mid_kernel<OUT, FT, FN>), grid, dim3(PP_WAVES * WAVE), lds, s, y, part, ld_part, xf, x_tt, Wp, T, K, N);
  return MLORA_OK;
}

template <int OUT>
int launch_gemm_mid(void* y, float* part, int ld_part, const MidShape& m, const f16* xf, int x_tt, const f16* Wp, int T, int K, int N,
                    hipStream_t s) {
  if (m.ft == 8) {
    if (m.fn == 4) return launch_gemm_mid_shape<OUT, 8, 4>(y, part, ld_part, m.ksplit, xf, x_tt, Wp, T, K, N, s);
    if (m.fn == 6) return launch_gemm_mid_shape<OUT, 8, 6>(y, part, ld_part, m.ksplit, xf, x_tt, Wp, T, K, N, s);
    return launch_gemm_mid_shape<OUT, 8, 8>(y, part, ld_part, m.ksplit, xf, x_tt, Wp, T, K, N, s);
  }
  if (m.fn == 4) return launch_gemm_mid_shape<OUT, 16, 4>(y, part, ld_part, m.ksplit, xf, x_tt, Wp, T, K, N, s);
  if (m.fn == 6) return launch_gemm_mid_shape<OUT, 16, 6>(y, part, ld_part, m.ksplit, xf, x_tt, Wp, T, K, N, s);
  return launch_gemm_mid_shape<OUT, 16, 8>(y, part, ld_part, m.ksplit, xf, x_tt, Wp, T, K, N, s);
}

template <int OUT, int FT, int FN, int WT_, int WN_>
int launch_gemm_lds(void* y, const f16* x, int ldx, const f16* Wp, int T, int K, int N, hipStream_t s) {
  constexpr size_t lds = 2 * (LBK / 32) * (FT + FN) * 512 * sizeof(f16);
  static const hipError_t configured =               // the attribute is per kernel, set once per process, by one thread
      lds > 64 * 1024 ? hipFuncSetAttribute((const void*)gemm_lds_kernel<OUT, FT, FN, WT_, WN_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)
                      : hipSuccess;
  if (configured != hipSuccess)
    return mlora_set_error(MLORA_ERR_LAUNCH, "gemm_packed: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(configured));
  hipLaunchKernelGGL((gemm_lds_kernel<OUT, FT, FN, WT_, WN_>), dim3(ceil_div(N, FN * 16), ceil_div(T, FT * 16)), dim3(256), lds, s,
                     y, x, ldx, Wp, T, K, N);
  return MLORA_OK;
}

// Block shape by problem size: 256 x 256 (wave 128 x 128) when there are enough blocks to fill the chip, else
// 256 tokens x 64 columns (wave 64 x 64, several workgroups per CU) so that a few hundred tokens still spread
// over all CUs.
template <int OUT>
int launch_gemm_lds_auto(void* y, const f16* x, int ldx, const f16* Wp, int T, int K, int N, hipStream_t s) {
  if ((long)ceil_div(T, 256) * ceil_div(N, 256) >= 256) {
    // x rows must be 16-byte aligned for the direct-to-LDS loads (ldx % 8 == 0 is checked; the base may be a slice)
    if (((uintptr_t)x & 15) == 0 && K % 64 == 0) return launch_gemm_pp<OUT>(y, x, ldx, 0, Wp, T, K, N, s);
    return launch_gemm_lds<OUT, 16, 16, 8, 8>(y, x, ldx, Wp, T, K, N, s);
  }
  return launch_gemm_lds<OUT, 16, 4, 4, 4>(y, x, ldx, Wp, T, K, N, s);
}

template <bool PACKED>
int gemm_dispatch(const char* who, void* y, int y_dtype, int mode, const void* x, int ldx, const void* W, int T, int K,
                  int N, void* stream) {
  if (int e = mlora_check_linear(who, y, y_dtype, mode, x, ldx, W, T, K, N)) return e;
  if (T == 0) return MLORA_OK;
  MLORA_CHECK(ceil_div(T, 128) <= 65535, MLORA_ERR_UNSUPPORTED, "%s: T=%d too large", who, T);
  const dim3 grid(ceil_div(N, 128), ceil_div(T, 128)), block(256);
  hipStream_t s = (hipStream_t)stream;
  const f16* xp = (const f16*)x;
  const f16* Wp = (const f16*)W;
  if constexpr (PACKED) {
    if (T > 128) {
      int e;
      if (mode == MLORA_ACCUMULATE) e = launch_gemm_lds_auto<OUT_ACC_F32>(y, xp, ldx, Wp, T, K, N, s);
      else if (y_dtype == MLORA_F32) e = launch_gemm_lds_auto<OUT_F32>(y, xp, ldx, Wp, T, K, N, s);
      else e = launch_gemm_lds_auto<OUT_F16>(y, xp, ldx, Wp, T, K, N, s);
      return e ? e : mlora_launch_status(who);
    }
  }
  if (mode == MLORA_ACCUMULATE) hipLaunchKernelGGL((gemm_kernel<OUT_ACC_F32, PACKED>), grid, block, 0, s, y, xp, ldx, Wp, T, K, N);
  else if (y_dtype == MLORA_F32) hipLaunchKernelGGL((gemm_kernel<OUT_F32, PACKED>), grid, block, 0, s, y, xp, ldx, Wp, T, K, N);
  else hipLaunchKernelGGL((gemm_kernel<OUT_F16, PACKED>), grid, block, 0, s, y, xp, ldx, Wp, T, K, N);
  return mlora_launch_status(who);
}

}  // namespace

extern "C" int mlora_gemm(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W, int T, int K, int N,
                          void* stream) {
  return gemm_dispatch<false>("gemm", y, y_dtype, mode, x, ldx, W, T, K, N, stream);
}

extern "C" int mlora_gemm_packed(void* y, int y_dtype, int mode, const void* x, int ldx, const void* Wp, int T, int K,
                                 int N, void* stream) {
  return gemm_dispatch<true>("gemm_packed", y, y_dtype, mode, x, ldx, Wp, T, K, N, stream);
}

extern "C" int mlora_linear(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W, int T, int K, int N,
                            void* stream) {
  if (T <= 64) return mlora_gemv(y, y_dtype, mode, x, ldx, W, T, K, N, stream);
  return mlora_gemm(y, y_dtype, mode, x, ldx, W, T, K, N, stream);
}

extern "C" int mlora_linear_packed(void* y, int y_dtype, int mode, const void* x, int ldx, const void* Wp, int T, int K,
                                   int N, void* stream) {
  if (T <= 64) return mlora_gemv_packed(y, y_dtype, mode, x, ldx, Wp, T, K, N, stream);
  return mlora_gemm_packed(y, y_dtype, mode, x, ldx, Wp, T, K, N, stream);
}

extern "C" int mlora_gemv_frag(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N, void* stream);

// 256 x 256 output blocks: enough of them to give every compute unit one, and whole pairs of 32-k steps
extern "C" int mlora_gemm_frag_preferred(int T, int K, int N) {
  return T > 64 && K > 0 && K % 64 == 0 && N > 0 && (long)ceil_div(T, PP_F * 16) * ceil_div(N, PP_F * 16) >= 256;
}

extern "C" int mlora_linear_frag(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N,
                                 void* stream) {
  if (T <= 64) return mlora_gemv_frag(y, y_dtype, mode, xf, Wp, T, K, N, stream);
  if (int e = mlora_check_linear("linear_frag", y, y_dtype, mode, xf, K, Wp, T, K, N)) return e;
  MLORA_CHECK(K % 32 == 0, MLORA_ERR_UNSUPPORTED, "linear_frag: K %% 32 != 0 (K=%d)", K);
  MLORA_CHECK(((uintptr_t)xf & 15) == 0, MLORA_ERR_INVALID, "linear_frag: xf must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const f16* x = (const f16*)xf;
  const f16* W = (const f16*)Wp;
  const int tt = mlora_frag_tiles(T);
  int e;
  if (mlora_gemm_frag_preferred(T, K, N)) {
    if (mode == MLORA_ACCUMULATE) e = launch_gemm_pp<OUT_ACC_F32>(y, x, 0, tt, W, T, K, N, s);
    else if (y_dtype == MLORA_F32) e = launch_gemm_pp<OUT_F32>(y, x, 0, tt, W, T, K, N, s);
    else e = launch_gemm_pp<OUT_F16>(y, x, 0, tt, W, T, K, N, s);
  } else {
    const MidShape m = gemm_mid_shape(T, K, N, 1);
    if (mode == MLORA_ACCUMULATE) e = launch_gemm_mid<OUT_ACC_F32>(y, nullptr, 0, m, x, tt, W, T, K, N, s);
    else if (y_dtype == MLORA_F32) e = launch_gemm_mid<OUT_F32>(y, nullptr, 0, m, x, tt, W, T, K, N, s);
    else e = launch_gemm_mid<OUT_F16>(y, nullptr, 0, m, x, tt, W, T, K, N, s);
  }
  return e ? e : mlora_launch_status("linear_frag");
}

extern "C" int mlora_linear_frag_lora(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N,
                                      const mlora_fused_lora* projs, int n_proj, const int32_t* blk_adapter, int r, void* stream) {
  if (int e = mlora_check_linear("linear_frag_lora", y, y_dtype, mode, xf, K, Wp, T, K, N)) return e;
  MLORA_CHECK(mlora_gemm_frag_preferred(T, K, N) && ((uintptr_t)xf & 15) == 0, MLORA_ERR_UNSUPPORTED,
              "linear_frag_lora: only shapes of the persistent GEMM (mlora_gemm_frag_preferred; T=%d K=%d N=%d)", T, K, N);
  MLORA_CHECK(projs && blk_adapter && n_proj >= 1 && n_proj <= 3 && (r == 32 || r == 64), MLORA_ERR_UNSUPPORTED,
              "linear_frag_lora: 1..3 projections of rank 32 or 64 (n_proj=%d r=%d)", n_proj, r);
  PPLora lo = {};
  for (int i = 0; i < n_proj; ++i) {
    const mlora_fused_lora& p = projs[i];
    MLORA_CHECK(p.B && p.v_hi && p.v_lo && (((uintptr_t)p.B | (uintptr_t)p.v_hi | (uintptr_t)p.v_lo) & 15) == 0, MLORA_ERR_INVALID,
                "linear_frag_lora: null or unaligned table of projection %d", i);
    // a 256-row block of the GEMM must lie inside one projection
    MLORA_CHECK(p.n_begin >= 0 && p.n_rows > 0 && p.n_begin % (PP_F * 16) == 0 && p.n_begin + p.n_rows <= N &&
                    (p.n_rows % (PP_F * 16) == 0 || p.n_begin + p.n_rows == N),
                MLORA_ERR_UNSUPPORTED, "linear_frag_lora: rows %d..%d of projection %d do not fall on 256-row blocks", p.n_begin,
                p.n_begin + p.n_rows, i);
    lo.B[i] = (const f16*)p.B; lo.vh[i] = (const f16*)p.v_hi; lo.vl[i] = (const f16*)p.v_lo;
    lo.n_begin[i] = p.n_begin; lo.n_rows[i] = p.n_rows;
  }
  lo.n_proj = n_proj; lo.r = r; lo.blk_adapter = blk_adapter;
  hipStream_t s = (hipStream_t)stream;
  const int tt = mlora_frag_tiles(T);
  int e;
  if (mode == MLORA_ACCUMULATE) e = launch_gemm_pp<OUT_ACC_F32>(y, (const f16*)xf, 0, tt, (const f16*)Wp, T, K, N, s, lo);
  else if (y_dtype == MLORA_F32) e = launch_gemm_pp<OUT_F32>(y, (const f16*)xf, 0, tt, (const f16*)Wp, T, K, N, s, lo);
  else e = launch_gemm_pp<OUT_F16>(y, (const f16*)xf, 0, tt, (const f16*)Wp, T, K, N, s, lo);
  return e ? e : mlora_launch_status("linear_frag_lora");
}

extern "C" int mlora_linear_frag_silu(void* act, const void* xf, const void* Wp, int T, int K, int I, const mlora_fused_lora* projs,
                                      int n_proj, const int32_t* blk_adapter, int r, void* stream) {
  MLORA_CHECK(act && xf && Wp, MLORA_ERR_INVALID, "linear_frag_silu: null pointer");
  MLORA_CHECK(T > 0 && K > 0 && I > 0 && I % 32 == 0 && I <= (1 << 29), MLORA_ERR_UNSUPPORTED,
              "linear_frag_silu: need I %% 32 == 0 (T=%d K=%d I=%d)", T, K, I);
  MLORA_CHECK(mlora_gemm_frag_preferred(T, K, 2 * I) && (((uintptr_t)xf | (uintptr_t)act) & 15) == 0, MLORA_ERR_UNSUPPORTED,
              "linear_frag_silu: only shapes of the persistent GEMM (mlora_gemm_frag_preferred; T=%d K=%d N=%d)", T, K, 2 * I);
  MLORA_CHECK(n_proj >= 0 && n_proj <= 2, MLORA_ERR_UNSUPPORTED, "linear_frag_silu: at most the gate and the up projection (n_proj=%d)", n_proj);
  PPLora lo = {};
  if (n_proj > 0) {
    MLORA_CHECK(projs && blk_adapter && (r == 32 || r == 64), MLORA_ERR_UNSUPPORTED,
                "linear_frag_silu: projections of rank 32 or 64 with the blocks' adapters (r=%d)", r);
    for (int i = 0; i < n_proj; ++i) {
      const mlora_fused_lora& p = projs[i];
      MLORA_CHECK(p.B && p.v_hi && p.v_lo && (((uintptr_t)p.B | (uintptr_t)p.v_hi | (uintptr_t)p.v_lo) & 15) == 0, MLORA_ERR_INVALID,
                  "linear_frag_silu: null or unaligned table of projection %d", i);
      MLORA_CHECK((p.n_begin == 0 || p.n_begin == I) && p.n_rows == I, MLORA_ERR_UNSUPPORTED,
                  "linear_frag_silu: projection %d must be the gate rows 0..I or the up rows I..2I (n_begin=%d n_rows=%d I=%d)", i,
                  p.n_begin, p.n_rows, I);
      const int slot = p.n_begin == 0 ? 0 : 1;
      MLORA_CHECK(lo.B[slot] == nullptr, MLORA_ERR_INVALID, "linear_frag_silu: two projections over the same rows");
      lo.B[slot] = (const f16*)p.B; lo.vh[slot] = (const f16*)p.v_hi; lo.vl[slot] = (const f16*)p.v_lo;
      lo.n_begin[slot] = p.n_begin; lo.n_rows[slot] = p.n_rows;
    }
    lo.n_proj = n_proj; lo.r = r; lo.blk_adapter = blk_adapter;
  }
  const int e = launch_gemm_pp<OUT_SILU>(act, (const f16*)xf, 0, mlora_frag_tiles(T), (const f16*)Wp, T, K, 2 * I, (hipStream_t)stream, lo);
  return e ? e : mlora_launch_status("linear_frag_silu");
}

// K slices the mid-size kernel would use for resid [T, N] += xf . Wp^T with at most ks_max slices (T > 64)
int mlora_gemm_mid_ksplit(int T, int K, int N, int ks_max) { return gemm_mid_shape(T, K, N, ks_max).ksplit; }

// resid [T, N] fp32 += xf . Wp^T over ks K slices: slice 0 into resid, slices 1.. into part[ks - 1][T][ld_part] (T > 64)
int mlora_gemm_mid_acc(float* resid, float* part, int ld_part, int ks, const void* xf, const void* Wp, int T, int K, int N,
                       void* stream) {
  MLORA_CHECK(K % 32 == 0 && ks >= 1 && (K / 32) / ks >= 1 && ((uintptr_t)xf & 15) == 0, MLORA_ERR_UNSUPPORTED,
              "linear_frag (K slices): need K %% 32 == 0 and at least one 32-k step per slice (K=%d ks=%d)", K, ks);
  MidShape m = gemm_mid_shape(T, K, N, ks);
  m.ksplit = ks;                               // the caller's partial buffers were sized for ks slices
  const int e = launch_gemm_mid<OUT_ACC_F32>(resid, part, ld_part, m, (const f16*)xf, mlora_frag_tiles(T), (const f16*)Wp, T, K, N,
                                             (hipStream_t)stream);
  return e ? e : mlora_launch_status("linear_frag (K slices)");
}
