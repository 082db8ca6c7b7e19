// Prefill-time base linear for gfx950:  y[T, N] (=|+=) x[T, K] . W[N, K]^T  for any T (MFMA-bound).
//
// Both operands are K-contiguous, which is the layout v_mfma_f32_16x16x32_f16 wants for its A and B
// fragments (a lane holds 8 consecutive k of one row), so fragments are loaded straight from global
// memory with 16-byte loads and reuse comes from the register tile: a wave owns a 64 x 64 output tile
// (4 x 4 MFMA tiles, 16 MFMAs per 8 fragment loads), a workgroup of 4 waves owns 128 x 128, and the
// next k-step's fragments are in flight while the current one is multiplied.
#include "common.h"

int mlora_check_linear(const char* who, const void* y, int y_dtype, int mode, const void* x, int ldx, const void* W,
                       int T, int K, int N);

namespace {

enum { OUT_F16 = 0, OUT_F32 = 1, OUT_ACC_F32 = 2 };

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

template <int OUT, int FT, int FN, int WT_, int WN_>
int launch_gemm_lds(void* y, const f16* x, int ldx, const f16* Wp, int T, int K, int N, hipStream_t s) {
  constexpr size_t lds = 2 * (LBK / 32) * (FT + FN) * 512 * sizeof(f16);
  static bool configured = false;                    // the attribute is per kernel, set once per process
  if (!configured && lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_lds_kernel<OUT, FT, FN, WT_, WN_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return mlora_set_error(MLORA_ERR_LAUNCH, "gemm_packed: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    configured = true;
  }
  hipLaunchKernelGGL((gemm_lds_kernel<OUT, FT, FN, WT_, WN_>), dim3(ceil_div(N, FN * 16), ceil_div(T, FT * 16)), dim3(256), lds, s,
                     y, x, ldx, Wp, T, K, N);
  return MLORA_OK;
}

// Block shape by problem size: 256 x 256 (wave 128 x 128) when there are enough blocks to fill the chip, else
// 256 tokens x 64 columns (wave 64 x 64, several workgroups per CU) so that a few hundred tokens still spread
// over all CUs.
template <int OUT>
int launch_gemm_lds_auto(void* y, const f16* x, int ldx, const f16* Wp, int T, int K, int N, hipStream_t s) {
  if ((long)ceil_div(T, 256) * ceil_div(N, 256) >= 256) return launch_gemm_lds<OUT, 16, 16, 8, 8>(y, x, ldx, Wp, T, K, N, s);
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
