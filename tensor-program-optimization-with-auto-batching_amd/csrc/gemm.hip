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
