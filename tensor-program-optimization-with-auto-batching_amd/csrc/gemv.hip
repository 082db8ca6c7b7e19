// Decode-time base linear for gfx950:  y[T, N] (=|+=) x[T, K] . W[N, K]^T  with T <= 64.
//
// The weight matrix is read exactly once, straight from HBM into MFMA operand registers: for
// v_mfma_f32_16x16x32_f16 a lane holds 8 consecutive k of one row, so a wave-wide 16-byte load covers
// 16 weight rows x 64 contiguous bytes.  The token block x (T x K fp16, L2-resident) is the other
// operand, so one weight fragment is applied to 16 tokens per MFMA and the kernel stays HBM-bound
// (32 tokens need 64 flop per weight element - beyond the vector ALUs, well inside the matrix cores).
// A workgroup of 8 waves owns 16*NT rows of W and splits K eight ways; partial tiles are summed in a
// fixed order through LDS, so results do not depend on scheduling.
#include "common.h"

namespace {

constexpr int GEMV_WAVES = 8;
constexpr int KSTEP = 32;   // k per MFMA
constexpr int UNROLL = 4;   // k-steps in flight per wave

enum { OUT_F16 = 0, OUT_F32 = 1, OUT_ACC_F32 = 2 };

template <int NT, int TT, int OUT>
__global__ __launch_bounds__(GEMV_WAVES* WAVE) void gemv_kernel(void* __restrict__ yv, const f16* __restrict__ x, int ldx,
                                                                const f16* __restrict__ W, int T, int K, int N) {
  __shared__ f32x4 red[GEMV_WAVES][NT * TT][WAVE];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int r16 = lane & 15;
  const int kg = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT);

  const f16* wp[NT];
  const f16* xp[TT];
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    int n = n0 + i * 16 + r16;
    n = n < N ? n : N - 1;
    wp[i] = W + (size_t)n * K + kg * 8;
  }
#pragma unroll
  for (int j = 0; j < TT; ++j) {
    int t = j * 16 + r16;
    t = t < T ? t : T - 1;
    xp[j] = x + (size_t)t * ldx + kg * 8;
  }

  f32x4 acc[NT][TT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // wave w takes k-steps w, w + 8, w + 16, ...; UNROLL of them are in flight at once
  const int stride = GEMV_WAVES * KSTEP;
  for (int k = wave * KSTEP; k < K; k += stride * UNROLL) {
    f16x8 a[UNROLL][NT], b[UNROLL][TT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int ku = k + u * stride;
      const bool in = ku < K;
      const int kc = in ? ku : 0;
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        a[u][i] = __builtin_nontemporal_load(reinterpret_cast<const f16x8*>(wp[i] + kc));
        if (!in) a[u][i] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
#pragma unroll
      for (int j = 0; j < TT; ++j) b[u][j] = ld8(xp[j] + kc);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
  }

#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) red[wave][i * TT + j][lane] = acc[i][j];
  __syncthreads();

  // thread e < NT*TT*64 sums tile (e / 64), lane slot (e % 64) over the 8 waves in order
  for (int e = threadIdx.x; e < NT * TT * WAVE; e += GEMV_WAVES * WAVE) {
    const int tile = e >> 6, sl = e & 63;
    f32x4 s = red[0][tile][sl];
#pragma unroll
    for (int w = 1; w < GEMV_WAVES; ++w) s += red[w][tile][sl];
    const int i = tile / TT, j = tile % TT;
    const int n = n0 + i * 16 + (sl >> 4) * 4;   // D[n][t]: lane holds rows 4*(lane/16)..+3, column lane%16
    const int t = j * 16 + (sl & 15);
    if (t < T && n < N) {                         // N % 4 == 0: the 4 rows are inside together
      const size_t o = (size_t)t * N + n;
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

template <int NT, int TT>
void launch_gemv(void* y, int out, const f16* x, int ldx, const f16* W, int T, int K, int N, hipStream_t s) {
  const dim3 grid(ceil_div(N, 16 * NT)), block(GEMV_WAVES * WAVE);
  if (out == OUT_F16) hipLaunchKernelGGL((gemv_kernel<NT, TT, OUT_F16>), grid, block, 0, s, y, x, ldx, W, T, K, N);
  else if (out == OUT_F32) hipLaunchKernelGGL((gemv_kernel<NT, TT, OUT_F32>), grid, block, 0, s, y, x, ldx, W, T, K, N);
  else hipLaunchKernelGGL((gemv_kernel<NT, TT, OUT_ACC_F32>), grid, block, 0, s, y, x, ldx, W, T, K, N);
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
  const int out = mode == MLORA_ACCUMULATE ? OUT_ACC_F32 : (y_dtype == MLORA_F32 ? OUT_F32 : OUT_F16);
  hipStream_t s = (hipStream_t)stream;
  const f16* xp = (const f16*)x;
  const f16* Wp = (const f16*)W;
  // two 16-row tiles per wave once there are enough rows to give every CU two workgroups
  const bool wide = N >= 32 * 512;
  if (T <= 16) {
    if (wide) launch_gemv<2, 1>(y, out, xp, ldx, Wp, T, K, N, s);
    else launch_gemv<1, 1>(y, out, xp, ldx, Wp, T, K, N, s);
  } else if (T <= 32) {
    if (wide) launch_gemv<2, 2>(y, out, xp, ldx, Wp, T, K, N, s);
    else launch_gemv<1, 2>(y, out, xp, ldx, Wp, T, K, N, s);
  } else {
    launch_gemv<1, 4>(y, out, xp, ldx, Wp, T, K, N, s);
  }
  return mlora_launch_status("gemv");
}
