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
#include "common.h"

namespace {

constexpr int KCHUNK = 512;   // K elements one wave covers per pass: 64 lanes x 8 fp16
constexpr int MAX_KC = 8;     // K-slices (partials) per token

struct KSplit { int ci; int kc; };

KSplit k_split(int K) {
  int ci = ceil_div(K, KCHUNK * MAX_KC);
  if (ci < 1) ci = 1;
  return {ci, ceil_div(K, KCHUNK * ci)};
}

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
      const float send = hi ? p[i] : p[i + half];
      const float keep = hi ? p[i + half] : p[i];
      p[i] = keep + __shfl_xor(send, off, WAVE);
    }
    j += hi ? half : 0;
    off >>= 1;
  }
#pragma unroll
  for (; off > 0; off >>= 1) p[0] += __shfl_xor(p[0], off, WAVE);
  return j;
}

template <int R>
__global__ __launch_bounds__(64) void lora_shrink_kernel(float* __restrict__ vpart, const f16* __restrict__ x,
                                                         const f16* __restrict__ A,
                                                         const int32_t* __restrict__ ids, int T, int K, int CI,
                                                         int frag_tt) {
  constexpr int G = R < 16 ? R : 16;   // A rows held in registers at once
  constexpr int TB = 4;                // tokens in flight
  const int a = blockIdx.x;
  const int c = blockIdx.y;
  const int lane = threadIdx.x;
  const int kbase = c * CI * KCHUNK + lane * 8;

  for (int t0 = 0; t0 < T; t0 += WAVE) {
    const int id = (t0 + lane < T) ? ids[t0 + lane] : -1;
    unsigned long long mask = __ballot(id == a);
    while (mask) {
      int tt[TB];
#pragma unroll
      for (int u = 0; u < TB; ++u) {
        if (mask) {
          tt[u] = t0 + __builtin_ctzll(mask);
          mask &= mask - 1;
        } else {
          tt[u] = -1;
        }
      }
      for (int jb = 0; jb < R; jb += G) {
        float p[TB][G];
#pragma unroll
        for (int u = 0; u < TB; ++u)
#pragma unroll
          for (int j = 0; j < G; ++j) p[u][j] = 0.f;
        for (int ci = 0; ci < CI; ++ci) {
          const int k = kbase + ci * KCHUNK;
          const bool kin = k < K;
          f16x8 xv[TB];
#pragma unroll
          for (int u = 0; u < TB; ++u) {
            xv[u] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (kin && tt[u] >= 0) xv[u] = ld8(x + (frag_tt ? frag_offset(tt[u], k, frag_tt) : (size_t)tt[u] * K + k));
          }
          f16x8 areg[G];
#pragma unroll
          for (int j = 0; j < G; ++j) {
            areg[j] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (kin) areg[j] = ld8(A + ((size_t)a * R + jb + j) * K + k);
          }
#pragma unroll
          for (int u = 0; u < TB; ++u)
#pragma unroll
            for (int j = 0; j < G; ++j) p[u][j] = dot8(areg[j], xv[u], p[u][j]);
        }
#pragma unroll
        for (int u = 0; u < TB; ++u) {
          if (tt[u] < 0) continue;   // wave-uniform
          const int j = reduce_transpose<G>(p[u], lane);
          if ((lane & (WAVE / G - 1)) == 0) vpart[((size_t)c * T + tt[u]) * R + jb + j] = p[u][0];
        }
      }
    }
  }
}

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
                                                         int T, int N, int ldy, int KC) {
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
    const int id = (t0 + lane < T) ? ids[t0 + lane] : -1;
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
        for (int o = LPR >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, WAVE);
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
  MLORA_CHECK(n_ad <= 65535, MLORA_ERR_UNSUPPORTED, "gather_mm: n_ad=%d exceeds 65535", n_ad);
  return MLORA_OK;
}

template <int R>
void launch_shrink(float* vpart, const f16* x, int frag_tt, const f16* A, const int32_t* ids, int T, int K, int n_ad,
                   hipStream_t s) {
  const KSplit ks = k_split(K);
  hipLaunchKernelGGL(lora_shrink_kernel<R>, dim3(n_ad, ks.kc), dim3(64), 0, s, vpart, x, A, ids, T, K, ks.ci, frag_tt);
}

template <int R, typename YT>
void launch_expand(YT* y, int ldy, const float* vpart, const f16* B, const int32_t* ids, float scaling, int T, int K, int N,
                   int n_ad, hipStream_t s) {
  constexpr int CH = 8 * (WAVE / (R / 8));
  hipLaunchKernelGGL((lora_expand_kernel<R, YT>), dim3(n_ad, ceil_div(N, CH)), dim3(64), 0, s, y, vpart, B, ids, scaling,
                     T, N, ldy, k_split(K).kc);
}

}  // namespace

extern "C" size_t mlora_gather_mm_workspace_bytes(int T, int K, int r) {
  if (T <= 0 || K <= 0 || r <= 0) return 0;
  return (size_t)k_split(K).kc * (size_t)T * (size_t)r * sizeof(float);
}

extern "C" int mlora_lora_shrink(void* v_part, const void* x, int x_layout, const void* A, const int32_t* tok_adapter,
                                 int T, int K, int r, int n_ad, void* stream) {
  if (int e = check_lora_shape(T, K, 8, r, n_ad)) return e;
  MLORA_CHECK(x_layout == MLORA_ROWMAJOR || (x_layout == MLORA_FRAG && T <= 64 && K % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "lora_shrink: fragment-ordered x needs T <= 64 and K %% 32 == 0 (layout=%d T=%d K=%d)", x_layout, T, K);
  const int frag_tt = x_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  MLORA_CHECK(v_part && x && A && tok_adapter, MLORA_ERR_INVALID, "lora_shrink: null pointer");
  if (T == 0) return MLORA_OK;
  hipStream_t s = (hipStream_t)stream;
  float* vp = (float*)v_part;
  const f16* xp = (const f16*)x;
  const f16* Ap = (const f16*)A;
  switch (r) {
    case 8: launch_shrink<8>(vp, xp, frag_tt, Ap, tok_adapter, T, K, n_ad, s); break;
    case 16: launch_shrink<16>(vp, xp, frag_tt, Ap, tok_adapter, T, K, n_ad, s); break;
    case 32: launch_shrink<32>(vp, xp, frag_tt, Ap, tok_adapter, T, K, n_ad, s); break;
    default: launch_shrink<64>(vp, xp, frag_tt, Ap, tok_adapter, T, K, n_ad, s); break;
  }
  return mlora_launch_status("lora_shrink");
}

extern "C" int mlora_lora_expand(void* y, int y_dtype, int ldy, const void* v_part, const void* B,
                                 const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                                 void* stream) {
  if (int e = check_lora_shape(T, K, N, r, n_ad)) return e;
  MLORA_CHECK(ldy >= N && ldy % 8 == 0, MLORA_ERR_INVALID, "lora_expand: need ldy >= N and ldy %% 8 == 0 (ldy=%d N=%d)", ldy, N);
  MLORA_CHECK(y && v_part && B && tok_adapter, MLORA_ERR_INVALID, "lora_expand: null pointer");
  MLORA_CHECK(y_dtype == MLORA_F16 || y_dtype == MLORA_F32, MLORA_ERR_INVALID, "lora_expand: bad y_dtype %d", y_dtype);
  if (T == 0) return MLORA_OK;
  hipStream_t s = (hipStream_t)stream;
  const float* vp = (const float*)v_part;
  const f16* Bp = (const f16*)B;
#define MLORA_EXPAND(R)                                                                                   \
  if (y_dtype == MLORA_F16) launch_expand<R, f16>((f16*)y, ldy, vp, Bp, tok_adapter, scaling, T, K, N, n_ad, s); \
  else launch_expand<R, float>((float*)y, ldy, vp, Bp, tok_adapter, scaling, T, K, N, n_ad, s)
  switch (r) {
    case 8: MLORA_EXPAND(8); break;
    case 16: MLORA_EXPAND(16); break;
    case 32: MLORA_EXPAND(32); break;
    default: MLORA_EXPAND(64); break;
  }
#undef MLORA_EXPAND
  return mlora_launch_status("lora_expand");
}

extern "C" int mlora_gather_mm(void* y, int y_dtype, int ldy, const void* x, int x_layout, const void* A, const void* B,
                               const int32_t* tok_adapter, float scaling, int T, int K, int N, int r, int n_ad,
                               void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_lora_shape(T, K, N, r, n_ad)) return e;
  MLORA_CHECK(workspace && workspace_bytes >= mlora_gather_mm_workspace_bytes(T, K, r) || T == 0, MLORA_ERR_WORKSPACE,
              "gather_mm: workspace of %zu bytes given, %zu needed", workspace_bytes,
              mlora_gather_mm_workspace_bytes(T, K, r));
  if (int e = mlora_lora_shrink(workspace, x, x_layout, A, tok_adapter, T, K, r, n_ad, stream)) return e;
  return mlora_lora_expand(y, y_dtype, ldy, workspace, B, tok_adapter, scaling, T, K, N, r, n_ad, stream);
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
