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
#include "lora_device.h"

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
                   int n_ad, hipStream_t s) {
  constexpr int CH = 8 * (WAVE / (R / 8));
  hipLaunchKernelGGL((lora_expand_kernel<R, YT>), dim3(n_ad, ceil_div(N, CH)), dim3(64), 0, s, y, vpart, B, ids, scaling,
                     T, N, ldy, lora_k_split(K).kc);
}

}  // namespace

extern "C" size_t mlora_gather_mm_workspace_bytes(int T, int K, int r) {
  if (T <= 0 || K <= 0 || r <= 0) return 0;
  return (size_t)lora_k_split(K).kc * (size_t)T * (size_t)r * sizeof(float);
}

extern "C" int mlora_lora_shrink(void* v_part, const void* x, int x_layout, const void* A, const int32_t* tok_adapter,
                                 int T, int K, int r, int n_ad, void* stream) {
  if (int e = check_lora_shape(T, K, 8, r, n_ad)) return e;
  MLORA_CHECK(x_layout == MLORA_ROWMAJOR || (x_layout == MLORA_FRAG && T <= 64 && K % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "lora_shrink: fragment-ordered x needs T <= 64 and K %% 32 == 0 (layout=%d T=%d K=%d)", x_layout, T, K);
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
  hipLaunchKernelGGL(lora_shrink_kernel, dim3(lora_shrink_units(b)), dim3(64), 0, (hipStream_t)stream, b);
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
