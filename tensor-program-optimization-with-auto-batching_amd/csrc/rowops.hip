// Row-wise operators for gfx950: RMSNorm, SiLU*mul, embedding gather, argmax.
// All are a few hundred KiB per call at decode batch sizes - one pass over the row in registers,
// 64-lane wave reductions, one LDS exchange between the waves of a block.
#include "lora_device.h"

namespace {

constexpr int ROW_THREADS = 256;

// LoRA expand carried by the RMSNorm launch: resid[t, :] += scaling * B[id_t] . v[t] before the row is normed.
struct LoraExpandRow {
  LoraVSource src;      // shrink results, one slot (src.v == nullptr: plain RMSNorm)
  const f16* B;         // [n_ad, H, r]
  const int32_t* ids;
  float scaling;
  int r, n_ad;
};

// Partial results of a K-split GEMV that accumulated into the row being normed: n blocks [T][ld] fp32, `stride`
// elements apart; columns 0..H-1 belong to the row, columns from H on to the appended adapter rows (dense shrink).
constexpr int MAX_PARTS = 3;
struct KSplitParts {
  const float* p;
  int n, ld;
  size_t stride;
};

template <int NTHREADS>
__device__ __forceinline__ float block_sum(float v, float* lds) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < NTHREADS / WAVE; ++w) s += lds[w];
  return s;
}

constexpr int NORM_THREADS = 512;

// One block of 512 threads per row; each thread keeps up to VPT 8-element vectors of the row in registers.
// With a LoRA expand attached (fp32 rows only) the block first streams B[id_row] ([H, r] fp16, coalesced 16-byte
// chunks, r/8 lanes per output column combined by shuffles), stages the H deltas in LDS, adds them to the
// residual row in place, and then norms the updated row.
// With PARTS the K-split partials of the row are added after the expand, in slice order, and the row is stored back.
template <typename XT, int VPT, bool PARTS = false>
__global__ __launch_bounds__(NORM_THREADS) void rmsnorm_kernel(f16* __restrict__ y, XT* __restrict__ x,
                                                               const f16* __restrict__ w, float eps, int H, int frag_tt,
                                                               LoraExpandRow lx, KSplitParts kp) {
  __shared__ float lds[NORM_THREADS / WAVE];
  __shared__ float lv[64];
  extern __shared__ float delta[];    // H floats when a LoRA expand is attached, otherwise empty
  // every argument is fetched now, in one round of scalar loads (left alone, the compiler fetches each group at its
  // first use, a dependent round each time)
  asm volatile("" ::"s"(y), "s"(x), "s"(w), "s"(eps), "s"(H), "s"(frag_tt), "s"(lx.src.v), "s"(lx.src.kc), "s"(lx.src.kq), "s"(lx.src.T));
  asm volatile("" ::"s"(lx.src.n_ad), "s"(lx.src.ld), "s"(lx.B), "s"(lx.ids), "s"(lx.scaling), "s"(lx.r), "s"(lx.n_ad), "s"(kp.p), "s"(kp.n), "s"(kp.ld), "s"(kp.stride));
  const int row = blockIdx.x;
  XT* xr = x + (size_t)row * H;
  // The row and the norm weight are requested first: neither depends on the adapter id, so their latency
  // overlaps the id -> (shrink results, B table) chain below.
  float v[VPT][8];
  f16x8 wv[VPT];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = (i * NORM_THREADS + threadIdx.x) * 8;
    if (c < H) {
      wv[i] = ld8(w + c);
      if constexpr (sizeof(XT) == 2) {
        const f16x8 t = ld8((const f16*)xr + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = (float)t[e];
      } else {
        const f32x4 lo = *reinterpret_cast<const f32x4*>((const float*)xr + c);
        const f32x4 hi = *reinterpret_cast<const f32x4*>((const float*)xr + c + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[i][e] = lo[e];
          v[i][4 + e] = hi[e];
        }
      }
    }
  }
  float pv[PARTS ? MAX_PARTS : 1][VPT][8];
  if constexpr (PARTS) {
#pragma unroll
    for (int q = 0; q < MAX_PARTS; ++q)
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int c = (i * NORM_THREADS + threadIdx.x) * 8;
        f32x4 lo = f32x4{0.f, 0.f, 0.f, 0.f}, hi = lo;
        if (q < kp.n && c < H) {
          const float* pr = kp.p + q * kp.stride + (size_t)row * kp.ld + c;
          lo = *reinterpret_cast<const f32x4*>(pr);
          hi = *reinterpret_cast<const f32x4*>(pr + 4);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pv[q][i][e] = lo[e];
          pv[q][i][4 + e] = hi[e];
        }
      }
  }
  bool has_delta = false;
  if constexpr (sizeof(XT) == 4) {
    if (lx.src.v != nullptr) {                      // block-uniform
      const int id = lx.ids[row];
      if (id >= 0 && id < lx.n_ad) {
        has_delta = true;
        const f16* __restrict__ B = lx.B + (size_t)id * H * lx.r;
        const int lpr = lx.r >> 3;                  // lanes (16-byte chunks) per output column
        const int chunks = H * lpr;
        // one batch is 16 chunks per thread: all of B[id] for rank 16 and H = 4096, so that the table is requested once,
        // as a whole, right behind the adapter id
        constexpr int NB = VPT == 1 ? 16 : 8;
        f16x8 bv[NB];
        auto load_batch = [&](int q0) {
#pragma unroll
          for (int u = 0; u < NB; ++u) {
            const int q = q0 + u * NORM_THREADS + threadIdx.x;
            bv[u] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (q < chunks) bv[u] = ld8(B + (size_t)q * 8);
          }
        };
        // the first batch of B and the shrink results go out together, before the barrier that publishes lv
        load_batch(0);
        float lvv = 0.f;
        if (threadIdx.x < lx.r) {
          if (PARTS && lx.src.kc == 0) {            // dense shrink rows were K-split with the matrix: add their partials
            const size_t col = (size_t)id * lx.r + threadIdx.x;
            float a = lx.src.v[(size_t)row * lx.src.ld + col];
            float pq[MAX_PARTS];                    // all requested before the first is added
#pragma unroll
            for (int q = 0; q < MAX_PARTS; ++q) pq[q] = q < kp.n ? kp.p[q * kp.stride + (size_t)row * kp.ld + H + col] : 0.f;
#pragma unroll
            for (int q = 0; q < MAX_PARTS; ++q)
              if (q < kp.n) a += pq[q];
            lvv = a * lx.scaling;
          } else {
            lvv = lora_v_from(lx.src, 0, id, lx.r, row, threadIdx.x, lx.scaling);
          }
        }
        if (threadIdx.x < lx.r) lv[threadIdx.x] = lvv;
        __syncthreads();
        // a thread's chunks all cover the same 8 ranks (the thread count is a multiple of the chunks per column)
        const int sub = threadIdx.x % lpr;
        float lvr[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) lvr[e] = lv[sub * 8 + e];
        for (int q0 = 0; q0 < chunks; q0 += NORM_THREADS * NB) {
          float part[NB];
#pragma unroll
          for (int u = 0; u < NB; ++u) {
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) s = fmaf((float)bv[u][e], lvr[e], s);
            part[u] = s;
          }
          if (q0 + NORM_THREADS * NB < chunks) load_batch(q0 + NORM_THREADS * NB);   // next batch flies during the reduce
#pragma unroll
          for (int u = 0; u < NB; ++u) {
            const int q = q0 + u * NORM_THREADS + threadIdx.x;
            float s = part[u];
            for (int o = 1; o < lpr; o <<= 1) s += __shfl_xor(s, o, WAVE);   // neighbouring groups of 8 first
            if (sub == 0 && q < chunks) delta[q / lpr] = s;
          }
        }
        __syncthreads();
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = (i * NORM_THREADS + threadIdx.x) * 8;
    if (c < H) {
      if constexpr (sizeof(XT) == 4) {
        if (has_delta) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] + delta[c + e];
        }
        if constexpr (PARTS) {
#pragma unroll
          for (int q = 0; q < MAX_PARTS; ++q)
            if (q < kp.n) {
#pragma unroll
              for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] + pv[q][i][e];
            }
        }
        if (has_delta || PARTS) {
          *reinterpret_cast<f32x4*>((float*)xr + c) = f32x4{v[i][0], v[i][1], v[i][2], v[i][3]};
          *reinterpret_cast<f32x4*>((float*)xr + c + 4) = f32x4{v[i][4], v[i][5], v[i][6], v[i][7]};
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(v[i][e], v[i][e], ss);
    }
  }
  ss = block_sum<NORM_THREADS>(ss, lds);
  const float inv = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int c = (i * NORM_THREADS + threadIdx.x) * 8;
    if (c < H) {
      f16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (f16)(v[i][e] * inv * (float)wv[i][e]);
      st8(y + (frag_tt ? frag_offset(row, c, frag_tt) : (size_t)row * H + c), o);
    }
  }
}

__global__ __launch_bounds__(ROW_THREADS) void silu_mul_kernel(f16* __restrict__ out, const f16* __restrict__ gate,
                                                               const f16* __restrict__ up, int ld, int I, int frag_tt) {
  const int row = blockIdx.y;
  const int c = (blockIdx.x * ROW_THREADS + threadIdx.x) * 8;
  if (c >= I) return;
  const f16x8 g = ld8(gate + (size_t)row * ld + c);
  const f16x8 u = ld8(up + (size_t)row * ld + c);
  f16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float gf = (float)g[e];
    o[e] = (f16)(gf / (1.f + expf(-gf)) * (float)u[e]);
  }
  st8(out + (frag_tt ? frag_offset(row, c, frag_tt) : (size_t)row * I + c), o);
}

template <typename OT>
__global__ __launch_bounds__(ROW_THREADS) void embed_kernel(OT* __restrict__ out, const f16* __restrict__ table,
                                                            const int32_t* __restrict__ ids, int H, int V) {
  const int row = blockIdx.x;
  const int id = ids[row];
  const bool ok = id >= 0 && id < V;
  for (int c = threadIdx.x * 8; c < H; c += ROW_THREADS * 8) {
    f16x8 t = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if (ok) t = ld8(table + (size_t)id * H + c);
    if constexpr (sizeof(OT) == 2) {
      st8((f16*)out + (size_t)row * H + c, t);
    } else {
      float* o = (float*)out + (size_t)row * H + c;
      *reinterpret_cast<f32x4*>(o) = f32x4{(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
      *reinterpret_cast<f32x4*>(o + 4) = f32x4{(float)t[4], (float)t[5], (float)t[6], (float)t[7]};
    }
  }
}

// (value, index) maximum with the lowest index winning ties; NaN never wins.
__device__ __forceinline__ void amax_merge(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

constexpr int AMAX_THREADS = 1024;   // one row per workgroup: many threads, few requests each
__global__ __launch_bounds__(AMAX_THREADS) void argmax_kernel(int32_t* __restrict__ ids, const float* __restrict__ logits, int V) {
  __shared__ float lv[AMAX_THREADS / WAVE];
  __shared__ int li[AMAX_THREADS / WAVE];
  const int row = blockIdx.x;
  const float* p = logits + (size_t)row * V;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  // 16-byte loads, eight in flight per thread (a vocabulary of 32000 is one round of requests); elements are merged in
  // increasing index order within a thread and the merge keeps the lower index on ties, so the result is the first
  // maximum whatever the traversal order
  const int V4 = ((size_t)p % 16 == 0) ? V / 4 : 0;
  for (int c0 = threadIdx.x; c0 < V4; c0 += AMAX_THREADS * 8) {
    f32x4 q[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + u * AMAX_THREADS;
      q[u] = c < V4 ? *reinterpret_cast<const f32x4*>(p + 4 * (size_t)c) : f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + u * AMAX_THREADS;
      if (c < V4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) amax_merge(bv, bi, q[u][e], 4 * c + e);
      }
    }
  }
  for (int c = 4 * V4 + threadIdx.x; c < V; c += AMAX_THREADS) amax_merge(bv, bi, p[c], c);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, WAVE);
    const int oi = __shfl_xor(bi, o, WAVE);
    amax_merge(bv, bi, ov, oi);
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) {
    lv[wave] = bv;
    li[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < AMAX_THREADS / WAVE; ++w) amax_merge(bv, bi, lv[w], li[w]);
    ids[row] = bi == 0x7fffffff ? 0 : bi;
  }
}

// RMSNorm of one 16-row token tile straight into fragment order, for token blocks of prefill size: wave r of the 16
// norms row r of the tile (the same sums in the same order as the row kernel above: a lane plays the threads
// lane, lane + 64, ... of that kernel's 512), the rows' 16-byte pieces meet in LDS, and every wave then writes whole
// 1 KiB fragments.  (The row kernel would write each fragment 16 bytes at a time from 16 workgroups.)
constexpr int TILE_PITCH = 128 + 8;    // fp16 elements per (k-step, k-group) slot of the staging buffer: 16 rows x 8, padded

template <typename XT, int MC>
__global__ __launch_bounds__(1024) void rmsnorm_tile_kernel(f16* __restrict__ y, const XT* __restrict__ x, const f16* __restrict__ w,
                                                            float eps, int T, int H, int frag_tt) {
  __shared__ __align__(16) f16 buf[2][64 * TILE_PITCH];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tt = blockIdx.x, row = tt * 16 + wave;
  const bool live = row < T;
  const XT* xr = x + (size_t)(live ? row : 0) * H;
  const int M = (H + 511) / 512;                      // 512-column blocks of a row (<= MC)
  float v[MC][8];
  float ssq[NORM_THREADS / WAVE];
#pragma unroll
  for (int q = 0; q < NORM_THREADS / WAVE; ++q) ssq[q] = 0.f;
#pragma unroll
  for (int m = 0; m < MC; ++m) {
    const int c = m * 512 + lane * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[m][e] = 0.f;
    if (live && c < H) {
      if constexpr (sizeof(XT) == 2) {
        const f16x8 t = ld8((const f16*)xr + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[m][e] = (float)t[e];
      } else {
        const f32x4 lo = *reinterpret_cast<const f32x4*>((const float*)xr + c);
        const f32x4 hi = *reinterpret_cast<const f32x4*>((const float*)xr + c + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[m][e] = lo[e];
          v[m][4 + e] = hi[e];
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ssq[m % (NORM_THREADS / WAVE)] = fmaf(v[m][e], v[m][e], ssq[m % (NORM_THREADS / WAVE)]);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < NORM_THREADS / WAVE; ++q) ss += wave_sum(ssq[q]);
  const float inv = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int m = 0; m < MC; ++m) {
    if (m < M) {                                       // uniform
      const int c = m * 512 + lane * 8;
      f16x8 o = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (c < H) {
        const f16x8 wv = ld8(w + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (f16)(v[m][e] * inv * (float)wv[e]);
      }
      f16* b = buf[m & 1];
      st8(b + lane * TILE_PITCH + wave * 8, o);        // slot = (k-step within the block) * 4 + k-group = lane
      __syncthreads();
      const int ks = m * 16 + wave;                    // this wave's fragment of the block
      if (ks * 32 < H) st8(y + ((size_t)ks * frag_tt + tt) * 512 + lane * 8, ld8(b + (wave * 4 + (lane >> 4)) * TILE_PITCH + (lane & 15) * 8));
    }
  }
}

// SiLU(gate) * up of a token block of prefill size into fragment order: a wave produces one whole fragment (16 tokens x
// 32 columns, 1 KiB contiguous), the four waves of a workgroup four neighbouring k-steps, so that the rows are read in
// runs of 256 bytes.
__global__ __launch_bounds__(ROW_THREADS) void silu_mul_tile_kernel(f16* __restrict__ out, const f16* __restrict__ gate,
                                                                    const f16* __restrict__ up, int ld, int T, int I, int frag_tt) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tt = blockIdx.y, ks = blockIdx.x * (ROW_THREADS / WAVE) + wave;
  const int c = ks * 32 + (lane >> 4) * 8;
  if (c >= I) return;
  const int t = tt * 16 + (lane & 15);
  f16x8 o = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  if (t < T) {
    const f16x8 g = ld8(gate + (size_t)t * ld + c);
    const f16x8 u = ld8(up + (size_t)t * ld + c);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gf = (float)g[e];
      o[e] = (f16)(gf / (1.f + expf(-gf)) * (float)u[e]);
    }
  }
  st8(out + ((size_t)ks * frag_tt + tt) * 512 + lane * 8, o);
}

}  // namespace

static int rmsnorm_impl(const char* who, void* y, int y_layout, void* x, int x_dtype, const void* w, float eps, int T,
                        int H, const LoraExpandRow& lx, void* stream, const KSplitParts& kp = KSplitParts()) {
  MLORA_CHECK(y_layout == MLORA_ROWMAJOR || (y_layout == MLORA_FRAG && H % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "%s: fragment-ordered output needs H %% 32 == 0 (layout=%d H=%d)", who, y_layout, H);
  const int frag_tt = y_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  MLORA_CHECK(y && x && w, MLORA_ERR_INVALID, "%s: null pointer", who);
  MLORA_CHECK(T >= 0 && H > 0 && H % 8 == 0 && H <= 16384, MLORA_ERR_UNSUPPORTED, "%s: need H %% 8 == 0, H <= 16384 (T=%d H=%d)", who, T, H);
  MLORA_CHECK(x_dtype == MLORA_F16 || x_dtype == MLORA_F32, MLORA_ERR_INVALID, "%s: bad x_dtype %d", who, x_dtype);
  if (T == 0) return MLORA_OK;
  hipStream_t s = (hipStream_t)stream;
  if (frag_tt && T > 64 && H <= 4096 && lx.src.v == nullptr && kp.n == 0) {      // a prefill-sized block: whole fragments per store
#define MLORA_RMS_TILE(XT, MC) \
  hipLaunchKernelGGL((rmsnorm_tile_kernel<XT, MC>), dim3(frag_tt), dim3(1024), 0, s, (f16*)y, (const XT*)x, (const f16*)w, eps, T, H, frag_tt)
    if (x_dtype == MLORA_F16) {
      if (H <= 1024) MLORA_RMS_TILE(f16, 2);
      else if (H <= 2048) MLORA_RMS_TILE(f16, 4);
      else MLORA_RMS_TILE(f16, 8);
    } else {
      if (H <= 1024) MLORA_RMS_TILE(float, 2);
      else if (H <= 2048) MLORA_RMS_TILE(float, 4);
      else MLORA_RMS_TILE(float, 8);
    }
#undef MLORA_RMS_TILE
    return mlora_launch_status(who);
  }
  const int vpt = ceil_div(H, NORM_THREADS * 8);
  const size_t dyn = lx.src.v ? (size_t)H * sizeof(float) : 0;   // LDS staging of the expand deltas
#define MLORA_RMS(XT, VPT) \
  hipLaunchKernelGGL((rmsnorm_kernel<XT, VPT>), dim3(T), dim3(NORM_THREADS), dyn, s, (f16*)y, (XT*)x, (const f16*)w, eps, H, frag_tt, lx, kp)
  if (kp.n > 0) {
    MLORA_CHECK(x_dtype == MLORA_F32 && vpt <= 2 && kp.n <= MAX_PARTS && kp.p, MLORA_ERR_UNSUPPORTED,
                "%s: K-split partials need an fp32 row, H <= 8192 and at most %d partial blocks (H=%d n=%d)", who, H, MAX_PARTS, kp.n);
    if (vpt <= 1) hipLaunchKernelGGL((rmsnorm_kernel<float, 1, true>), dim3(T), dim3(NORM_THREADS), dyn, s, (f16*)y, (float*)x, (const f16*)w, eps, H, frag_tt, lx, kp);
    else hipLaunchKernelGGL((rmsnorm_kernel<float, 2, true>), dim3(T), dim3(NORM_THREADS), dyn, s, (f16*)y, (float*)x, (const f16*)w, eps, H, frag_tt, lx, kp);
  } else if (x_dtype == MLORA_F16) {
    if (vpt <= 1) MLORA_RMS(f16, 1);
    else if (vpt <= 2) MLORA_RMS(f16, 2);
    else MLORA_RMS(f16, 4);
  } else {
    if (vpt <= 1) MLORA_RMS(float, 1);
    else if (vpt <= 2) MLORA_RMS(float, 2);
    else MLORA_RMS(float, 4);
  }
#undef MLORA_RMS
  return mlora_launch_status(who);
}

extern "C" int mlora_rmsnorm(void* y, int y_layout, const void* x, int x_dtype, const void* w, float eps, int T, int H,
                             void* stream) {
  return rmsnorm_impl("rmsnorm", y, y_layout, const_cast<void*>(x), x_dtype, w, eps, T, H, LoraExpandRow(), stream);
}

extern "C" int mlora_lora_expand_rmsnorm(void* y, int y_layout, float* resid, const void* v_part, int v_dense, const void* B,
                                         const int32_t* tok_adapter, float scaling, const void* w, float eps, int T, int H,
                                         int K, int r, int n_ad, void* stream) {
  MLORA_CHECK(v_part && B && tok_adapter, MLORA_ERR_INVALID, "lora_expand_rmsnorm: null LoRA argument");
  MLORA_CHECK((r == 8 || r == 16 || r == 32 || r == 64) && n_ad > 0 && K > 0, MLORA_ERR_UNSUPPORTED,
              "lora_expand_rmsnorm: rank %d not in {8,16,32,64} or bad n_ad/K", r);
  LoraExpandRow lx = {};
  lx.src.v = (const float*)v_part;
  lx.src.kc = v_dense ? 0 : lora_k_split(K).kc;
  lx.src.kq = 1;
  lx.src.T = T; lx.src.n_ad = n_ad; lx.src.ld = n_ad * r;
  lx.B = (const f16*)B;
  lx.ids = tok_adapter;
  lx.scaling = scaling;
  lx.r = r; lx.n_ad = n_ad;
  return rmsnorm_impl("lora_expand_rmsnorm", y, y_layout, resid, MLORA_F32, w, eps, T, H, lx, stream);
}

extern "C" int mlora_rmsnorm_ksplit(void* y, int y_layout, float* resid, const float* part, int ks, int ld_part, const void* w,
                                    float eps, int T, int H, const void* v_part, int v_dense, const void* B,
                                    const int32_t* tok_adapter, float scaling, int K, int r, int n_ad, void* stream) {
  MLORA_CHECK(ks >= 1 && ks <= MAX_PARTS + 1 && (ks == 1 || (part && ld_part >= H && ld_part % 4 == 0)), MLORA_ERR_INVALID,
              "rmsnorm_ksplit: ks=%d outside 1..%d, or bad partials (ld_part=%d H=%d)", ks, MAX_PARTS + 1, ld_part, H);
  LoraExpandRow lx = {};
  if (B) {
    MLORA_CHECK(v_part && tok_adapter, MLORA_ERR_INVALID, "rmsnorm_ksplit: null LoRA argument");
    MLORA_CHECK((r == 8 || r == 16 || r == 32 || r == 64) && n_ad > 0 && K > 0, MLORA_ERR_UNSUPPORTED,
                "rmsnorm_ksplit: rank %d not in {8,16,32,64} or bad n_ad/K", r);
    MLORA_CHECK(!v_dense || ks == 1 || ld_part >= H + n_ad * r, MLORA_ERR_INVALID,
                "rmsnorm_ksplit: partials of a dense shrink need ld_part >= H + n_ad * r (ld_part=%d)", ld_part);
    lx.src.v = (const float*)v_part;
    lx.src.kc = v_dense ? 0 : lora_k_split(K).kc;
    lx.src.kq = 1;
    lx.src.T = T; lx.src.n_ad = n_ad; lx.src.ld = n_ad * r;
    lx.B = (const f16*)B;
    lx.ids = tok_adapter;
    lx.scaling = scaling;
    lx.r = r; lx.n_ad = n_ad;
  }
  KSplitParts kp = {};
  if (ks > 1) {
    kp.p = part; kp.n = ks - 1; kp.ld = ld_part; kp.stride = (size_t)T * ld_part;
  }
  return rmsnorm_impl("rmsnorm_ksplit", y, y_layout, resid, MLORA_F32, w, eps, T, H, lx, stream, kp);
}

extern "C" int mlora_silu_mul(void* out, int out_layout, const void* gate, const void* up, int ld, int T, int I,
                              void* stream) {
  MLORA_CHECK(out_layout == MLORA_ROWMAJOR || (out_layout == MLORA_FRAG && I % 32 == 0), MLORA_ERR_UNSUPPORTED,
              "silu_mul: fragment-ordered output needs I %% 32 == 0 (layout=%d I=%d)", out_layout, I);
  const int frag_tt = out_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  MLORA_CHECK(out && gate && up, MLORA_ERR_INVALID, "silu_mul: null pointer");
  MLORA_CHECK(T >= 0 && I > 0 && I % 8 == 0 && ld >= I && ld % 8 == 0, MLORA_ERR_UNSUPPORTED, "silu_mul: need I %% 8 == 0, ld >= I, ld %% 8 == 0 (T=%d I=%d ld=%d)", T, I, ld);
  MLORA_CHECK(T <= 65535, MLORA_ERR_UNSUPPORTED, "silu_mul: T=%d exceeds 65535", T);
  if (T == 0) return MLORA_OK;
  if (frag_tt && T > 64) {
    hipLaunchKernelGGL(silu_mul_tile_kernel, dim3(ceil_div(I, 32 * (ROW_THREADS / WAVE)), frag_tt), dim3(ROW_THREADS), 0,
                       (hipStream_t)stream, (f16*)out, (const f16*)gate, (const f16*)up, ld, T, I, frag_tt);
    return mlora_launch_status("silu_mul");
  }
  hipLaunchKernelGGL(silu_mul_kernel, dim3(ceil_div(I, ROW_THREADS * 8), T), dim3(ROW_THREADS), 0, (hipStream_t)stream,
                     (f16*)out, (const f16*)gate, (const f16*)up, ld, I, frag_tt);
  return mlora_launch_status("silu_mul");
}

extern "C" int mlora_embed(void* out, int out_dtype, const void* table, const int32_t* ids, int T, int H, int V, void* stream) {
  MLORA_CHECK(out && table && ids, MLORA_ERR_INVALID, "embed: null pointer");
  MLORA_CHECK(T >= 0 && H > 0 && H % 8 == 0 && V > 0, MLORA_ERR_UNSUPPORTED, "embed: need H %% 8 == 0 (T=%d H=%d V=%d)", T, H, V);
  MLORA_CHECK(out_dtype == MLORA_F16 || out_dtype == MLORA_F32, MLORA_ERR_INVALID, "embed: bad out_dtype %d", out_dtype);
  if (T == 0) return MLORA_OK;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == MLORA_F16) hipLaunchKernelGGL(embed_kernel<f16>, dim3(T), dim3(ROW_THREADS), 0, s, (f16*)out, (const f16*)table, ids, H, V);
  else hipLaunchKernelGGL(embed_kernel<float>, dim3(T), dim3(ROW_THREADS), 0, s, (float*)out, (const f16*)table, ids, H, V);
  return mlora_launch_status("embed");
}

extern "C" int mlora_argmax(int32_t* ids, const float* logits, int B, int V, void* stream) {
  MLORA_CHECK(ids && logits, MLORA_ERR_INVALID, "argmax: null pointer");
  MLORA_CHECK(B >= 0 && V > 0, MLORA_ERR_INVALID, "argmax: bad shape B=%d V=%d", B, V);
  if (B == 0) return MLORA_OK;
  hipLaunchKernelGGL(argmax_kernel, dim3(B), dim3(AMAX_THREADS), 0, (hipStream_t)stream, ids, logits, V);
  return mlora_launch_status("argmax");
}
