// Paged-KV attention for gfx950: RoPE + cache append, decode attention, prefill attention.
//
// Cache layout per layer (16-token pages):
//   k_cache [n_pages, Hkv, D/32, 4, 16, 8]  rotated keys in matrix-core fragment order: element (token, d) of a
//                                   page sits at ((d/32 * 4 + (d%32)/8) * 16 + token) * 8 + d%8, so the
//                                   16-token x 32-dim operand of one MFMA is a contiguous 1 KiB block
//   v_cache [n_pages, Hkv, D, 16]  values         - token-minor, so a lane's 16-byte load holds 8
//                                                   consecutive tokens of one dim
// Both attention kernels read K and V straight into MFMA operands: no LDS transpose, no shuffles.
// The page-table walk is integer-only: page = block_table[seq, pos / 16], slot = pos % 16.
#include "lora_device.h"

namespace {

constexpr int PAGE = MLORA_PAGE_SIZE;

// element (token, d) inside one head's K page
__device__ __forceinline__ int k_page_offset(int token, int d) {
  return (((d >> 5) * 4 + ((d >> 3) & 3)) * PAGE + token) * 8 + (d & 7);
}

// LoRA expand of the q, k, v projections carried by the RoPE / append kernel: delta rows are added to the
// projection output (and rounded to fp16, as the stand-alone expand does) before rotation and storage.
struct LoraExpandQKV {
  LoraVSource src;           // shrink results of the q, k, v slots (src.v == nullptr: no LoRA in this launch)
  const f16* B[3];           // [n_ad, N_p, r] per projection, nullptr = projection not adapted
  const int32_t* ids;
  float scaling;
  int r, n_ad;
};

// The o projection's LoRA shrink taken off the attention output where it is produced: the workgroup of (sequence t,
// kv head) adds nothing to the output itself but writes, for each of its query heads h, the head's share of
// v = A[id_t] . attn[t, :]  -  vpart[h][t][j] = sum over the head's D dims of f16(attn[t, h, d]) * A[id_t][j][h D + d]
// (fp32) - so that the consumer adds Hq head shares per (token, rank entry) in head order and needs no pass over K.
struct OShrinkHeads {
  const f16* A;           // [n_ad, r, Hq * D]; nullptr: no shrink in this launch
  float* vpart;           // [Hq, T, r]
  const int32_t* ids;     // [T]
  int r, n_ad, T;
};

// thread (query head qh, rank entry j, 8-dim piece c) of the workgroup of kv head kh: its 16 bytes of A[id] ...
template <int D>
__device__ __forceinline__ f16x8 oshrink_piece(const OShrinkHeads& os, int id, int G, int kh, int Hq) {
  constexpr int OPC = D / 8;
  const int oc = threadIdx.x % OPC, oj = (threadIdx.x / OPC) % os.r, oq = threadIdx.x / (OPC * os.r);
  return ld8(os.A + ((size_t)id * os.r + oj) * ((size_t)Hq * D) + (size_t)(kh * G + oq) * D + oc * 8);
}

// ... and its product with the head's output as stored (outs: the workgroup's G x D fp16 outputs in LDS, published by a
// barrier), summed over the D / 8 pieces of the row, which sit in neighbouring lanes
template <int D>
__device__ __forceinline__ void oshrink_head_shares(const OShrinkHeads& os, f16x8 a8, const f16* __restrict__ outs, int G, int kh, int b) {
  constexpr int OPC = D / 8;
  const int oc = threadIdx.x % OPC, oj = (threadIdx.x / OPC) % os.r, oq = threadIdx.x / (OPC * os.r);
  float sum = dot8(a8, *reinterpret_cast<const f16x8*>(&outs[oq * D + oc * 8]), 0.f);
#pragma unroll
  for (int o = 1; o < OPC; o <<= 1) sum += __shfl_xor(sum, o, WAVE);
  if (oc == 0) os.vpart[((size_t)(kh * G + oq) * os.T + b) * os.r + oj] = sum;
}

// grid (T, Hq + 2 Hkv), 64 threads: thread i rotates the pair (i, i + D/2) of one head of one token
__global__ __launch_bounds__(64) void rope_kv_append_kernel(f16* __restrict__ qkv, f16* __restrict__ k_cache,
                                                            f16* __restrict__ v_cache,
                                                            const int32_t* __restrict__ block_table, int max_blocks,
                                                            const int32_t* __restrict__ tok_seq,
                                                            const int32_t* __restrict__ tok_pos,
                                                            const float* __restrict__ rope_cos,
                                                            const float* __restrict__ rope_sin, int max_pos, int Hq,
                                                            int Hkv, int D, int n_pages, int n_seq, int T,
                                                            LoraExpandQKV lx) {
#pragma clang fp contract(off)
  __shared__ float lv[64];
  const int t = blockIdx.x, hh = blockIdx.y, i = threadIdx.x;
  const int half = D >> 1;
  const int proj = hh < Hq ? 0 : (hh < Hq + Hkv ? 1 : 2);
  const int head = hh - (proj == 0 ? 0 : (proj == 1 ? Hq : Hq + Hkv));
  // Two dependent rounds of loads instead of five: the indices first, then everything they address.
  const bool lora = lx.src.v != nullptr && lx.B[proj] != nullptr;          // block-uniform
  const int seq = tok_seq[t], pos = tok_pos[t];
  const int id = lora ? lx.ids[t] : -1;
  const bool adapted = lora && id >= 0 && id < lx.n_ad;
  const bool valid = !(seq < 0 || seq >= n_seq || pos < 0 || pos >= max_pos || pos / PAGE >= max_blocks);
  const bool active = valid && i < half;
  f16* src = qkv + ((size_t)t * (Hq + 2 * Hkv) + hh) * D;
  f16 h1 = (f16)0.f, h2 = (f16)0.f;
  float c = 0.f, s = 0.f;
  int page = -1;
  f16x8 b1[8], b2[8];
  float lvv = 0.f;
  if (adapted && i < lx.r) lvv = lora_v_from(lx.src, proj, id, lx.r, t, i, lx.scaling);
  if (active) {
    h1 = src[i];
    h2 = src[i + half];
    if (hh >= Hq) page = block_table[(size_t)seq * max_blocks + pos / PAGE];
    if (hh < Hq + Hkv) {
      c = rope_cos[(size_t)pos * half + i];
      s = rope_sin[(size_t)pos * half + i];
    }
    if (adapted) {
      const int n_rows = (proj == 0 ? Hq : Hkv) * D;
      const f16* brow = lx.B[proj] + ((size_t)id * n_rows + (size_t)head * D) * lx.r;
      lora_row_load(brow + (size_t)i * lx.r, lx.r, b1);
      lora_row_load(brow + (size_t)(i + half) * lx.r, lx.r, b2);
    }
  }
  if (adapted) {
    if (i < lx.r) lv[i] = lvv;
    __syncthreads();
  }
  if (!active) return;
  if (adapted) {
    {
#pragma clang fp contract(fast)
      h1 = (f16)((float)h1 + lora_row_dot_regs(b1, lv, lx.r));
      h2 = (f16)((float)h2 + lora_row_dot_regs(b2, lv, lx.r));
    }
  }
  if (hh >= Hq + Hkv) {
    if (page < 0 || page >= n_pages) return;
    f16* dst = v_cache + ((size_t)page * Hkv + (hh - Hq - Hkv)) * D * PAGE + pos % PAGE;
    dst[(size_t)i * PAGE] = h1;
    dst[(size_t)(i + half) * PAGE] = h2;
    return;
  }
  const float x1 = (float)h1, x2 = (float)h2;
  // Separately rounded products (fp contraction is off in this kernel) and an fp32 result that is
  // materialised before the fp16 conversion (the empty asm keeps the compiler from fusing the add
  // and the convert into one single-rounding instruction): the rotation is then the same IEEE fp32
  // arithmetic as a plain CPU evaluation, and the stored fp16 keys are reproducible bit for bit.
  float r1 = x1 * c - x2 * s;
  float r2 = x2 * c + x1 * s;
  asm volatile("" : "+v"(r1), "+v"(r2));
  const f16 o1 = (f16)r1, o2 = (f16)r2;
  if (hh < Hq) {
    src[i] = o1;
    src[i + half] = o2;
  } else {
    if (page < 0 || page >= n_pages) return;
    f16* dst = k_cache + ((size_t)page * Hkv + (hh - Hq)) * PAGE * D;
    dst[k_page_offset(pos % PAGE, i)] = o1;
    dst[k_page_offset(pos % PAGE, i + half)] = o2;
  }
}

// Variant for more than 64 tokens that moves 16 bytes at a time: one WAVE per (16 consecutive tokens, head of q / k / v),
// four heads per workgroup, no barriers.  Lane l owns the sequence, position and cache page of token l % 16 of the tile and
// hands them to the lanes that work on that token; the lanes of a load cover whole half rows of a head (128 contiguous
// bytes at D = 128), so every cache line is consumed by the instruction that fetches it.  q heads are rotated in place in
// chunks of 8 pairs.  A rotated K chunk is one 16-byte piece of its token's page (fragment order), wherever the token
// lies.  V of a tile that is slots 0..15 of one page (prompts that start on a page boundary) is transposed through LDS
// into the page's contiguous [D][16] block; V of other tiles (a decode step: every token its own sequence) goes out
// element by element.  Measured at 4096 prompt tokens, D = 128: 32 + 2 x 32 heads 37 us (5.4 TB/s), 32 + 2 x 8 heads 22 us; the
// earlier mapping (a lane kept one token, 64-byte pieces per token and load, V gathered 2 bytes at a time) took 53 / 31 us.
// Same arithmetic per element as rope_kv_append_kernel.  rope_cos / rope_sin must be 16-byte aligned.
template <int D>
__global__ __launch_bounds__(256) void rope_kv_append_tile_kernel(f16* __restrict__ qkv, f16* __restrict__ k_cache,
                                                                  f16* __restrict__ v_cache,
                                                                  const int32_t* __restrict__ block_table, int max_blocks,
                                                                  const int32_t* __restrict__ tok_seq,
                                                                  const int32_t* __restrict__ tok_pos,
                                                                  const float* __restrict__ rope_cos,
                                                                  const float* __restrict__ rope_sin, int max_pos, int Hq,
                                                                  int Hkv, int n_pages, int n_seq, int T) {
  constexpr int half = D / 2;
  constexpr int NCH = half / 8;                               // 8-pair chunks of a head row
  constexpr int VT_LD = 20;
  __shared__ __align__(16) f16 vts[4][D][VT_LD];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int HH = Hq + 2 * Hkv;
  const int t0 = blockIdx.x * 16;
  const int hh = blockIdx.y * 4 + wave;                       // a head of the fused row: q heads, then k heads, then v heads
  if (hh >= HH) return;
  const int tk = lane & 15, t = t0 + tk;
  int seq = -1, pos = -1;
  if (t < T) {
    seq = tok_seq[t];
    pos = tok_pos[t];
    if (seq < 0 || seq >= n_seq || pos < 0 || pos >= max_pos || pos / PAGE >= max_blocks) seq = -1;
  }
  // rotation of one element d of a head row (x1 = first-half element, x2 = its partner in the second half)
  auto rot = [&](float x1, float x2, float c, float s, bool second) -> f16 {
    float r;
    {
#pragma clang fp contract(off)
      r = second ? x2 * c + x1 * s : x1 * c - x2 * s;
    }
    asm volatile("" : "+v"(r));
    return (f16)r;
  };
  // chunk ch of a token at position p: pairs 8 ch .. 8 ch + 7 of a head row at src, rotated
  auto rot_chunk = [&](const f16* src, int p, int ch, f16x8& o_lo, f16x8& o_hi) {
    const int p0 = ch * 8;
    const f16x8 lo = ld8(src + p0), hi = ld8(src + p0 + half);
    const float* cp = rope_cos + (size_t)p * half + p0;
    const float* sp = rope_sin + (size_t)p * half + p0;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(cp), c1 = *reinterpret_cast<const f32x4*>(cp + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(sp), s1 = *reinterpret_cast<const f32x4*>(sp + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float c = e < 4 ? c0[e & 3] : c1[e & 3], sn = e < 4 ? s0[e & 3] : s1[e & 3];
      o_lo[e] = rot((float)lo[e], (float)hi[e], c, sn, false);
      o_hi[e] = rot((float)lo[e], (float)hi[e], c, sn, true);
    }
  };
  // Work items of a wave: NCH consecutive lanes take the chunks of one token's half row (whole 128-byte lines per
  // load), TPI tokens per pass; the token's sequence and position come from the lane that owns it.
  constexpr int TPI = WAVE / NCH, NPASS = 16 / TPI;
  const int ch = lane % NCH;
  int tkj[NPASS], seqj[NPASS], posj[NPASS];
#pragma unroll
  for (int j = 0; j < NPASS; ++j) {
    tkj[j] = lane / NCH + TPI * j;
    seqj[j] = __shfl(seq, tkj[j], WAVE);
    posj[j] = __shfl(pos, tkj[j], WAVE);
  }
  if (hh < Hq) {                                              // q: rotate in place
#pragma unroll
    for (int j = 0; j < NPASS; ++j) {
      if (seqj[j] < 0) continue;
      f16* src = qkv + ((size_t)(t0 + tkj[j]) * HH + hh) * D;
      f16x8 o_lo, o_hi;
      rot_chunk(src, posj[j], ch, o_lo, o_hi);
      st8(src + ch * 8, o_lo);
      st8(src + ch * 8 + half, o_hi);
    }
    return;
  }
  const bool is_v = hh >= Hq + Hkv;                           // wave-uniform
  const int kh = is_v ? hh - Hq - Hkv : hh - Hq;
  // the cache page of the lane's own token (-1: nothing to store), then of the tokens the lane works on
  int page_own = -1;
  if (seq >= 0) {
    page_own = block_table[(size_t)seq * max_blocks + pos / PAGE];
    if (page_own >= n_pages) page_own = -1;
  }
  int pagej[NPASS];
#pragma unroll
  for (int j = 0; j < NPASS; ++j) pagej[j] = __shfl(page_own, tkj[j], WAVE);
  if (!is_v) {
    // K: a token's chunk of 8 elements is one 16-byte piece of its page's fragment rows (the pieces of a page's 16
    // tokens lie side by side: a tile that is one whole page writes whole lines)
#pragma unroll
    for (int j = 0; j < NPASS; ++j) {
      if (pagej[j] < 0) continue;
      const f16* ksrc = qkv + ((size_t)(t0 + tkj[j]) * HH + Hq + kh) * D;
      f16* kd = k_cache + ((size_t)pagej[j] * Hkv + kh) * PAGE * D;
      const int slot = posj[j] % PAGE;
      f16x8 o_lo, o_hi;
      rot_chunk(ksrc, posj[j], ch, o_lo, o_hi);
      st8(kd + ((size_t)ch * 16 + slot) * 8, o_lo);
      st8(kd + ((size_t)(ch + NCH) * 16 + slot) * 8, o_hi);
    }
    return;
  }
  const int seq0 = __shfl(seq, 0, WAVE), pos0 = __shfl(pos, 0, WAVE);
  const bool al = __ballot(page_own >= 0 && seq == seq0 && pos == pos0 + tk) == ~0ull && (pos0 % PAGE) == 0;   // wave-uniform
  if (al) {
    // V of a tile that is one whole page: the 16 x D tile is transposed through the wave's own LDS rows (row stride 20
    // elements: the 2-byte writes of a pass spread over the banks, the 8-byte reads stay aligned), then leaves as the
    // page's contiguous 32 D bytes.
    const int page = __shfl(page_own, 0, WAVE);
    f16(*vt)[VT_LD] = vts[wave];
#pragma unroll
    for (int j = 0; j < NPASS; ++j) {
      const f16* vsrc = qkv + ((size_t)(t0 + tkj[j]) * HH + Hq + Hkv + kh) * D;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const f16x8 x = ld8(vsrc + hf * half + ch * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) vt[hf * half + ch * 8 + e][tkj[j]] = x[e];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f16* vd = v_cache + ((size_t)page * Hkv + kh) * D * PAGE;
#pragma unroll
    for (int it = lane; it < D * 2; it += WAVE) {
      const int d = it >> 1, tg = it & 1;
      const f16x4 a = *reinterpret_cast<const f16x4*>(&vt[d][tg * 8]), b = *reinterpret_cast<const f16x4*>(&vt[d][tg * 8 + 4]);
      f16x8 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) { o[e] = a[e]; o[4 + e] = b[e]; }
      st8(vd + (size_t)it * 8, o);
    }
    return;
  }
  // V of tokens of several pages or sequences (a decode step: every token its own sequence): element-wise into each
  // token's slot of its page, all loads of the wave issued before the first store
  f16x8 xv[NPASS][2];
#pragma unroll
  for (int j = 0; j < NPASS; ++j) {
    const int tl = t0 + tkj[j] < T ? t0 + tkj[j] : T - 1;
    const f16* vsrc = qkv + ((size_t)tl * HH + Hq + Hkv + kh) * D;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) xv[j][hf] = ld8(vsrc + hf * half + ch * 8);
  }
#pragma unroll
  for (int j = 0; j < NPASS; ++j) {
    if (pagej[j] < 0) continue;
    f16* vd = v_cache + ((size_t)pagej[j] * Hkv + kh) * D * PAGE + posj[j] % PAGE;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int e = 0; e < 8; ++e) vd[(size_t)(hf * half + ch * 8 + e) * PAGE] = xv[j][hf][e];
  }
}

// ---------------------------------------------------------------------------------------------
// Decode: one workgroup (4 waves) per (sequence, kv head); the G = Hq / Hkv <= 16 query heads that share the
// kv head are the 16 columns of the matrix-core tiles, so K and V are read once per group.  A wave takes
// pages w, w+4, ...  Per page:
//   S^T = K . Q^T      4 (D=128) v_mfma_f32_16x16x32_f16, K fragments are contiguous 1 KiB loads;
//                      accumulator rows are the page's tokens (lane group g holds tokens 4g..4g+3), columns
//                      the query heads - a lane keeps the online-softmax state (m, l) of its own column
//   O^T += V^T . P^T   one MFMA per 16 dims; the lane's four probabilities are already the B operand it
//                      must supply (hi + lo fp16 halves in k-slots 0-3 / 4-7, V repeated in both, so P
//                      enters with ~22 mantissa bits), and the rescale factor alpha is the lane's own.
// The four waves' (m, l, O) states are merged through LDS.
// ---------------------------------------------------------------------------------------------
constexpr int ATT_WAVES = 4;

// Waves per workgroup of the decode kernels.  A CU holds 16 waves either way (one page each in flight); few, large
// workgroups spread the per-workgroup work (new token, merge of the waves' states) over more waves and keep a CU busy
// when sequences x kv heads are few (small batches, grouped-query models); many small ones balance better when the
// launch runs in several rounds (measured: eight waves up to 2048 workgroups' worth, four beyond).  Limited by the LDS
// merge buffer [NW][G][D].
int attn_waves(int B, int Hkv, int G, int D) {
  const long wgs = (long)B * Hkv;
  int nw = wgs > 2048 ? ATT_WAVES : wgs > 256 ? 8 : 16;
  while (nw > ATT_WAVES && (size_t)nw * G * D * sizeof(float) > 48 * 1024) nw >>= 1;
  return nw;
}

template <int D, int NW>   // NW waves per workgroup share the pages of one (sequence, kv head)
__global__ __launch_bounds__(NW * WAVE, 4) void paged_attn_decode_kernel(
    f16* __restrict__ out, const f16* __restrict__ qkv, const f16* __restrict__ k_cache, const f16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ seq_ids,
    const int32_t* __restrict__ ctx_len, int Hq, int Hkv, int n_pages, int n_seq, float scale, int frag_tt, OShrinkHeads os) {
  constexpr int NKB = D / 32;   // k-blocks of the QK^T product
  constexpr int NDB = D / 16;   // dim blocks of the output
  __shared__ float sm[NW][16], sl[NW][16];
  __shared__ __align__(16) f16 outs[16 * D];   // the workgroup's outputs as stored, for the o shrink
  extern __shared__ float sacc[];   // [NW][G][D]

  // arguments, then the sequence's scalars, then its first page ids: three grouped rounds of scalar loads (see
  // rope_attn_decode_kernel)
  asm volatile("" ::"s"(out), "s"(qkv), "s"(k_cache), "s"(v_cache), "s"(block_table), "s"(max_blocks), "s"(seq_ids), "s"(ctx_len));
  asm volatile("" ::"s"(Hq), "s"(Hkv), "s"(n_pages), "s"(n_seq), "s"(scale), "s"(frag_tt));
  asm volatile("" ::"s"(os.A), "s"(os.vpart), "s"(os.ids), "s"(os.r), "s"(os.n_ad), "s"(os.T));
  const int b = blockIdx.y, kh = blockIdx.x;
  const int G = Hq / Hkv;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const int seq = seq_ids[b];
  int ctx = ctx_len[b];
  const int oid_raw = (os.A != nullptr ? os.ids : seq_ids)[b];
  asm volatile("" ::"s"(seq), "s"(ctx), "s"(oid_raw));
  // the o shrink (see OShrinkHeads): the thread's 16 bytes of A[id] are requested now and wait in registers for the epilogue
  const bool o_on = os.A != nullptr && oid_raw >= 0 && oid_raw < os.n_ad;        // uniform
  const bool o_mine = o_on && (int)threadIdx.x < G * os.r * (D / 8);
  f16x8 oa = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  if (o_mine) oa = oshrink_piece<D>(os, oid_raw, G, kh, Hq);
  if (seq < 0 || seq >= n_seq) ctx = 0;
  if (ctx > max_blocks * PAGE) ctx = max_blocks * PAGE;
  const int npages = (ctx + PAGE - 1) / PAGE;
  const int32_t* __restrict__ bt = block_table + (size_t)(seq < 0 || seq >= n_seq ? 0 : seq) * max_blocks;

  // Q^T as the B operand: lane holds q[head kh*G + col][kb*32 + g*8 .. +8], zero for unused columns
  f16x8 qf[NKB];
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb) qf[kb] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  if (col < G) {
    const f16* qp = qkv + ((size_t)b * (Hq + 2 * Hkv) + kh * G + col) * D + g * 8;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) qf[kb] = ld8(qp + kb * 32);
  }

  float m = -INFINITY, l = 0.f;
  f32x4 O[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) O[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int e_first = bt[wave < max_blocks ? wave : 0];
  int page = wave < npages ? e_first : -1;
  for (int pg = wave; pg < npages; pg += NW) {
    const int next = pg + NW < npages ? bt[pg + NW] : -1;   // the next page id is requested one page ahead
    if (page >= 0 && page < n_pages) {                      // wave-uniform
      const f16* kp = k_cache + ((size_t)page * Hkv + kh) * PAGE * D + lane * 8;
      const f16* vp = v_cache + (((size_t)page * Hkv + kh) * D + col) * PAGE + g * 4;   // dim col (+16 db), tokens 4g..
      f16x8 kf[NKB];
      f16x4 vf[NDB];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) kf[kb] = ld8(kp + kb * 512);
#pragma unroll
      for (int db = 0; db < NDB; ++db) vf[db] = *reinterpret_cast<const f16x4*>(vp + db * 16 * PAGE);

      f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f};   // st[r] = S[token 4g + r][head col]
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) st = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[kb], qf[kb], st, 0, 0, 0);

      float pm = -INFINITY;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        st[r] = (pg * PAGE + 4 * g + r >= ctx) ? -INFINITY : st[r] * scale;
        pm = fmaxf(pm, st[r]);
      }
      pm = fmaxf(pm, __shfl_xor(pm, 16, WAVE));
      pm = fmaxf(pm, __shfl_xor(pm, 32, WAVE));
      const float m_new = fmaxf(m, pm);       // finite: the first token of a visited page is < ctx
      const float alpha = __expf(m - m_new);
      f16x8 pa;
      float ps = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __expf(st[r] - m_new);
        ps += p;
        const f16 hi = (f16)p;
        pa[r] = hi;
        pa[4 + r] = (f16)(p - (float)hi);
      }
      l = l * alpha + ps;                     // per-lane share of the column's sum; lanes are combined at the end
      m = m_new;
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        O[db] *= alpha;
        const f16x8 vv = f16x8{vf[db][0], vf[db][1], vf[db][2], vf[db][3], vf[db][0], vf[db][1], vf[db][2], vf[db][3]};
        O[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vv, pa, O[db], 0, 0, 0);   // O^T[dim 16db+4g+r][head col]
      }
    }
    page = next;
  }
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (col < G) {
#pragma unroll
    for (int db = 0; db < NDB; ++db)
      *reinterpret_cast<f32x4*>(&sacc[((size_t)wave * G + col) * D + db * 16 + 4 * g]) = O[db];
    if (g == 0) {
      sm[wave][col] = m;
      sl[wave][col] = l;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < G * D; e += NW * WAVE) {
    const int qh = e / D, d = e % D;
    float M = sm[0][qh];
#pragma unroll
    for (int w = 1; w < NW; ++w) M = fmaxf(M, sm[w][qh]);
    float L = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = sm[w][qh] == -INFINITY ? 0.f : __expf(sm[w][qh] - M);
      L += sl[w][qh] * f;
      o += sacc[((size_t)w * G + qh) * D + d] * f;
    }
    const int h = kh * G + qh;
    const size_t oo = frag_tt ? frag_offset(b, h * D + d, frag_tt) : ((size_t)b * Hq + h) * D + d;
    const f16 of = (f16)(L > 0.f ? o / L : 0.f);
    out[oo] = of;
    if (o_on) outs[qh * D + d] = of;
  }
  if (o_on) {                                                // uniform
    __syncthreads();
    if (o_mine) oshrink_head_shares<D>(os, oa, outs, G, kh, b);
  }
}

// ---------------------------------------------------------------------------------------------
// Decode step in one launch: RoPE + cache append (+ LoRA expand of q, k, v) + attention.  Same workgroup shape
// and page loop as paged_attn_decode_kernel.  The workgroup first finishes the new token of its sequence for its
// own heads - projection output + LoRA delta, rotation of q and k exactly as rope_kv_append_kernel does it - keeps
// the rotated q, the new k and the new v in LDS and stores k, v to their page slot.  In the page loop the wave that
// meets the page of the new token overwrites that token's lanes of the K / V fragments from LDS, so it never
// depends on reading back what the workgroup has just stored.  Results are those of the two separate kernels,
// bit for bit; the q rows of qkv are left unrotated.
// ---------------------------------------------------------------------------------------------
template <int D, int RG, int NW>   // RG: 8-wide rank groups the B-row registers hold (rank <= 8 RG); NW: waves per workgroup
__global__ __launch_bounds__(NW * WAVE, 4) void rope_attn_decode_kernel(
    f16* __restrict__ out, const f16* __restrict__ qkv, f16* __restrict__ k_cache, f16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ seq_ids,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ ctx_len, const float* __restrict__ rope_cos,
    const float* __restrict__ rope_sin, int max_pos, int Hq, int Hkv, int n_pages, int n_seq, float scale, int frag_tt,
    LoraExpandQKV lx, OShrinkHeads os) {
  constexpr int NKB = D / 32;
  constexpr int NDB = D / 16;
  constexpr int half = D / 2;
  __shared__ float sm[NW][16], sl[NW][16];
  __shared__ float lv[3][64];
  __shared__ f16x8 oslice[NW * WAVE];            // a thread's piece of A_o[id] waits here from the prologue to the epilogue
  __shared__ float lvq[LORA_MAX_KQ][3][64];     // K-range blocks of dense shrink results before they are added
  __shared__ __align__(16) f16 qs[16 * D];       // rotated q of the group's heads
  __shared__ __align__(16) f16 knew[D], vnew[D];   // the new token's rotated key and its value
  extern __shared__ float sacc[];                  // [NW][G][D]

  // Three dependent rounds of scalar loads stand before the first page request - the arguments, then what they point at
  // for this sequence, then its page ids - and every workgroup of the launch waits them out at the same time.  All
  // arguments are therefore fetched at once (the empty asm statements make the compiler materialise them here instead
  // of at their first use, each group behind a wait of its own), and the loads of a round are unconditional, with
  // clamped indices, so that they go out together.
  asm volatile("" ::"s"(out), "s"(qkv), "s"(k_cache), "s"(v_cache), "s"(block_table), "s"(max_blocks), "s"(seq_ids), "s"(tok_pos));
  asm volatile("" ::"s"(ctx_len), "s"(rope_cos), "s"(rope_sin), "s"(max_pos), "s"(Hq), "s"(Hkv), "s"(n_pages), "s"(n_seq));
  asm volatile("" ::"s"(scale), "s"(frag_tt), "s"(lx.src.v), "s"(lx.src.kc), "s"(lx.src.kq), "s"(lx.src.T), "s"(lx.ids), "s"(lx.scaling));
  asm volatile("" ::"s"(lx.B[0]), "s"(lx.B[1]), "s"(lx.B[2]), "s"(lx.r), "s"(lx.n_ad), "s"(lx.src.n_ad), "s"(lx.src.ld));
  asm volatile("" ::"s"(os.A), "s"(os.vpart), "s"(os.ids), "s"(os.r), "s"(os.n_ad), "s"(os.T));
  const int b = blockIdx.y, kh = blockIdx.x;
  const int G = Hq / Hkv;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const bool lora = lx.src.v != nullptr;
  const int seq = seq_ids[b];
  const int pos = tok_pos[b];
  int ctx = ctx_len[b];
  const int id_raw = (lora ? lx.ids : seq_ids)[b];
  const int oid_raw = (os.A != nullptr ? os.ids : seq_ids)[b];
  asm volatile("" ::"s"(seq), "s"(pos), "s"(ctx), "s"(id_raw), "s"(oid_raw));
  const int id = lora ? id_raw : -1;
  const bool o_on = os.A != nullptr && oid_raw >= 0 && oid_raw < os.n_ad;        // uniform
  const bool seq_ok = seq >= 0 && seq < n_seq;
  if (!seq_ok) ctx = 0;
  if (ctx > max_blocks * PAGE) ctx = max_blocks * PAGE;
  const int npages = (ctx + PAGE - 1) / PAGE;
  const int32_t* __restrict__ bt = block_table + (size_t)(seq_ok ? seq : 0) * max_blocks;
  const bool pos_ok = seq_ok && pos >= 0 && pos < max_pos && pos / PAGE < max_blocks;   // the append condition of rope_kv_append
  const int new_pg = pos_ok ? pos / PAGE : -1, new_slot = pos & (PAGE - 1);
  const bool adapted = lora && id >= 0 && id < lx.n_ad;

  // The wave's first TWO pages are requested before anything else: together with the other waves' that is enough traffic
  // to keep the memory system busy for the whole time the new token takes (the second buffer lives in registers the
  // accumulators only need later, and is gone after the second page).
  constexpr bool PF2 = RG <= 2;      // the wide-rank variant has no registers to spare for the second buffer
  const int e_new = bt[pos_ok ? new_pg : 0];
  const int e_first = bt[wave < max_blocks ? wave : 0];
  const int e_second = bt[wave + NW < max_blocks ? wave + NW : 0];
  asm volatile("" ::"s"(e_new), "s"(e_first), "s"(e_second));
  const int new_page = pos_ok ? e_new : -1;
  int page = wave < npages ? e_first : -1;
  const int page2 = PF2 && wave + NW < npages ? e_second : -1;
  f16x8 kf[NKB], kf2[PF2 ? NKB : 1];
  f16x4 vf[NDB], vf2[PF2 ? NDB : 1];
  auto load_into = [&](f16x8 (&k)[NKB], f16x4 (&v)[NDB], int pgid) {
    const f16* kp = k_cache + ((size_t)pgid * Hkv + kh) * PAGE * D + lane * 8;
    const f16* vp = v_cache + (((size_t)pgid * Hkv + kh) * D + col) * PAGE + g * 4;   // dim col (+16 db), tokens 4g..
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) k[kb] = ld8(kp + kb * 512);
#pragma unroll
    for (int db = 0; db < NDB; ++db) v[db] = *reinterpret_cast<const f16x4*>(vp + db * 16 * PAGE);
  };
  auto load_page = [&](int pgid) { load_into(kf, vf, pgid); };
  if (page >= 0 && page < n_pages) load_page(page);
  if constexpr (PF2) {
    if (page2 >= 0 && page2 < n_pages) load_into(kf2, vf2, page2);
  }

  // ---- the new token: heads kh*G .. kh*G+G-1 of q, head kh of k and of v; one (head, pair) item per thread and pass.
  // An item's loads (projection output, rows of B, rotation factors) do not depend on the shrink results, so the
  // first pass issues them before the barrier that publishes lv.
  const int items = (G + 2) * half;
  f16 h1, h2;
  f16x8 b1[RG], b2[RG];
  float rc, rs;
  int hl, pi, proj;
  bool with_delta;
  auto issue = [&](int it) {
    hl = it / half;                                              // local head: 0..G-1 q, G k, G+1 v
    pi = it % half;
    proj = hl < G ? 0 : (hl == G ? 1 : 2);
    const int hh = proj == 0 ? kh * G + hl : (proj == 1 ? Hq + kh : Hq + Hkv + kh);   // head index inside qkv
    const int head = proj == 0 ? kh * G + hl : kh;               // head index inside its projection
    const f16* src = qkv + ((size_t)b * (Hq + 2 * Hkv) + hh) * D;
    h1 = src[pi];
    h2 = src[pi + half];
    with_delta = adapted && lx.B[proj] != nullptr;
    if (with_delta) {
      const int n_rows = (proj == 0 ? Hq : Hkv) * D;
      const f16* brow = lx.B[proj] + ((size_t)id * n_rows + (size_t)head * D) * lx.r;
      lora_row_load(brow + (size_t)pi * lx.r, lx.r, b1);
      lora_row_load(brow + (size_t)(pi + half) * lx.r, lx.r, b2);
    }
    rc = 1.f;
    rs = 0.f;
    if (proj != 2 && pos >= 0 && pos < max_pos) {
      rc = rope_cos[(size_t)pos * half + pi];
      rs = rope_sin[(size_t)pos * half + pi];
    }
  };
  auto finish = [&]() {
    if (with_delta) {
      h1 = (f16)((float)h1 + lora_row_dot_regs(b1, lv[proj], lx.r));
      h2 = (f16)((float)h2 + lora_row_dot_regs(b2, lv[proj], lx.r));
    }
    if (proj == 2) {
      vnew[pi] = h1;
      vnew[pi + half] = h2;
      if (new_page >= 0 && new_page < n_pages) {
        f16* dst = v_cache + ((size_t)new_page * Hkv + kh) * D * PAGE + new_slot;
        dst[(size_t)pi * PAGE] = h1;
        dst[(size_t)(pi + half) * PAGE] = h2;
      }
    } else {
      const float x1 = (float)h1, x2 = (float)h2;
      float r1, r2;
      {
#pragma clang fp contract(off)
        r1 = x1 * rc - x2 * rs;                    // separately rounded products, as in rope_kv_append_kernel
        r2 = x2 * rc + x1 * rs;
      }
      asm volatile("" : "+v"(r1), "+v"(r2));     // the fp32 result exists before the conversion
      const f16 o1 = (f16)r1, o2 = (f16)r2;
      if (proj == 0) {
        qs[hl * D + pi] = o1;
        qs[hl * D + pi + half] = o2;
      } else {
        knew[pi] = o1;
        knew[pi + half] = o2;
        if (new_page >= 0 && new_page < n_pages) {
          f16* dst = k_cache + ((size_t)new_page * Hkv + kh) * PAGE * D;
          dst[k_page_offset(new_slot, pi)] = o1;
          dst[k_page_offset(new_slot, pi + half)] = o2;
        }
      }
    }
  };
  const bool first = threadIdx.x < items;
  if (first) issue(threadIdx.x);
  // the o shrink's operand: thread (query head qh, rank entry j, 8-dim piece c) takes its 16 bytes of A_o[id] now and
  // parks them in LDS once they are there (the launcher has checked that the G * r * D / 8 items fit the workgroup)
  constexpr int OPC = D / 8;
  const bool o_mine = o_on && (int)threadIdx.x < G * os.r * OPC;
  f16x8 oa = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
  if (o_mine) oa = oshrink_piece<D>(os, oid_raw, G, kh, Hq);
  if (adapted) {
    if (lx.src.kc == 0 && lx.src.kq > 1) {
      // dense shrink results in kq blocks of K-range partials: one thread per (block, entry) fetches, then the blocks
      // are added in order - no thread waits for more than one load
      for (int e = threadIdx.x; e < lx.src.kq * 3 * lx.r; e += NW * WAVE) {
        const int q = e / (3 * lx.r), pj = (e / lx.r) % 3, j = e % lx.r;
        lvq[q][pj][j] = lx.B[pj] != nullptr
                            ? lx.src.v[((size_t)q * lx.src.T + b) * lx.src.ld + ((size_t)pj * lx.src.n_ad + id) * lx.r + j]
                            : 0.f;
      }
      __syncthreads();
      for (int e = threadIdx.x; e < 3 * lx.r; e += NW * WAVE) {
        const int pj = e / lx.r, j = e % lx.r;
        float a = lvq[0][pj][j];
        for (int q = 1; q < lx.src.kq; ++q) a += lvq[q][pj][j];
        lv[pj][j] = a * lx.scaling;
      }
    } else {
      for (int e = threadIdx.x; e < 3 * lx.r; e += NW * WAVE) {
        const int pj = e / lx.r, j = e % lx.r;
        lv[pj][j] = lx.B[pj] != nullptr ? lora_v_from(lx.src, pj, id, lx.r, b, j, lx.scaling) : 0.f;
      }
    }
    __syncthreads();
  }
  if (first) finish();
  if (o_mine) oslice[threadIdx.x] = oa;
  for (int it = threadIdx.x + NW * WAVE; it < items; it += NW * WAVE) {
    issue(it);
    finish();
  }
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  f32x4 O[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) O[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  // one page: scores against the rotated queries (Q^T as the B operand, read from LDS: lane holds
  // q[head col][kb*32 + g*8 .. +8], zero for unused columns), online softmax, value accumulation
  auto process = [&](f16x8 (&k)[NKB], f16x4 (&v)[NDB], int pg) {
    if (pg == new_pg) {                                   // wave-uniform: this page holds the token appended above
      if (col == new_slot) {
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) k[kb] = *reinterpret_cast<const f16x8*>(&knew[kb * 32 + g * 8]);
      }
      if ((new_slot >> 2) == g) {
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const f16 nv = vnew[db * 16 + col];
          const int e = new_slot & 3;
          v[db][0] = e == 0 ? nv : v[db][0];
          v[db][1] = e == 1 ? nv : v[db][1];
          v[db][2] = e == 2 ? nv : v[db][2];
          v[db][3] = e == 3 ? nv : v[db][3];
        }
      }
    }
    f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      const f16x8 qf = col < G ? *reinterpret_cast<const f16x8*>(&qs[col * D + kb * 32 + g * 8]) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
      st = __builtin_amdgcn_mfma_f32_16x16x32_f16(k[kb], qf, st, 0, 0, 0);
    }
    float pm = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      st[r] = (pg * PAGE + 4 * g + r >= ctx) ? -INFINITY : st[r] * scale;
      pm = fmaxf(pm, st[r]);
    }
    pm = fmaxf(pm, __shfl_xor(pm, 16, WAVE));
    pm = fmaxf(pm, __shfl_xor(pm, 32, WAVE));
    const float m_new = fmaxf(m, pm);
    const float alpha = __expf(m - m_new);
    f16x8 pa;
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p = __expf(st[r] - m_new);
      ps += p;
      const f16 hi = (f16)p;
      pa[r] = hi;
      pa[4 + r] = (f16)(p - (float)hi);
    }
    l = l * alpha + ps;
    m = m_new;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      O[db] *= alpha;
      const f16x8 vv = f16x8{v[db][0], v[db][1], v[db][2], v[db][3], v[db][0], v[db][1], v[db][2], v[db][3]};
      O[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vv, pa, O[db], 0, 0, 0);
    }
  };
  // the two pages requested at the start, then one page at a time with the next page id requested one page ahead
  constexpr int AHEAD = PF2 ? 2 : 1;
  int next = wave + AHEAD * NW < npages ? bt[wave + AHEAD * NW] : -1;
  if (page >= 0 && page < n_pages) process(kf, vf, wave);
  if constexpr (PF2) {
    if (page2 >= 0 && page2 < n_pages) process(kf2, vf2, wave + NW);
  }
  page = next;
  for (int pg = wave + AHEAD * NW; pg < npages; pg += NW) {
    next = pg + NW < npages ? bt[pg + NW] : -1;
    if (page >= 0 && page < n_pages) {                      // wave-uniform
      load_page(page);
      process(kf, vf, pg);
    }
    page = next;
  }
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  if (col < G) {
#pragma unroll
    for (int db = 0; db < NDB; ++db)
      *reinterpret_cast<f32x4*>(&sacc[((size_t)wave * G + col) * D + db * 16 + 4 * g]) = O[db];
    if (g == 0) {
      sm[wave][col] = m;
      sl[wave][col] = l;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < G * D; e += NW * WAVE) {
    const int qh = e / D, d = e % D;
    float M = sm[0][qh];
#pragma unroll
    for (int w = 1; w < NW; ++w) M = fmaxf(M, sm[w][qh]);
    float L = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = sm[w][qh] == -INFINITY ? 0.f : __expf(sm[w][qh] - M);
      L += sl[w][qh] * f;
      o += sacc[((size_t)w * G + qh) * D + d] * f;
    }
    const int h = kh * G + qh;
    const size_t oo = frag_tt ? frag_offset(b, h * D + d, frag_tt) : ((size_t)b * Hq + h) * D + d;
    const f16 of = (f16)(L > 0.f ? o / L : 0.f);
    out[oo] = of;
    if (o_on) qs[qh * D + d] = of;                           // the rotated queries are no longer needed: the outputs as stored
  }
  if (o_on) {                                                // uniform
    __syncthreads();
    if (o_mine) oshrink_head_shares<D>(os, oslice[threadIdx.x], qs, G, kh, b);
  }
}

// ---------------------------------------------------------------------------------------------
// Prefill: four waves own 128 consecutive query tokens of one head, a wave 32 of them as two 16-query tiles.  S^T = K . Q^T
// on v_mfma_f32_16x16x32_f16 puts the key index on the accumulator rows, which is exactly the A-operand layout the matrix
// core wants for P in O = P . V (a lane's four accumulator rows are the four keys it must supply): no shuffles between
// the two products.  The keys are walked in blocks of 64 (four pages).  The block's K and V pages go from the cache
// straight into LDS (a page per wave; a head's page of K or V is 4 KiB contiguous in the cache), double buffered - the
// next block is in flight while this one is multiplied - with one barrier per block, and all waves take their
// fragments from there: a page is fetched once per 128 queries, and a K or V fragment read from LDS is multiplied with
// both of the wave's query tiles - with one tile per wave the LDS reads (32 KiB per wave and block for 48 MFMAs) were
// what the kernel waited for, and more waves per SIMD only made that worse.  Two workgroups share a compute unit.  The
// softmax bookkeeping (running maximum, rescaling of O, the fp16 hi + lo split of P) is done once per 64 keys and tile
// - the two tiles' chains are independent, which gives the scheduler something to fill the waits with - and a P . V
// product covers 32 keys per MFMA (k-slots 0-3 and 4-7 of a lane are its four keys of two pages), hi and lo halves of
// P in two MFMAs on the same V fragment.  Blocks above the causal diagonal of a tile are skipped by that tile; blocks
// below it need no mask.  Token blocks that span several sequences are worked off one sequence at a time with the
// other queries masked.  The results cross LDS once more to leave as whole 16-byte pieces.
// Workgroups are dispatched longest key range first over all heads (grid = (heads, token blocks), late token blocks
// first): with the token block as the fast grid dimension the long workgroups of the last heads started late and ran
// alone at the end - 0.9 resident waves per SIMD on average, 551 instead of 336 us for one sequence of 4096 tokens.
// (8 x 512 tokens, 32 heads of 128: 60 us, 0.29 PFLOP/s of causal QK^T + PV; one sequence of 4096: 269 us, 0.51.  With the V pieces
// in LDS in cache order - the 8-byte V reads of 16 neighbouring dims then fall on every other 16-byte bank group, twice: by
// counters 60 % of the LDS cycles were bank conflicts - and the compiler's own pairing of these reads (two dims of one page,
// then 28 register moves per 16 MFMAs to put an operand's halves side by side): 71 and 304 us.  With the hi half
// of P rounded to nearest, converted back and subtracted - ten instructions per pair of probabilities instead of six: 73 and 315 us; with O and l
// rescaled in every block on top of that: 77 and 336 us; before the dispatch order was changed: 90 and 551 us; with one query tile per wave on top of that: 121 and 599 us; that form with eight waves per workgroup and four waves per SIMD: 102 and 655;
// with 32-key blocks and a four-deep ring: 134 and 732; adding P . V of the previous block under the softmax arithmetic
// of the current one: no faster.)
// ---------------------------------------------------------------------------------------------
constexpr int PF_WAVES = 4;
constexpr int PF_QT = 2;         // 16-query tiles per wave: a K or V fragment read from LDS serves that many MFMAs
constexpr int PF_PAGES = 4;      // pages per key block
constexpr int PF_RING = 2;       // key-block buffers

__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

template <int D>
__global__ __launch_bounds__(PF_WAVES* WAVE, 2) void paged_attn_prefill_block_kernel(
    f16* __restrict__ out, int frag_tt, const f16* __restrict__ qkv, const f16* __restrict__ k_cache, const f16* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
    int T, int Hq, int Hkv, int n_pages, int n_seq, float scale) {
  constexpr int NKB = D / 32;                // k-blocks of the QK^T product
  constexpr int NDB = D / 16;                // dim blocks of the output
  constexpr int PE = PAGE * D;               // elements of one page of K (or V) of one head
  constexpr int CH = PE / 512;               // 1 KiB pieces of such a page
  constexpr int WPP = PF_WAVES / PF_PAGES;    // waves that share the fetch of a page
  constexpr int HC = CH / WPP;               // 1 KiB pieces of K (and of V) a wave fetches per block
  constexpr int BUF = 2 * PF_PAGES * PE;     // one buffer: K pages, then V pages
  constexpr int OLD = D + 8;                 // padded row of the output staging
  constexpr int QT = PF_QT;                  // 16-query tiles of a wave
  constexpr int WTOK = 16 * QT;              // queries of a wave
  constexpr int NTOK = PF_WAVES * WTOK;
  static_assert(PF_WAVES % PF_PAGES == 0 && CH % WPP == 0 && NTOK <= 2 * WAVE, "whole waves per page; at most two tokens per lane in the sequence scan");
  static_assert((size_t)NTOK * OLD <= (size_t)PF_RING * BUF, "the output staging fits the ring");
  extern __shared__ __align__(16) f16 smem[];   // [PF_RING][BUF]
  __shared__ int s_seq[NTOK], s_pos[NTOK];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int qi = lane & 15, g = lane >> 4;
  // grid = (heads, token blocks): workgroups are dispatched head by head within a token block, late token blocks
  // (long key ranges) first, so that the longest workgroups of every head start at once and the short ones fill in
  const int t0 = (gridDim.y - 1 - blockIdx.y) * NTOK;
  const int tw = t0 + wave * WTOK;
  const int h = blockIdx.x, kh = h / (Hq / Hkv);

  // the V slots start at zero: a slot whose page is never fetched (a sequence shorter than a key block) is multiplied
  // by P = 0 and must hold finite numbers
  for (int i = threadIdx.x; i < PF_RING * PF_PAGES * PE / 8; i += PF_WAVES * WAVE) {
    const int bsel = i / (PF_PAGES * PE / 8), o = i % (PF_PAGES * PE / 8);
    st8(smem + bsel * BUF + PF_PAGES * PE + o * 8, f16x8{0, 0, 0, 0, 0, 0, 0, 0});
  }
  for (int i = threadIdx.x; i < NTOK; i += PF_WAVES * WAVE) {
    const int t = t0 + i;
    int sq = t < T ? tok_seq[t] : -1;
    int ps = t < T ? tok_pos[t] : -1;
    if (sq < 0 || sq >= n_seq || ps < 0 || ps >= max_blocks * PAGE) sq = -1;
    s_seq[i] = sq;
    s_pos[i] = ps;
  }
  __syncthreads();
  const int seq_a = s_seq[lane], pos_a = s_pos[lane];                // token t0 + lane
  const int seq_b = WAVE + lane < NTOK ? s_seq[(WAVE + lane) % NTOK] : -1, pos_b = s_pos[(WAVE + lane) % NTOK];   // token t0 + 64 + lane
  int my_seq[QT], my_pos[QT];
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    my_seq[u] = s_seq[wave * WTOK + u * 16 + qi];
    my_pos[u] = s_pos[wave * WTOK + u * 16 + qi];
  }

  f16x8 qf[QT][NKB];                         // Q as the B operand: q[query qi of tile u][kb * 32 + g * 8 ..]
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    const int tq = tw + u * 16 + qi < T ? tw + u * 16 + qi : T - 1;
    const f16* qp = qkv + ((size_t)tq * (Hq + 2 * Hkv) + h) * D + g * 8;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) qf[u][kb] = ld8(qp + kb * 32);
  }
  const float c = scale * 1.44269504088896340736f;                  // softmax in base 2
  float m[QT], l[QT];
  f32x4 O[QT][NDB];
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    m[u] = -INFINITY;
    l[u] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db) O[u][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  unsigned long long todo_a = __ballot(seq_a >= 0), todo_b = __ballot(seq_b >= 0);
  while (todo_a | todo_b) {                                          // one pass per sequence of the token block (uniform over the workgroup)
    const int cur = __builtin_amdgcn_readfirstlane(todo_a ? __shfl(seq_a, __builtin_ctzll(todo_a), WAVE)
                                                          : __shfl(seq_b, __builtin_ctzll(todo_b), WAVE));
    todo_a &= ~__ballot(seq_a == cur);
    todo_b &= ~__ballot(seq_b == cur);
    int run_max = max(seq_a == cur ? pos_a : -1, seq_b == cur ? pos_b : -1);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) run_max = max(run_max, __shfl_xor(run_max, o, WAVE));
    run_max = __builtin_amdgcn_readfirstlane(run_max);
    const int npages = run_max / PAGE + 1, nblk = (npages + PF_PAGES - 1) / PF_PAGES;
    // per query tile: is it part of this sequence, and between which positions do its queries lie
    bool in_run[QT], all_in[QT];
    int tmax[QT], tmin[QT];
    int wmax = -1;
#pragma unroll
    for (int u = 0; u < QT; ++u) {
      in_run[u] = my_seq[u] == cur;
      int hi = in_run[u] ? my_pos[u] : -1, lo = in_run[u] ? my_pos[u] : 0x7fffffff;
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) {
        hi = max(hi, __shfl_xor(hi, o, WAVE));
        lo = min(lo, __shfl_xor(lo, o, WAVE));
      }
      tmax[u] = __builtin_amdgcn_readfirstlane(hi);                  // lanes 0-15 hold the 16 queries; all g copies agree
      tmin[u] = __builtin_amdgcn_readfirstlane(lo);
      all_in[u] = (__ballot(in_run[u]) & 0xffffull) == 0xffffull;
      wmax = max(wmax, tmax[u]);
    }
    const int32_t* __restrict__ bt = block_table + (size_t)cur * max_blocks;

    // this wave's part of block b into its ring slot: HC pieces of K and HC pieces of V, always - a page past the
    // sequence or outside the cache is replaced by page 0 (finite data; every key of it is masked), so that the
    // number of loads in flight tells which blocks have landed
    auto issue = [&](int b) {
      const int pg = b * PF_PAGES + wave / WPP;
      int page = pg < npages ? bt[pg] : 0;
      page = page >= 0 && page < n_pages ? page : 0;
      const size_t src = ((size_t)page * Hkv + kh) * PE + (wave % WPP) * HC * 512;
      f16* kd = smem + (b % PF_RING) * BUF + (wave / WPP) * PE + (wave % WPP) * HC * 512;
      // the V pieces of a page pair alternate (piece j of the even page, piece j of the odd page, piece j + 1 ...): a
      // lane's four keys of both pages are then 1 KiB apart and one two-address LDS read delivers the whole operand
      f16* vd = smem + (b % PF_RING) * BUF + PF_PAGES * PE + ((((wave / WPP) >> 1) * CH + (wave % WPP) * HC) * 2 + ((wave / WPP) & 1)) * 512;
      // K pieces keep their order.  A 1 KiB piece of V is 32 dims x (two 16-byte halves of the 16 keys): lane l fetches
      // half l / 32 of dim l % 32, so that the LDS copy holds the 32 first halves side by side, then the 32 second
      // halves - the 16 lanes that read the same half of 16 neighbouring dims then hit 16 different 16-byte bank groups
      // (in cache order they hit every other one, twice)
      const int vsrc = (lane & 31) * PAGE + (lane >> 5) * 8;
#pragma unroll
      for (int j = 0; j < HC; ++j) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(k_cache + src + j * 512 + lane * 8),
                                         (__attribute__((address_space(3))) void*)(kd + j * 512), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(v_cache + src + j * 512 + vsrc),
                                         (__attribute__((address_space(3))) void*)(vd + j * 1024), 16, 0, 0);
      }
    };
#pragma unroll
    for (int b = 0; b < PF_RING - 1; ++b)
      if (b < nblk) issue(b);
    for (int b = 0; b < nblk; ++b) {
      // this wave's part of block b has landed: only the loads of the younger blocks (at most two) may be in flight
      const int younger = nblk - 1 - b < PF_RING - 2 ? nblk - 1 - b : PF_RING - 2;   // uniform
      if (younger == 2) {
        if constexpr (2 * HC == 4) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if constexpr (2 * HC == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
      } else if (younger == 1) {
        if constexpr (2 * HC == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if constexpr (2 * HC == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      static_assert(PF_RING <= 4 && (2 * HC == 2 || 2 * HC == 4 || 2 * HC == 8), "the immediates above are 2 HC loads per block in flight");
      // everybody's has; nobody reads block b - 1 any more.  The bare barrier: __syncthreads() would first wait for the
      // loads of the younger blocks as well (see bare_barrier)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      bare_barrier();
      if (b + PF_RING - 1 < nblk) issue(b + PF_RING - 1);           // into the slot of block b - 1
      if (wmax < b * PF_PAGES * PAGE) continue;                      // wave-uniform: the block lies above this wave's diagonal
      const f16* kb_ = smem + (b % PF_RING) * BUF;
      const f16* vb_ = kb_ + PF_PAGES * PE;
      // All pages are multiplied without branches; what must not count is masked after the product.  A page that
      // was not fetched (past the sequence, or a page id outside the cache) leaves older, finite data in its slot.
      bool live[PF_PAGES];                                           // uniform
      bool all_live = true;
#pragma unroll
      for (int p = 0; p < PF_PAGES; ++p) {
        const int pg = b * PF_PAGES + p;
        const int page = pg < npages ? bt[pg] : -1;
        live[p] = page >= 0 && page < n_pages;
        all_live = all_live && live[p];
      }
      bool act[QT];                                                  // uniform: the tile has queries at or below the block
#pragma unroll
      for (int u = 0; u < QT; ++u) act[u] = tmax[u] >= b * PF_PAGES * PAGE;
      // S^T of the block for the wave's query tiles: a K fragment is read from LDS once and multiplied with every tile
      f32x4 st[QT][PF_PAGES];                                        // st[u][p][r] = S[key 4g + r of page p][query qi of tile u] (tiles at work only)
#pragma unroll
      for (int p = 0; p < PF_PAGES; ++p) {
        f16x8 kf[NKB];
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb) kf[kb] = ld8(kb_ + p * PE + kb * 512 + lane * 8);
#pragma unroll
        for (int u = 0; u < QT; ++u) {
          if (act[u]) {                                              // the first product starts from a zero operand, not from zeroed registers
            f32x4 sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[0], qf[u][0], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
            for (int kb = 1; kb < NKB; ++kb) sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[kb], qf[u][kb], sacc, 0, 0, 0);
            st[u][p] = sacc;
          }
        }
      }
      // online softmax per tile; P as fp16 hi + lo halves (~22 mantissa bits): hi is P rounded to fp16, lo the remainder
      f16x8 ph[QT][PF_PAGES / 2], pl[QT][PF_PAGES / 2];
#pragma unroll
      for (int u = 0; u < QT; ++u) {
        if (!act[u]) continue;
        if (!(all_in[u] && all_live && (b + 1) * PF_PAGES * PAGE - 1 <= tmin[u])) {   // uniform: some key of the block is masked
          // key (p, r) of this lane lies `p * PAGE + r` behind the block's first key of the lane's group: one
          // subtraction per tile, then a compare with a constant per score
          const int lim = in_run[u] ? my_pos[u] - (b * PF_PAGES * PAGE + 4 * g) : -1;
#pragma unroll
          for (int p = 0; p < PF_PAGES; ++p) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const bool masked = !live[p] || p * PAGE + r > lim;
              st[u][p][r] = masked ? -INFINITY : st[u][p][r];
            }
          }
        }
        // the block's maximum per query: the scores are finite or -inf, never NaN, so the three-input maximum is taken as
        // the instruction gives it (through fmaxf the compiler first passes every score through a quieting v_max)
        static_assert(PF_PAGES == 4, "the tree below names the sixteen scores of four pages");
        const float t0 = max3_raw(st[u][0][0], st[u][0][1], st[u][0][2]), t1 = max3_raw(st[u][0][3], st[u][1][0], st[u][1][1]);
        const float t2 = max3_raw(st[u][1][2], st[u][1][3], st[u][2][0]), t3 = max3_raw(st[u][2][1], st[u][2][2], st[u][2][3]);
        const float t4 = max3_raw(st[u][3][0], st[u][3][1], st[u][3][2]);
        float pm = max3_raw(max3_raw(t0, t1, t2), max3_raw(t3, t4, st[u][3][3]), t0);
        pm = max3_raw(pm, __shfl_xor(pm, 16, WAVE), pm);
        pm = max3_raw(pm, __shfl_xor(pm, 32, WAVE), pm);
        // The reference maximum m moves - and O and l are rescaled - only when some query of the tile meets a score more
        // than 2^8 above it (always in the tile's first block); otherwise the block's P are taken relative to the old
        // reference and may reach 256, which fp16 holds exactly as well.  After the first blocks of a sequence that
        // saves the rescaling arithmetic (32 multiplies, four cross-lane moves, an exponential) of almost every block.
        const bool need = (pm - m[u]) * c > 8.f;                     // m = -inf: true for a finite pm, false (NaN) for pm = -inf
        if (__ballot(need)) {                                        // wave-uniform
          const float m_new = fmaxf(m[u], pm);
          const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f((m[u] - m_new) * c);
          l[u] *= alpha;
          m[u] = m_new;
          float ar[4];                                               // O rows are queries 4g + r; their alpha lives in lanes with qi == 4g + r
#pragma unroll
          for (int r = 0; r < 4; ++r) ar[r] = __shfl(alpha, 4 * g + r, WAVE);
#pragma unroll
          for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) O[u][db][r] *= ar[r];
        }
        const float mc = m[u] == -INFINITY ? 0.f : m[u] * c;
        float ps = 0.f;
#pragma unroll
        for (int p = 0; p < PF_PAGES; ++p) {
#pragma unroll
          for (int r = 0; r < 4; r += 2) {
            // hi = P cut to fp16's eleven significant bits (a mask: exact in fp16 down to its normal range), lo = the
            // exact remainder cut to eleven bits of its own; both pairs leave through one two-element conversion each
            const float p0 = __builtin_amdgcn_exp2f(fmaf(st[u][p][r], c, -mc));       // exp2(-inf) = 0 for masked keys
            const float p1 = __builtin_amdgcn_exp2f(fmaf(st[u][p][r + 1], c, -mc));
            ps += p0;
            ps += p1;
            const float h0 = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, p0) & 0xffffe000u);
            const float h1 = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, p1) & 0xffffe000u);
            const auto hh = __builtin_amdgcn_cvt_pkrtz(h0, h1), ll = __builtin_amdgcn_cvt_pkrtz(p0 - h0, p1 - h1);
            ph[u][p / 2][(p & 1) * 4 + r] = hh[0];
            ph[u][p / 2][(p & 1) * 4 + r + 1] = hh[1];
            pl[u][p / 2][(p & 1) * 4 + r] = ll[0];
            pl[u][p / 2][(p & 1) * 4 + r + 1] = ll[1];
          }
        }
        l[u] += ps;
      }
      // O += P . V: a V fragment (dim db * 16 + qi, keys 4g .. of the pair's two pages) is read once for all tiles
      static_assert(PF_PAGES % 2 == 0, "page pairs");
#pragma unroll
      for (int pp = 0; pp < PF_PAGES / 2; ++pp) {
        __builtin_amdgcn_sched_barrier(0);                           // the V fragments are not requested before they fit the register file
        f16x8 vv[NDB];
        // dim db * 16 + qi, keys 4 g .. of the pair's two pages: piece db / 2 of the pair, half g / 2, then dim (db % 2) * 16 + qi
        // of that piece; the odd page's copy lies 1 KiB behind.  One two-address read per operand, written out: left to
        // itself the compiler pairs the reads of two neighbouring dims of one page and then moves the halves together,
        // 28 register moves per 16 MFMAs.  Reads issued this way are not in the compiler's count of outstanding LDS
        // operations, hence the explicit wait.
        const unsigned vaddr = (unsigned)(size_t)(const __attribute__((address_space(3))) f16*)(vb_ + pp * CH * 1024 + ((g >> 1) * 32 + qi) * 8 + (g & 1) * 4);
#pragma unroll
        for (int db = 0; db < NDB; db += 2) {
          asm volatile("ds_read2_b64 %0, %2 offset1:128\n\tds_read2_b64 %1, %2 offset0:32 offset1:160"
                       : "=&v"(vv[db]), "=&v"(vv[db + 1]) : "v"(vaddr + (db >> 1) * 2048));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int u = 0; u < QT; ++u) {
          if (!act[u]) continue;
#pragma unroll
          for (int db = 0; db < NDB; ++db) O[u][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph[u][pp], vv[db], O[u][db], 0, 0, 0);
#pragma unroll
          for (int db = 0; db < NDB; ++db) O[u][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pl[u][pp], vv[db], O[u][db], 0, 0, 0);
        }
      }
    }
    __syncthreads();                                                 // the buffers are free for the next sequence (and for the output)
  }
  // results through the wave's own piece of LDS: [16 QT queries][D] fp16, then 16-byte pieces out
  f16* os = smem + wave * WTOK * OLD;
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    float lu = l[u];
    lu += __shfl_xor(lu, 16, WAVE);
    lu += __shfl_xor(lu, 32, WAVE);
    const float inv = lu > 0.f ? 1.f / lu : 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float ir = __shfl(inv, 4 * g + r, WAVE);
#pragma unroll
      for (int db = 0; db < NDB; ++db) os[(u * 16 + 4 * g + r) * OLD + db * 16 + qi] = (f16)(O[u][db][r] * ir);
    }
  }
  __builtin_amdgcn_wave_barrier();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if (frag_tt) {
#pragma unroll
    for (int u = 0; u < QT; ++u) {
#pragma unroll
      for (int j = 0; j < D / 32; ++j) {                             // one whole fragment per store instruction
        const int tok = lane & 15, kg = lane >> 4;
        const int t = tw + u * 16 + tok;
        if (t < T) st8(out + frag_offset(t, h * D + j * 32 + kg * 8, frag_tt), ld8(os + (u * 16 + tok) * OLD + j * 32 + kg * 8));
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < WTOK * (D / 8) / WAVE; ++i) {
      const int ch = i * WAVE + lane, row = ch / (D / 8), c8 = ch % (D / 8);
      if (tw + row < T) st8(out + ((size_t)(tw + row) * Hq + h) * D + c8 * 8, ld8(os + row * OLD + c8 * 8));
    }
  }
}

int check_attn(const char* who, int Hq, int Hkv, int D, int n_pages, int n_seq, int max_blocks) {
  MLORA_CHECK(D == 64 || D == 128, MLORA_ERR_UNSUPPORTED, "%s: head_dim %d not in {64, 128}", who, D);
  MLORA_CHECK(Hq > 0 && Hkv > 0 && Hq % Hkv == 0, MLORA_ERR_INVALID, "%s: bad heads Hq=%d Hkv=%d", who, Hq, Hkv);
  MLORA_CHECK(n_pages > 0 && n_seq > 0 && max_blocks > 0, MLORA_ERR_INVALID, "%s: bad cache shape n_pages=%d n_seq=%d max_blocks=%d", who, n_pages, n_seq, max_blocks);
  MLORA_CHECK(Hq + 2 * Hkv <= 65535, MLORA_ERR_UNSUPPORTED, "%s: too many heads", who);
  return MLORA_OK;
}

}  // namespace

static int rope_kv_append_impl(const char* who, void* qkv, void* k_cache, void* v_cache, const int32_t* block_table,
                               int max_blocks, const int32_t* tok_seq, const int32_t* tok_pos, const float* rope_cos,
                               const float* rope_sin, int max_pos, int T, int Hq, int Hkv, int D, int n_pages, int n_seq,
                               const LoraExpandQKV& lx, void* stream) {
  if (int e = check_attn(who, Hq, Hkv, D, n_pages, n_seq, max_blocks)) return e;
  MLORA_CHECK(qkv && k_cache && v_cache && block_table && tok_seq && tok_pos && rope_cos && rope_sin, MLORA_ERR_INVALID, "%s: null pointer", who);
  MLORA_CHECK(T >= 0 && max_pos > 0, MLORA_ERR_INVALID, "%s: bad T=%d max_pos=%d", who, T, max_pos);
  if (T == 0) return MLORA_OK;
  if (T > 64 && lx.src.v == nullptr && (((uintptr_t)rope_cos | (uintptr_t)rope_sin) & 15) == 0) {
    const dim3 grid(ceil_div(T, 16), ceil_div(Hq + 2 * Hkv, 4));
    if (D == 128)
      hipLaunchKernelGGL(rope_kv_append_tile_kernel<128>, grid, dim3(256), 0, (hipStream_t)stream, (f16*)qkv, (f16*)k_cache,
                         (f16*)v_cache, block_table, max_blocks, tok_seq, tok_pos, rope_cos, rope_sin, max_pos, Hq, Hkv, n_pages,
                         n_seq, T);
    else
      hipLaunchKernelGGL(rope_kv_append_tile_kernel<64>, grid, dim3(256), 0, (hipStream_t)stream, (f16*)qkv, (f16*)k_cache,
                         (f16*)v_cache, block_table, max_blocks, tok_seq, tok_pos, rope_cos, rope_sin, max_pos, Hq, Hkv, n_pages,
                         n_seq, T);
    return mlora_launch_status(who);
  }
  hipLaunchKernelGGL(rope_kv_append_kernel, dim3(T, Hq + 2 * Hkv), dim3(64), 0, (hipStream_t)stream, (f16*)qkv,
                     (f16*)k_cache, (f16*)v_cache, block_table, max_blocks, tok_seq, tok_pos, rope_cos, rope_sin,
                     max_pos, Hq, Hkv, D, n_pages, n_seq, T, lx);
  return mlora_launch_status(who);
}

extern "C" int mlora_rope_kv_append(void* qkv, void* k_cache, void* v_cache, const int32_t* block_table, int max_blocks,
                                    const int32_t* tok_seq, const int32_t* tok_pos, const float* rope_cos,
                                    const float* rope_sin, int max_pos, int T, int Hq, int Hkv, int D, int n_pages,
                                    int n_seq, void* stream) {
  return rope_kv_append_impl("rope_kv_append", qkv, k_cache, v_cache, block_table, max_blocks, tok_seq, tok_pos, rope_cos,
                             rope_sin, max_pos, T, Hq, Hkv, D, n_pages, n_seq, LoraExpandQKV(), stream);
}

extern "C" int mlora_rope_kv_append_lora(void* qkv, void* k_cache, void* v_cache, const int32_t* block_table,
                                         int max_blocks, const int32_t* tok_seq, const int32_t* tok_pos,
                                         const float* rope_cos, const float* rope_sin, int max_pos, int T, int Hq, int Hkv,
                                         int D, int n_pages, int n_seq, const void* v_part, int v_dense,
                                         const void* const* B, const int32_t* tok_adapter, float scaling, int K, int r,
                                         int n_ad, void* stream) {
  MLORA_CHECK(v_part && B && tok_adapter, MLORA_ERR_INVALID, "rope_kv_append_lora: null LoRA argument");
  MLORA_CHECK((r == 8 || r == 16 || r == 32 || r == 64) && n_ad > 0 && K > 0, MLORA_ERR_UNSUPPORTED,
              "rope_kv_append_lora: rank %d not in {8,16,32,64} or bad n_ad/K", r);
  MLORA_CHECK(v_dense >= 0 && v_dense <= LORA_MAX_KQ, MLORA_ERR_UNSUPPORTED,
              "rope_kv_append_lora: v_dense=%d outside 0..%d (K-range blocks of dense shrink results)", v_dense, LORA_MAX_KQ);
  LoraExpandQKV lx = {};
  lx.src.v = (const float*)v_part;
  lx.src.kc = v_dense ? 0 : lora_k_split(K).kc;
  lx.src.kq = v_dense > 0 ? v_dense : 1;
  lx.src.T = T; lx.src.n_ad = n_ad; lx.src.ld = 3 * n_ad * r;
  for (int i = 0; i < 3; ++i) lx.B[i] = (const f16*)B[i];
  lx.ids = tok_adapter;
  lx.scaling = scaling;
  lx.r = r; lx.n_ad = n_ad;
  return rope_kv_append_impl("rope_kv_append_lora", qkv, k_cache, v_cache, block_table, max_blocks, tok_seq, tok_pos,
                             rope_cos, rope_sin, max_pos, T, Hq, Hkv, D, n_pages, n_seq, lx, stream);
}

static int paged_attn_decode_impl(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                                  const int32_t* block_table, int max_blocks, const int32_t* seq_ids,
                                  const int32_t* ctx_len, int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                  const int32_t* tok_adapter, int r, int n_ad, const void* o_A, void* o_vpart, void* stream) {
  if (int e = check_attn("paged_attn_decode", Hq, Hkv, D, n_pages, n_seq, max_blocks)) return e;
  MLORA_CHECK(out && qkv && k_cache && v_cache && block_table && seq_ids && ctx_len, MLORA_ERR_INVALID, "paged_attn_decode: null pointer");
  MLORA_CHECK(B >= 0 && B <= 65535, MLORA_ERR_INVALID, "paged_attn_decode: bad B=%d (0..65535)", B);
  MLORA_CHECK(out_layout == MLORA_ROWMAJOR || out_layout == MLORA_FRAG, MLORA_ERR_INVALID, "paged_attn_decode: bad out_layout %d", out_layout);
  const int frag_tt = out_layout == MLORA_FRAG ? mlora_frag_tiles(B) : 0;
  if (B == 0) return MLORA_OK;
  const float scale = 1.f / sqrtf((float)D);
  hipStream_t s = (hipStream_t)stream;
  const int G = Hq / Hkv;
  MLORA_CHECK(G <= 16, MLORA_ERR_UNSUPPORTED, "paged_attn_decode: more than 16 query heads per kv head (%d)", G);
  OShrinkHeads os = {};
  if (o_A != nullptr) {
    MLORA_CHECK(o_vpart && tok_adapter && n_ad > 0, MLORA_ERR_INVALID, "paged_attn_decode: null o-shrink argument");
    MLORA_CHECK(mlora_rope_attn_oshrink_ok(B, Hq, Hkv, D, r), MLORA_ERR_UNSUPPORTED,
                "paged_attn_decode: the o shrink of rank %d does not fit the workgroup of this launch (B=%d Hq=%d Hkv=%d D=%d)", r, B, Hq, Hkv, D);
    os.A = (const f16*)o_A;
    os.vpart = (float*)o_vpart;
    os.ids = tok_adapter;
    os.r = r; os.n_ad = n_ad; os.T = B;
  }
  const int nw = attn_waves(B, Hkv, G, D);
  const size_t lds = (size_t)nw * G * D * sizeof(float);
#define MLORA_ATTN(DD, NWV)                                                                                                   \
  hipLaunchKernelGGL((paged_attn_decode_kernel<DD, NWV>), dim3(Hkv, B), dim3(NWV * WAVE), lds, s, (f16*)out, (const f16*)qkv, \
                     (const f16*)k_cache, (const f16*)v_cache, block_table, max_blocks, seq_ids, ctx_len, Hq, Hkv, n_pages,   \
                     n_seq, scale, frag_tt, os)
  if (D == 128) {
    if (nw == 16) MLORA_ATTN(128, 16);
    else if (nw == 8) MLORA_ATTN(128, 8);
    else MLORA_ATTN(128, 4);
  } else {
    if (nw == 16) MLORA_ATTN(64, 16);
    else if (nw == 8) MLORA_ATTN(64, 8);
    else MLORA_ATTN(64, 4);
  }
#undef MLORA_ATTN
  return mlora_launch_status("paged_attn_decode");
}

extern "C" int mlora_paged_attn_decode(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                                       const int32_t* block_table, int max_blocks, const int32_t* seq_ids,
                                       const int32_t* ctx_len, int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                       void* stream) {
  return paged_attn_decode_impl(out, out_layout, qkv, k_cache, v_cache, block_table, max_blocks, seq_ids, ctx_len, B, Hq, Hkv, D, n_pages,
                                n_seq, nullptr, 0, 0, nullptr, nullptr, stream);
}

extern "C" int mlora_paged_attn_decode_oshrink(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                                               const int32_t* block_table, int max_blocks, const int32_t* seq_ids,
                                               const int32_t* ctx_len, int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                               const int32_t* tok_adapter, int r, int n_ad, const void* o_A, void* o_vpart,
                                               void* stream) {
  MLORA_CHECK(o_A && o_vpart, MLORA_ERR_INVALID, "paged_attn_decode_oshrink: null o-shrink argument");
  return paged_attn_decode_impl(out, out_layout, qkv, k_cache, v_cache, block_table, max_blocks, seq_ids, ctx_len, B, Hq, Hkv, D, n_pages,
                                n_seq, tok_adapter, r, n_ad, o_A, o_vpart, stream);
}

// the o shrink's items (query heads of a kv head x rank entries x 8-dim pieces) must fit the workgroup the launch uses
extern "C" int mlora_rope_attn_oshrink_ok(int B, int Hq, int Hkv, int D, int r) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || (D != 64 && D != 128)) return 0;
  if (r != 8 && r != 16 && r != 32 && r != 64) return 0;
  const int G = Hq / Hkv;
  if (G > 16) return 0;
  return G * r * (D / 8) <= attn_waves(B, Hkv, G, D) * WAVE ? 1 : 0;
}

static int rope_attn_decode_impl(void* out, int out_layout, const void* qkv, void* k_cache, void* v_cache,
                                 const int32_t* block_table, int max_blocks, const int32_t* seq_ids,
                                 const int32_t* tok_pos, const int32_t* ctx_len, const float* rope_cos,
                                 const float* rope_sin, int max_pos, int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                 const void* v_part, int v_dense, const void* const* Bmat, const int32_t* tok_adapter,
                                 float scaling, int K, int r, int n_ad, const void* o_A, void* o_vpart, void* stream) {
  if (int e = check_attn("rope_attn_decode", Hq, Hkv, D, n_pages, n_seq, max_blocks)) return e;
  MLORA_CHECK(out && qkv && k_cache && v_cache && block_table && seq_ids && tok_pos && ctx_len && rope_cos && rope_sin,
              MLORA_ERR_INVALID, "rope_attn_decode: null pointer");
  MLORA_CHECK(B >= 0 && B <= 65535 && max_pos > 0, MLORA_ERR_INVALID, "rope_attn_decode: bad B=%d (0..65535) max_pos=%d", B, max_pos);
  MLORA_CHECK(out_layout == MLORA_ROWMAJOR || out_layout == MLORA_FRAG, MLORA_ERR_INVALID, "rope_attn_decode: bad out_layout %d", out_layout);
  const int G = Hq / Hkv;
  MLORA_CHECK(G <= 16, MLORA_ERR_UNSUPPORTED, "rope_attn_decode: more than 16 query heads per kv head (%d)", G);
  LoraExpandQKV lx = {};
  if (v_part != nullptr) {
    MLORA_CHECK(Bmat && tok_adapter, MLORA_ERR_INVALID, "rope_attn_decode: null LoRA argument");
    MLORA_CHECK((r == 8 || r == 16 || r == 32 || r == 64) && n_ad > 0 && K > 0, MLORA_ERR_UNSUPPORTED,
                "rope_attn_decode: rank %d not in {8,16,32,64} or bad n_ad/K", r);
    MLORA_CHECK(v_dense >= 0 && v_dense <= LORA_MAX_KQ, MLORA_ERR_UNSUPPORTED,
                "rope_attn_decode: v_dense=%d outside 0..%d (K-range blocks of dense shrink results)", v_dense, LORA_MAX_KQ);
    lx.src.v = (const float*)v_part;
    lx.src.kc = v_dense ? 0 : lora_k_split(K).kc;
    lx.src.kq = v_dense > 0 ? v_dense : 1;
    lx.src.T = B; lx.src.n_ad = n_ad; lx.src.ld = 3 * n_ad * r;
    for (int i = 0; i < 3; ++i) lx.B[i] = (const f16*)Bmat[i];
    lx.ids = tok_adapter;
    lx.scaling = scaling;
    lx.r = r; lx.n_ad = n_ad;
  }
  OShrinkHeads os = {};
  if (o_A != nullptr) {
    MLORA_CHECK(o_vpart && tok_adapter && n_ad > 0, MLORA_ERR_INVALID, "rope_attn_decode: null o-shrink argument");
    MLORA_CHECK(mlora_rope_attn_oshrink_ok(B > 0 ? B : 1, Hq, Hkv, D, r), MLORA_ERR_UNSUPPORTED,
                "rope_attn_decode: the o shrink of rank %d does not fit the workgroup of this launch (B=%d Hq=%d Hkv=%d D=%d)", r, B, Hq, Hkv, D);
    os.A = (const f16*)o_A;
    os.vpart = (float*)o_vpart;
    os.ids = tok_adapter;
    os.r = r; os.n_ad = n_ad; os.T = B;
  }
  if (B == 0) return MLORA_OK;
  const int frag_tt = out_layout == MLORA_FRAG ? mlora_frag_tiles(B) : 0;
  const float scale = 1.f / sqrtf((float)D);
  const int nw = attn_waves(B, Hkv, G, D);
  const size_t lds = (size_t)nw * G * D * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
#define MLORA_ROPE_ATTN(DD, RG, NWV)                                                                                             \
  hipLaunchKernelGGL((rope_attn_decode_kernel<DD, RG, NWV>), dim3(Hkv, B), dim3(NWV * WAVE), lds, s, (f16*)out, (const f16*)qkv, \
                     (f16*)k_cache, (f16*)v_cache, block_table, max_blocks, seq_ids, tok_pos, ctx_len, rope_cos, rope_sin,       \
                     max_pos, Hq, Hkv, n_pages, n_seq, scale, frag_tt, lx, os)
#define MLORA_ROPE_ATTN_NW(DD, RG)             \
  do {                                         \
    if (nw == 16) MLORA_ROPE_ATTN(DD, RG, 16); \
    else if (nw == 8) MLORA_ROPE_ATTN(DD, RG, 8); \
    else MLORA_ROPE_ATTN(DD, RG, 4);           \
  } while (0)
  const bool small_rank = v_part == nullptr || r <= 16;
  if (D == 128) {
    if (small_rank) MLORA_ROPE_ATTN_NW(128, 2);
    else MLORA_ROPE_ATTN_NW(128, 8);
  } else {
    if (small_rank) MLORA_ROPE_ATTN_NW(64, 2);
    else MLORA_ROPE_ATTN_NW(64, 8);
  }
#undef MLORA_ROPE_ATTN_NW
#undef MLORA_ROPE_ATTN
  return mlora_launch_status("rope_attn_decode");
}

extern "C" int mlora_rope_attn_decode(void* out, int out_layout, const void* qkv, void* k_cache, void* v_cache,
                                      const int32_t* block_table, int max_blocks, const int32_t* seq_ids,
                                      const int32_t* tok_pos, const int32_t* ctx_len, const float* rope_cos,
                                      const float* rope_sin, int max_pos, int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                      const void* v_part, int v_dense, const void* const* Bmat, const int32_t* tok_adapter,
                                      float scaling, int K, int r, int n_ad, void* stream) {
  return rope_attn_decode_impl(out, out_layout, qkv, k_cache, v_cache, block_table, max_blocks, seq_ids, tok_pos, ctx_len, rope_cos,
                               rope_sin, max_pos, B, Hq, Hkv, D, n_pages, n_seq, v_part, v_dense, Bmat, tok_adapter, scaling, K, r, n_ad,
                               nullptr, nullptr, stream);
}

extern "C" int mlora_rope_attn_decode_oshrink(void* out, int out_layout, const void* qkv, void* k_cache, void* v_cache,
                                              const int32_t* block_table, int max_blocks, const int32_t* seq_ids,
                                              const int32_t* tok_pos, const int32_t* ctx_len, const float* rope_cos,
                                              const float* rope_sin, int max_pos, int B, int Hq, int Hkv, int D, int n_pages,
                                              int n_seq, const void* v_part, int v_dense, const void* const* Bmat,
                                              const int32_t* tok_adapter, float scaling, int K, int r, int n_ad, const void* o_A,
                                              void* o_vpart, void* stream) {
  MLORA_CHECK(o_A && o_vpart, MLORA_ERR_INVALID, "rope_attn_decode_oshrink: null o-shrink argument");
  return rope_attn_decode_impl(out, out_layout, qkv, k_cache, v_cache, block_table, max_blocks, seq_ids, tok_pos, ctx_len, rope_cos,
                               rope_sin, max_pos, B, Hq, Hkv, D, n_pages, n_seq, v_part, v_dense, Bmat, tok_adapter, scaling, K, r, n_ad,
                               o_A, o_vpart, stream);
}

extern "C" int mlora_paged_attn_prefill(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                                        const int32_t* block_table, int max_blocks, const int32_t* tok_seq,
                                        const int32_t* tok_pos, int T, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                        void* stream) {
  if (int e = check_attn("paged_attn_prefill", Hq, Hkv, D, n_pages, n_seq, max_blocks)) return e;
  MLORA_CHECK(out && qkv && k_cache && v_cache && block_table && tok_seq && tok_pos, MLORA_ERR_INVALID, "paged_attn_prefill: null pointer");
  MLORA_CHECK(T >= 0 && ceil_div(T, PF_WAVES * 16 * PF_QT) <= 65535, MLORA_ERR_INVALID, "paged_attn_prefill: bad T=%d", T);
  MLORA_CHECK(out_layout == MLORA_ROWMAJOR || out_layout == MLORA_FRAG, MLORA_ERR_INVALID, "paged_attn_prefill: bad out_layout %d", out_layout);
  if (T == 0) return MLORA_OK;
  const int frag_tt = out_layout == MLORA_FRAG ? mlora_frag_tiles(T) : 0;
  const float scale = 1.f / sqrtf((float)D);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(Hq, ceil_div(T, PF_WAVES * 16 * PF_QT));
#define MLORA_PREFILL(DD)                                                                                                          \
  do {                                                                                                                             \
    constexpr size_t lds = (size_t)PF_RING * 2 * PF_PAGES * PAGE * DD * sizeof(f16);                                                    \
    /* the attribute is per kernel, set once per process; a local static is initialised by one thread */                           \
    static const hipError_t configured =                                                                                           \
        hipFuncSetAttribute((const void*)paged_attn_prefill_block_kernel<DD>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
    if (configured != hipSuccess)                                                                                                  \
      return mlora_set_error(MLORA_ERR_LAUNCH, "paged_attn_prefill: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(configured)); \
    hipLaunchKernelGGL(paged_attn_prefill_block_kernel<DD>, grid, dim3(PF_WAVES * WAVE), lds, s, (f16*)out, frag_tt, (const f16*)qkv, \
                       (const f16*)k_cache, (const f16*)v_cache, block_table, max_blocks, tok_seq, tok_pos, T, Hq, Hkv, n_pages, n_seq, scale); \
  } while (0)
  if (D == 128) MLORA_PREFILL(128);
  else MLORA_PREFILL(64);
#undef MLORA_PREFILL
  return mlora_launch_status("paged_attn_prefill");
}
