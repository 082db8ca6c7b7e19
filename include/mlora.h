/*
 * mlora.h - C ABI of the MI355X (gfx950) multi-LoRA decode/prefill hot path.
 *
 * The reference (llm-db/tensor-program-optimization-with-auto-batching) is pure Python and exposes no
 * FFI; its per-layer operators are TVM Relax ops lowered to generated GPU kernels, or torch modules.
 * Each entry point below replaces one of those operators and cites it.  A Python host (torch tensors
 * for device memory and streams) binds this library with ctypes.
 *
 * Conventions
 *   - every pointer is a caller-owned DEVICE pointer unless named host_*; nothing here allocates
 *     device memory; work is enqueued on `stream` (a hipStream_t passed as void*; NULL = default
 *     stream) and the call returns without synchronising;
 *   - fp16 tensors are IEEE binary16, row-major, innermost dimension contiguous;
 *   - return value 0 = success, negative = MLORA_ERR_*; mlora_last_error() gives the message of the
 *     last failure on the calling thread;
 *   - shapes are validated on the host before any launch; a rejected call launches nothing.
 *
 * Two tiers of entry points
 *   PUBLIC, one per reference operator - what a binding of the reference needs and what stays stable:
 *     mlora_gather_mm (+ _workspace_bytes, _static, _multi, _multi_proj, _batch), mlora_lora_shrink / _expand,
 *     mlora_write_tensor_part, mlora_linear / mlora_linear_packed / mlora_linear_frag (and the gemv / gemm kernels
 *     they dispatch to), mlora_pack_weight, mlora_pack_activation, mlora_rmsnorm, mlora_silu_mul, mlora_embed,
 *     mlora_argmax, mlora_rope_kv_append, mlora_paged_attn_decode, mlora_paged_attn_prefill, and
 *     mlora_decode_step (one whole decode step from a plan); for prefill passes whose tokens come in adapter
 *     segments, mlora_linear_frag_lora and mlora_linear_frag_silu (linear, LoRA delta and - for gate / up - the
 *     SiLU product in one GEMM).
 *   INTERNAL, the fused forms from "Decode-step variants" down to mlora_rmsnorm_ksplit - the building blocks of
 *     mlora_decode_step, exported so that the Python host can run the same step operator by operator (the parity
 *     tests compare the two bit for bit).  Their argument lists follow the tiling of the kernels (K-range block
 *     counts, appended weight rows, partial buffers) and may change with it; a binding should call
 *     mlora_decode_step instead.
 */
#ifndef MLORA_H
#define MLORA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLORA_OK                 0
#define MLORA_ERR_INVALID       -1   /* bad shape / argument */
#define MLORA_ERR_UNSUPPORTED   -2   /* shape outside what the kernels cover */
#define MLORA_ERR_WORKSPACE     -3   /* workspace missing or too small */
#define MLORA_ERR_LAUNCH        -4   /* HIP reported a launch error */

#define MLORA_F16 0
#define MLORA_F32 1

/* y = acc, or y += acc, in the epilogue of the linear kernels */
#define MLORA_STORE       0
#define MLORA_ACCUMULATE  1

/* Activation layouts.  MLORA_ROWMAJOR: x[T, K], innermost contiguous.  MLORA_FRAG: the order in which the
 * matrix cores consume a token block,
 *     Xf[k/32][t/16][(k%32)/8][t%16][k%8]     with TT sixteen-token tiles per 32-k step: TT = 1, 2 or 4 for
 *                                             T <= 16, 32, 64 and ceil(T / 16) beyond,
 * so that the 16-token x 32-k operand fragment is one contiguous 1 KiB block; mlora_frag_activation_elems
 * gives the buffer size.  Producers (RMSNorm, SiLU*mul, attention) can write it directly; the decode GEMV, the
 * persistent prefill GEMM (mlora_linear_frag) and the LoRA shrink read it.  Rows t >= T of the last tile hold
 * whatever the buffer held: they reach only outputs that are never stored. */
#define MLORA_ROWMAJOR 0
#define MLORA_FRAG     1

#define MLORA_PAGE_SIZE 16   /* tokens per KV page; the only page size the kernels accept */

int mlora_version(void);
const char* mlora_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * Adapter-indexed LoRA delta ("gather-matmul"):
 *     y[t, :] += scaling * B[id_t] . (A[id_t] . x[t, :])      for every t with 0 <= id_t < n_ad
 * fp16 operands, fp32 accumulation; rows with id_t outside [0, n_ad) are left untouched.
 *
 * Replaces: GatherBMMLinear.forward hot branch (huggingface/custom_peft/lora_gatherbmm_linear_layer.py:14-20:
 *   stack of per-request A / scaled B, two bmm, add to the base result); the TVM adapter forward
 *   take -> matmul -> matmul -> *scaling (tvm/llama_auto_batcher/compile_tvm.py:106-112) with its fused
 *   take_matmul kernel (tvm/custom/fuse_take_matmul.py:85-105); and, because rows are addressed by
 *   token, the row gather/scatter around it in the mixed path (compile_tvm.py:147-153,
 *   tvm/custom/write_tensor_part.py:3-20).
 *
 * Layouts (PEFT orientation): x [T, K] f16 (x_layout: row-major, or fragment order when T <= 64);
 *   A [n_ad, r, K] f16; B [n_ad, N, r] f16;
 *   y [T, N] f16 or f32 (y_dtype) with row stride ldy elements (y may be a column slice of a fused
 *   projection output); tok_adapter [T] int32.
 * Constraints: r in {8, 16, 32, 64}; K % 8 == 0; N % 8 == 0; ldy >= N, ldy % 8 == 0.
 * workspace: mlora_gather_mm_workspace_bytes(T, K, r) bytes of device scratch (shrink partials);
 *   contents need not be initialised.
 * ------------------------------------------------------------------------------------------- */
size_t mlora_gather_mm_workspace_bytes(int T, int K, int r);
int mlora_gather_mm(void* y, int y_dtype, int ldy, const void* x, int x_layout, const void* A, const void* B,
                    const int32_t* tok_adapter, float scaling,
                    int T, int K, int N, int r, int n_ad,
                    void* workspace, size_t workspace_bytes, void* stream);
/* mlora_gather_mm for callers that cannot allocate and have no workspace to hand over (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference: its tensors all come from
 * the Python caller.  Same arguments, semantics and result bits as mlora_gather_mm, minus the workspace: the scratch
 * the kernels need (shrink results of batches above 64 tokens) lives in a buffer built into the library,
 * MLORA_GATHER_MM_STATIC_BYTES per GPU, held until the process ends.  The call allocates nothing.  Shapes with
 * mlora_gather_mm_workspace_bytes(T, K, r) above that size are rejected with MLORA_ERR_WORKSPACE.  Every call on a
 * GPU shares that GPU's buffer: calls that overlap in time on one GPU (two streams, two threads) race; the buffer's
 * contents are never read before they are written within a call, so nothing needs clearing between calls. */
#define MLORA_GATHER_MM_STATIC_BYTES (8u << 20)
size_t mlora_gather_mm_static_max_bytes(void);
int mlora_gather_mm_static(void* y, int y_dtype, int ldy, const void* x, int x_layout, const void* A, const void* B,
                           const int32_t* tok_adapter, float scaling,
                           int T, int K, int N, int r, int n_ad, void* stream);
/* Several independent gather-matmul problems of one shape and one token->adapter table in ONE launch (decode
 * shapes: T <= 64 and (K-slices + 1) * T * r * 4 <= 48 KiB of LDS, else MLORA_ERR_UNSUPPORTED).
 * sets: DEVICE array of n_sets records of four pointers {y, x, A, B}, laid out as above.  This is how a decode step
 * meets the op: every layer and projection has its own A / B / x / y, and the ~2 us of work per problem is far below
 * the cost of a launch.  Same result bits as n_sets calls of mlora_gather_mm.  Replaces the same reference code.
 * workspace: NULL, or n_sets * mlora_gather_mm_workspace_bytes(T, K, r) bytes of device scratch.  With a workspace and
 * eight or more sets the call runs as two streaming passes over all sets (a shrink launch that leaves its fp32
 * partials in the workspace, then an expand launch): no request of either pass waits on more than the table row, which
 * is what lets a many-problem call run at HBM bandwidth; without a workspace, or for fewer sets, one launch whose
 * workgroups shrink into LDS and expand from there.  Same result bits either way. */
/* Adapters of several ranks in one batch.  Bucket b holds the adapters of one rank and scaling,
 *   A [n_ad, r, K], B [n_ad, N, r]; token t uses adapter tok_adapter[t] of bucket tok_bucket[t]; a token whose
 *   bucket is outside [0, n_buckets) or whose adapter id is outside [0, n_ad) of its bucket is left untouched.
 * Every table is read at its own rank: nothing is padded to the largest rank and no rank is split into chunks, and
 * rows are addressed by token, so there is no gather of x rows nor scatter of results.  Same result bits as one
 * mlora_gather_mm call per bucket with the other buckets' tokens masked to -1.  workspace: the largest
 * mlora_gather_mm_workspace_bytes(T, K, r) over the buckets.  A decode-sized batch (T <= 64) with at most four
 * buckets is ONE launch: the kernel is built for the largest rank and a workgroup (one adapter) runs at its own
 * bucket's rank; otherwise one launch sequence per bucket, ordered on `stream`.
 * All buckets are validated before the first launch.  `buckets` is a HOST array; a bucket with A == B == NULL is
 * skipped (its adapters do not target this projection) and its tokens are left untouched.
 *
 * Replaces: the per-type loop of the mixed decode (tvm/llama_auto_batcher/compile_tvm.py:135-155: take rows, delta,
 * write_tensor_part scatter, add) and the padded / splitted / sequential multi-rank strategies of the case study
 * (tvm/lora_only/case_study/multiple_ranks.py:21-151), which all compute this sum. */
typedef struct mlora_lora_bucket {
  const void* A;
  const void* B;
  int r;
  int n_ad;
  float scaling;
} mlora_lora_bucket;
int mlora_gather_mm_multi(void* y, int y_dtype, int ldy, const void* x, int x_layout,
                          const mlora_lora_bucket* buckets, int n_buckets,
                          const int32_t* tok_bucket, const int32_t* tok_adapter,
                          int T, int K, int N, void* workspace, size_t workspace_bytes, void* stream);
/* The same for n_proj projections that read the same x and write disjoint column ranges of one y (q, k, v inside the
 * fused qkv row; gate and up): projection p adds to columns col_offset[p] .. col_offset[p] + n_cols[p] - 1 of y
 * (col_offset[p] % 8 == 0) with the tables buckets[p * n_buckets + b] (B [n_ad, n_cols[p], r]).  A decode-sized batch
 * with at most eight non-null (projection, bucket) entries is ONE launch.  Larger batches: per bucket, up to three
 * projections that carry it with the same rank, table size and scaling share one shrink and one expand launch on the
 * matrix cores, provided the workspace holds one slice of mlora_gather_mm_workspace_bytes(T, K, r) per projection
 * (otherwise, and for everything else, one mlora_gather_mm per projection and bucket).  Same result bits as one
 * mlora_gather_mm_multi call per projection.  buckets, col_offset and n_cols are HOST arrays.
 * Replaces: q_ft_proj + v_ft_proj of the patched attention forward, one take-matmul pair each
 * (tvm/llama_auto_batcher/compile_tvm.py:126-155). */
int mlora_gather_mm_multi_proj(void* y, int y_dtype, int ldy, const void* x, int x_layout,
                               const mlora_lora_bucket* buckets, int n_buckets, int n_proj,
                               const int32_t* col_offset, const int32_t* n_cols,
                               const int32_t* tok_bucket, const int32_t* tok_adapter,
                               int T, int K, void* workspace, size_t workspace_bytes, void* stream);
int mlora_gather_mm_batch(const void* const* sets, int n_sets, int y_dtype, int ldy, int x_layout,
                          const int32_t* tok_adapter, float scaling,
                          int T, int K, int N, int r, int n_ad,
                          void* workspace, size_t workspace_bytes, void* stream);

/* The two halves of the above, for callers that fuse differently:
 *   shrink: v_part[c, t, :] = A[id_t][:, chunk c] . x[t, chunk c]   (fp32 partials per K-chunk)
 *   expand: y[t, :] += scaling * B[id_t] . sum_c v_part[c, t, :]
 * Same layouts and constraints; v_part is the workspace described above. */
int mlora_lora_shrink(void* v_part, const void* x, int x_layout, const void* A, const int32_t* tok_adapter,
                      int T, int K, int r, int n_ad, void* stream);
int mlora_lora_expand(void* y, int y_dtype, int ldy, const void* v_part, const void* B, const int32_t* tok_adapter,
                      float scaling, int T, int K, int N, int r, int n_ad, void* stream);

/* Z = X; Z[ids[a], :] = Y[a, :]  - row scatter of the mixed-adapter-type path.
 * Replaces: write_tensor_part (tvm/custom/write_tensor_part.py:3-20).  X, Z [B, PH] f16, Y [A, PH] f16,
 * ids [A] int32 (rows with ids outside [0, B) are skipped).  Z may alias X. */
int mlora_write_tensor_part(void* Z, const void* X, const void* Y, const int32_t* ids,
                            int B, int A, int PH, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Base linear  y[T, N] (=|+=) x[T, K] . W[N, K]^T   (bias-free), fp16 operands, fp32 accumulation.
 * Replaces: nn.Linear(bias=False) of the q/k/v/o, gate/up/down projections and lm_head
 *   (tvm/llama_auto_batcher/llama_for_causal_lm.py:31-33,44-47,105), including the fp32 cast of the
 *   logits (:124-128) when y_dtype = MLORA_F32, and the residual add (:80-83) when mode =
 *   MLORA_ACCUMULATE with an fp32 y.
 *
 * mlora_gemv: weight-streaming kernel for T <= 64 (decode).   mlora_gemm: MFMA-tiled kernel for any T.
 * mlora_linear picks between them.  x row stride ldx (elements) lets x be a column slice.
 * Constraints: K % 32 == 0, N % 4 == 0, ldx % 8 == 0; MLORA_ACCUMULATE needs y_dtype = MLORA_F32.
 * ------------------------------------------------------------------------------------------- */
int mlora_gemv(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W,
               int T, int K, int N, void* stream);
int mlora_gemm(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W,
               int T, int K, int N, void* stream);
int mlora_linear(void* y, int y_dtype, int mode, const void* x, int ldx, const void* W,
                 int T, int K, int N, void* stream);

/* Fragment-ordered weight layout for the same linears.  The reference re-lays out weights once at load
 * time as well (stack + transpose, tvm/llama_auto_batcher/compile_tvm.py:296-314); here the one-time step
 * stores W in the order the matrix cores consume it,
 *     Wp[n/16][k/32][(k%32)/8][n%16][k%8]      (rows padded with zeros to a multiple of 16)
 * so every (16 rows x 32 k) operand fragment is one contiguous 1 KiB block and a wave streams
 * consecutive blocks.  mlora_pack_weight writes mlora_packed_weight_elems(N, K) fp16 elements to dst
 * (dst must not alias src).  The *_packed entry points take Wp in place of W; everything else is as
 * for mlora_gemv / mlora_gemm / mlora_linear. */
size_t mlora_packed_weight_elems(int N, int K);
int mlora_pack_weight(void* dst, const void* src, int N, int K, void* stream);
int mlora_gemv_packed(void* y, int y_dtype, int mode, const void* x, int ldx, const void* Wp,
                      int T, int K, int N, void* stream);
int mlora_gemm_packed(void* y, int y_dtype, int mode, const void* x, int ldx, const void* Wp,
                      int T, int K, int N, void* stream);
int mlora_linear_packed(void* y, int y_dtype, int mode, const void* x, int ldx, const void* Wp,
                        int T, int K, int N, void* stream);

/* Linear with both operands in fragment order: Wp as above, xf in MLORA_FRAG layout.  Every operand load of
 * the kernel is then a contiguous 1 KiB block.  mlora_pack_activation converts a row-major x (row stride ldsrc)
 * into fragment order for callers whose producer cannot write it directly.
 * mlora_gemv_frag: the decode GEMV, T <= 64.  mlora_linear_frag: any T - the GEMV up to 64 tokens, beyond that
 * the persistent matrix-core GEMM (needs K % 64 == 0), which copies both operands from global memory straight
 * into LDS.  mlora_gemm_frag_preferred says whether that GEMM is the efficient choice for a shape (at least
 * one 256 x 256 output block per compute unit); callers use it to decide which layout their producers write.
 * Replaces, like the other linears: nn.Linear(bias=False) (llama_for_causal_lm.py:26-38,58-62). */
size_t mlora_frag_activation_elems(int T, int K);
int mlora_pack_activation(void* dst, const void* src, int ldsrc, int T, int K, void* stream);
int mlora_gemv_frag(void* y, int y_dtype, int mode, const void* xf, const void* Wp,
                    int T, int K, int N, void* stream);
int mlora_linear_frag(void* y, int y_dtype, int mode, const void* xf, const void* Wp,
                      int T, int K, int N, void* stream);
int mlora_gemm_frag_preferred(int T, int K, int N);

/* The prefill linear that carries its LoRA deltas as extra k-steps of the base GEMM, for token blocks that agree on
 * one adapter: y (=|+=) [xf | v_hi | v_lo] . [Wp | B[a] | B[a]]^T per 256-token block whose tokens all name adapter a,
 * with v = scaling * x . A[a]^T split into fp16 hi + lo halves - no second pass over y.
 *   mlora_lora_block_adapters - blk_adapter[b] = the adapter all valid tokens of block b (256 tokens) name, or -1
 *                               (no adapter, or several); tok_rest[t] = -1 where the block's delta rides in the GEMM,
 *                               else tok_adapter[t]: the ids a separate mlora_gather_mm still has to serve;
 *   mlora_lora_shrink_split   - the matrix-core shrink of n_proj <= 3 projections that read the same x, then
 *                               v_hi[p], v_lo[p] [T][r] fp16 (r in {32, 64}); workspace: n_proj *
 *                               mlora_gather_mm_workspace_bytes(T, K, r) bytes; rows of tokens without adapter
 *                               (id outside [0, n_ad)) are zero, so such a token gets a zero delta;
 *   mlora_linear_frag_lora    - mlora_linear_frag on a shape that mlora_gemm_frag_preferred accepts, with up to three
 *                               projections = row ranges [n_begin, n_begin + n_rows) of the fused weight (on 256-row
 *                               boundaries), each with its B table [n_ad][n_rows][r] and its v halves.
 * Against mlora_linear_frag followed by mlora_gather_mm the result differs in where it is rounded (once, after the
 * sum, instead of after the base product and again after the delta) and in the fp32 summation order.
 * Replaces: the base linear plus q_ft_proj / v_ft_proj style deltas of the prefill entry points
 * (tvm/llama_auto_batcher/compile_tvm.py:116-160). */
typedef struct mlora_fused_lora {
  const void* B;      /* [n_ad][n_rows][r] fp16, row-major */
  const void* v_hi;   /* [T][r] fp16 */
  const void* v_lo;
  int n_begin;
  int n_rows;
} mlora_fused_lora;
int mlora_lora_block_adapters(int32_t* blk_adapter, int32_t* tok_rest, const int32_t* tok_adapter, int T, int n_ad,
                              void* stream);
int mlora_lora_shrink_split(void* const* v_hi, void* const* v_lo, const void* x, int x_layout, const void* const* A, int n_proj,
                            const int32_t* tok_adapter, float scaling, int T, int K, int r, int n_ad,
                            void* workspace, size_t workspace_bytes, void* stream);
int mlora_linear_frag_lora(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N,
                           const mlora_fused_lora* projs, int n_proj, const int32_t* blk_adapter, int r, void* stream);

/* Gate/up projection of a prefill-sized token block with the SiLU product in the epilogue of the persistent GEMM:
 *   act = f16( silu(f16(gate)) * f16(up) ),  [gate | up] = xf . Wp^T (+ the LoRA deltas as in mlora_linear_frag_lora),
 * written in MLORA_FRAG order for the down projection; the [T, 2I] projection output never reaches memory.
 * Wp is the fragment-ordered fused [2I, K] matrix (gate rows, then up rows) that mlora_linear_frag takes - no second
 * copy; I % 32 == 0 and mlora_gemm_frag_preferred(T, K, 2I).  n_proj = 0: no adapters (projs, blk_adapter may be NULL).
 * Otherwise projs names the gate projection (n_begin = 0), the up projection (n_begin = I) or both (n_rows = I each),
 * and every token of a 256-token block must name the block's adapter blk_adapter[b] or none: a block that mixes
 * adapters needs its deltas before the SiLU and has to take mlora_linear_frag_lora, mlora_gather_mm and
 * mlora_silu_mul instead.  Same result bits as those calls in sequence.
 * Replaces: gate_proj, up_proj, op.silu and the multiply (llama_for_causal_lm.py:35-36) with the LoRA of
 * lora.py:26-30 on either projection, in one launch. */
int mlora_linear_frag_silu(void* act, const void* xf, const void* Wp, int T, int K, int I,
                           const mlora_fused_lora* projs, int n_proj, const int32_t* blk_adapter, int r, void* stream);

/* y[t, :] = f16( x[t, :] * rsqrt(mean(x[t, :]^2) + eps) * w )   row-wise, statistics in fp32.
 * Replaces: nn.RMSNorm(hidden, -1, eps, bias=False) (llama_for_causal_lm.py:76-77,93).
 * x [T, H] f16 or f32 (x_dtype), w [H] f16, y [T, H] f16 in y_layout.  H % 8 == 0, H <= 16384. */
int mlora_rmsnorm(void* y, int y_layout, const void* x, int x_dtype, const void* w, float eps, int T, int H,
                  void* stream);

/* out[t, i] = f16( silu(gate[t, i]) * up[t, i] );  gate and up are column slices with row stride ld
 * (elements) so a fused [T, 2I] projection output can be passed as (p, p + I, 2I).
 * Replaces: op.silu(gate_proj(x)) * up_proj(x) (llama_for_causal_lm.py:35-36).  I % 8 == 0. */
int mlora_silu_mul(void* out, int out_layout, const void* gate, const void* up, int ld, int T, int I, void* stream);

/* out[t, :] = table[ids[t], :] widened to out_dtype.  Replaces: nn.Embedding lookup
 * (llama_for_causal_lm.py:121-122).  table [V, H] f16; ids outside [0, V) produce a zero row. */
int mlora_embed(void* out, int out_dtype, const void* table, const int32_t* ids, int T, int H, int V, void* stream);

/* ids[b] = argmax_v logits[b, v], lowest index on ties (numpy.argmax).
 * Replaces: the host-side np.argmax over D2H-copied logits (tvm/llama_auto_batcher/llama_exec_graph.py:92,134-137). */
int mlora_argmax(int32_t* ids, const float* logits, int B, int V, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Paged KV cache (16-token pages) - replaces TVM's TIRPagedKVCache as configured at
 * llama_for_causal_lm.py:148-174 (RoPE applied inside the cache op, rotary_dim = head_dim, scale 1,
 * no sliding window) and driven by kv_state_begin_forward / attention_with_fused_qkv / end_forward
 * (tvm/llama_auto_batcher/llama_exec_graph.py:75-85,121-127; llama_for_causal_lm.py:55-64).
 *
 * Layouts, per layer:
 *   k_cache [n_pages, Hkv, D/32, 4, 16, 8] f16 - rotated keys; a 16-token page of one head is contiguous and
 *       in matrix-core fragment order: element (token, d) at ((d/32 * 4 + (d%32)/8) * 16 + token) * 8 + d%8
 *   v_cache [n_pages, Hkv, D, 16] f16   - values, token-minor inside a page
 *   block_table [n_seq, max_blocks] int32 - physical page of logical block j of sequence s
 *   qkv [T, Hq + 2 Hkv, D] f16 - fused projection output, token-major
 *   rope_cos / rope_sin [max_pos, D/2] f32 - tables; element i pairs with element i + D/2
 *
 * mlora_rope_kv_append: for token t (sequence tok_seq[t], position tok_pos[t]) rotate the q heads in
 *   place inside qkv, rotate k and write k, v into the page slot of that position.
 * mlora_paged_attn_decode: one query per sequence; out[b, h, :] = softmax(q . K^T / sqrt(D)) V over the
 *   first ctx_len[b] cached positions of sequence seq_ids[b] (the new token already appended).
 * mlora_paged_attn_prefill: query token t (sequence tok_seq[t], position tok_pos[t]) attends to cached
 *   positions 0..tok_pos[t]; tokens of a sequence must be consecutive in t with increasing positions.
 * The attention kernels multiply whole pages and mask afterwards: every slot of a page that a block table names
 * must hold finite numbers before its first use, or P = 0 times a non-finite V turns the output into NaN.  The
 * prefill kernel also reads PAGE 0 in place of every page slot past a sequence's end (and of a page id outside
 * [0, n_pages)), again with P = 0: page 0 must hold finite numbers whether or not a block table names it.
 * Allocating the whole cache zero-filled satisfies both.
 * q is read from qkv (already rotated).  out [T, Hq * D] f16 in out_layout.  D in {64, 128};
 * Hq % Hkv == 0, Hq / Hkv <= 16 and B <= 65535 for decode.
 * ------------------------------------------------------------------------------------------- */
int mlora_rope_kv_append(void* qkv, void* k_cache, void* v_cache,
                         const int32_t* block_table, int max_blocks,
                         const int32_t* tok_seq, const int32_t* tok_pos,
                         const float* rope_cos, const float* rope_sin, int max_pos,
                         int T, int Hq, int Hkv, int D, int n_pages, int n_seq, void* stream);
int mlora_paged_attn_decode(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                            const int32_t* block_table, int max_blocks,
                            const int32_t* seq_ids, const int32_t* ctx_len,
                            int B, int Hq, int Hkv, int D, int n_pages, int n_seq, void* stream);
int mlora_paged_attn_prefill(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                             const int32_t* block_table, int max_blocks,
                             const int32_t* tok_seq, const int32_t* tok_pos,
                             int T, int Hq, int Hkv, int D, int n_pages, int n_seq, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Decode-step variants that carry the LoRA work of a projection inside a neighbouring launch, so that the
 * adapter delta adds no launches of its own (results are bit-identical to the separate calls):
 *   mlora_gemv_frag_lora      - mlora_gemv_frag, plus the shrink partials of n_proj <= 3 projections that read
 *                               the same xf (A[p] [n_ad, r, K], a NULL slot is skipped); v_part is [n_proj][kc][T][r] fp32,
 *                               n_proj * mlora_gather_mm_workspace_bytes(T, K, r) bytes;
 *   mlora_gemv_frag_split     - mlora_gemv_frag over a weight that has N_ext extra rows appended after its N_main
 *                               rows: the stacked A tables of all adapters ([n_ad * r, K] per adapted projection,
 *                               packed together with W).  Rows < N_main go to y as usual, the extra rows to
 *                               y2 [T, N_ext] fp32: the shrink of every (token, adapter) pair, for the cost of the
 *                               A bytes alone and with no dependence on the token->adapter table;
 *   mlora_rope_kv_append_lora - mlora_rope_kv_append, after adding scaling * B[p][id_t] . v to the q, k, v
 *                               rows of qkv (B[p] [n_ad, N_p, r] or NULL).  v_dense = 0: v_part holds the K-slice
 *                               partials written by mlora_gemv_frag_lora with this K; v_dense = kq >= 1: v_part is
 *                               y2 [kq][T, 3 * n_ad * r] of mlora_gemv_frag_split (kq = 1) or
 *                               mlora_gemv_frag_split_kq (slot p = projection p; the kq blocks are added in order);
 *                               v_dense must lie in 0..4 (the kernels keep at most four blocks), else MLORA_ERR_UNSUPPORTED.
 *                               (One argument for two facts - which form the shrink results have, and how many
 *                               blocks - because the ids-based form has no block count: 0 is not a count.)
 *   mlora_lora_expand_rmsnorm - resid[t, :] += scaling * B[id_t] . v (B [n_ad, H, r]; v_part [kc][T][r] partials
 *                               of a shrink over K inputs, or y2 [T, n_ad * r] when v_dense = 1), then
 *                               y = RMSNorm(resid) as mlora_rmsnorm.
 * These replace the same reference operators as mlora_gather_mm, mlora_rope_kv_append and mlora_rmsnorm.
 * ------------------------------------------------------------------------------------------- */
int mlora_gemv_frag_lora(void* y, int y_dtype, int mode, const void* xf, const void* Wp, int T, int K, int N,
                         void* v_part, const void* const* A, int n_proj, const int32_t* tok_adapter, int r, int n_ad,
                         void* stream);
/* Gate/up projection with the SiLU product in its epilogue:  act = silu(f16(x . Wgate^T)) * f16(x . Wup^T), written
 * in MLORA_FRAG order for the down projection (T <= 64).  Wil_p is the fragment-ordered [2I, K] matrix whose 16-row
 * tiles alternate gate and up (tile 2j = gate rows 16j.., tile 2j+1 = up rows 16j..), so one workgroup holds both
 * halves of a channel.  Replaces: gate_proj, up_proj, op.silu and the multiply (llama_for_causal_lm.py:35-36) in
 * one launch; same result bits as mlora_gemv_frag followed by mlora_silu_mul. */
int mlora_gemv_frag_silu(void* act, const void* xf, const void* Wil_p, int T, int K, int I, void* stream);
/* The split GEMV with f16 y as one workgroup per compute unit: the appended rows are cut into kq ranges of K and come
 * back as kq blocks of partial sums, y2 [kq][T][N_ext] fp32, which the reader adds in block order (pass kq as v_dense
 * to mlora_rope_attn_decode / mlora_rope_kv_append_lora).  mlora_gemv_split_kq names kq for a shape (1: the form does
 * not apply; mlora_gemv_frag_split_kq with kq == 1 is mlora_gemv_frag_split).  No counterpart in the reference beyond
 * the linear itself (llama_for_causal_lm.py:44-47). */
int mlora_gemv_split_kq(int T, int K, int N_main, int N_ext);
int mlora_gemv_frag_split_kq(void* y, float* y2, int kq, const void* xf, const void* Wp, int T, int K, int N_main,
                             int N_ext, void* stream);
int mlora_gemv_frag_split(void* y, int y_dtype, int mode, float* y2, const void* xf, const void* Wp,
                          int T, int K, int N_main, int N_ext, void* stream);
int mlora_rope_kv_append_lora(void* qkv, void* k_cache, void* v_cache,
                              const int32_t* block_table, int max_blocks,
                              const int32_t* tok_seq, const int32_t* tok_pos,
                              const float* rope_cos, const float* rope_sin, int max_pos,
                              int T, int Hq, int Hkv, int D, int n_pages, int n_seq,
                              const void* v_part, int v_dense, const void* const* B, const int32_t* tok_adapter,
                              float scaling, int K, int r, int n_ad, void* stream);
/* RoPE + cache append + decode attention (+ the LoRA expand of q, k, v) in ONE launch, for a decode step in which
 * row b of qkv is the new token of sequence seq_ids[b] at position tok_pos[b] and ctx_len[b] = tok_pos[b] + 1.
 * Results equal mlora_rope_kv_append[_lora] followed by mlora_paged_attn_decode bit for bit (out and both caches),
 * except that the q rows of qkv are left unrotated.  v_part == NULL: no LoRA (B, tok_adapter ignored); otherwise
 * the LoRA arguments are those of mlora_rope_kv_append_lora.  Replaces: attention_with_fused_qkv
 * (tvm/llama_auto_batcher/llama_for_causal_lm.py:55-64) for the decode entry points, with the q/v adapter deltas of
 * compile_tvm.py:126-134 applied inside. */
int mlora_rope_attn_decode(void* out, int out_layout, const void* qkv, void* k_cache, void* v_cache,
                           const int32_t* block_table, int max_blocks,
                           const int32_t* seq_ids, const int32_t* tok_pos, const int32_t* ctx_len,
                           const float* rope_cos, const float* rope_sin, int max_pos,
                           int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                           const void* v_part, int v_dense, const void* const* Bmat, const int32_t* tok_adapter,
                           float scaling, int K, int r, int n_ad, void* stream);
/* The same launch, which in addition takes the o projection's LoRA shrink off the attention output where it is
 * produced: o_vpart[h][b][j] = sum over the D dims of head h of f16(out[b, h, d]) * o_A[id_b][j][h D + d]  (fp32,
 * [Hq][B][r]; o_A [n_ad, r, Hq * D]; rows of tokens without adapter are left untouched), one share per query head,
 * for a consumer that adds the Hq shares in a fixed order (mlora_gemv_frag_acc_ksplit_delta).  out and the caches are
 * those of mlora_rope_attn_decode bit for bit.  tok_adapter, r and n_ad serve both the q/k/v expand (if v_part is
 * given) and the o shrink.  mlora_rope_attn_oshrink_ok says whether the launch for (B, Hq, Hkv, D) has room for
 * rank r (its Hq / Hkv * r * D / 8 items must fit one workgroup).  Replaces: the lora_A half of the o projection's
 * injected forward (tvm/llama_auto_batcher/lora.py:16-24, compile_tvm.py:126-134). */
int mlora_rope_attn_oshrink_ok(int B, int Hq, int Hkv, int D, int r);
int mlora_rope_attn_decode_oshrink(void* out, int out_layout, const void* qkv, void* k_cache, void* v_cache,
                                   const int32_t* block_table, int max_blocks,
                                   const int32_t* seq_ids, const int32_t* tok_pos, const int32_t* ctx_len,
                                   const float* rope_cos, const float* rope_sin, int max_pos,
                                   int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                   const void* v_part, int v_dense, const void* const* Bmat, const int32_t* tok_adapter,
                                   float scaling, int K, int r, int n_ad, const void* o_A, void* o_vpart, void* stream);
/* The decode attention without the RoPE / append part (mlora_paged_attn_decode: out bit for bit) that also writes the
 * o projection's shrink in head shares, as mlora_rope_attn_decode_oshrink does (same o_A, o_vpart, tok_adapter, r, n_ad;
 * mlora_rope_attn_oshrink_ok applies), and the expand of such shares as a launch of its own:
 *   y[t, :] += scaling * B[id_t] . sum_h vpart[h][t]   for the tokens that name an adapter (y fp32 [T, N], B [n_ad, N, r];
 *   mlora_lora_expand_shares_ok(N, r): N % 16 == 0, rank 8, 16, 32 or 64, N dividing over a token's workgroups).
 * Together they are the o projection's adapter delta of a decode step of more than 64 sequences (mlora_decode_step takes
 * them where both apply).  Replace: tvm/llama_auto_batcher/lora.py:16-24 for the o projection (compile_tvm.py:126-134). */
int mlora_paged_attn_decode_oshrink(void* out, int out_layout, const void* qkv, const void* k_cache, const void* v_cache,
                                    const int32_t* block_table, int max_blocks, const int32_t* seq_ids, const int32_t* ctx_len,
                                    int B, int Hq, int Hkv, int D, int n_pages, int n_seq,
                                    const int32_t* tok_adapter, int r, int n_ad, const void* o_A, void* o_vpart, void* stream);
int mlora_lora_expand_shares_ok(int N, int r);
int mlora_lora_expand_shares(float* y, const float* vpart, int n_vpart, const void* B, const int32_t* tok_adapter, float scaling,
                             int T, int N, int r, int n_ad, void* stream);
int mlora_lora_expand_rmsnorm(void* y, int y_layout, float* resid, const void* v_part, int v_dense, const void* B,
                              const int32_t* tok_adapter, float scaling, const void* w, float eps,
                              int T, int H, int K, int r, int n_ad, void* stream);

/* ---------------------------------------------------------------------------------------------
 * K split of the accumulating decode GEMV over a narrow weight (o_proj, down_proj: 256 row tiles give one
 * workgroup per compute unit only at one tile each, which makes every workgroup read the whole token block for 16
 * rows).  With a split, a workgroup takes four row tiles (two beyond 32 tokens) and 1/ks of K; slice 0 accumulates into y as usual and
 * slices 1..ks-1 store fp32 partial results that the next reader of y adds in slice order - in the decoder layer
 * that reader is always an RMSNorm, so the sum is formed there and no extra pass or atomics are needed
 * (results do not depend on scheduling).
 *   mlora_gemv_ksplit          - the number of slices (1..4) this library uses for (T, K, N_total); 1 = no split;
 *   mlora_gemv_shrink_rows     - what shrink units that ride in the launch (mlora_gemv_frag_acc_ksplit with A) add to
 *                                N_total in that rule: they occupy workgroups like rows do; a constant allowance
 *                                (0 without units), so that the slice count does not depend on the adapters of a batch;
 *   mlora_gemv_ksplit_bytes    - size of the partials buffer, part [ks-1][T][N_total] fp32;
 *   mlora_gemv_frag_acc_ksplit - y[T, N_main] (fp32) += xf . Wp^T over slice 0, partials of the other slices to
 *                                `part`.  N_ext > 0: appended rows as in mlora_gemv_frag_split (their slice-0 result
 *                                goes to y2 [T, N_ext], their partials to columns N_main.. of `part`).  A != NULL
 *                                (N_ext must be 0): shrink partials of n_proj projections as in
 *                                mlora_gemv_frag_lora.  ks = 1 needs no `part` and equals the unsplit calls.
 *   mlora_rmsnorm_ksplit       - resid[t, :] (+= LoRA expand as in mlora_lora_expand_rmsnorm when B != NULL)
 *                                += part[0][t, :H] + ... + part[ks-2][t, :H], stored back, then y = RMSNorm(resid).
 *                                ld_part = N_total of the GEMV that wrote `part`; with v_dense = 1 the shrink results
 *                                are y2 plus columns H.. of the partials.
 *   mlora_gemv_frag_acc_ksplit_delta - the same accumulating K-split GEMV over the base weight alone, with the
 *                                projection's LoRA expand done by workgroups that ride at the front of the launch.  The
 *                                shrink results come as n_vpart shares, vpart [n_vpart][T][r] fp32 (added in a fixed
 *                                order; mlora_rope_attn_decode_oshrink writes one share per attention head):
 *                                delta[t, :] = scaling * B[id_t] . sum_h vpart[h][t] (zeros for a token without adapter)
 *                                goes to slot ks-1 of `part` ([ks][T][N] fp32: ks-1 slice partials, then the delta
 *                                rows), so a reader that adds ks slots (mlora_rmsnorm_ksplit with ks + 1, no B) obtains
 *                                y + x . W^T + delta.  ks must be mlora_gemv_delta_ride_ksplit(T, K, N, r) (0: the shape
 *                                is not served; T <= 64, rank 8, 16, 32 or 64; at most 3, so that the reader adds at
 *                                most 3 slots).
 * These replace the same reference operators as mlora_gemv_frag (llama_for_causal_lm.py:31-33,44-47, the o_proj and
 * down_proj linears with the residual add of :79-84), mlora_rmsnorm (:76-77) and, for the delta form, the LoRA branch
 * of the injected linear forward (tvm/llama_auto_batcher/lora.py:16-24).
 * ------------------------------------------------------------------------------------------- */
int mlora_gemv_ksplit(int T, int K, int N_total);
int mlora_gemv_delta_ride_ksplit(int T, int K, int N, int r);
int mlora_gemv_frag_acc_ksplit_delta(float* y, float* part, int ks, const void* xf, const void* Wp, int T, int K, int N,
                                     const float* vpart, int n_vpart, const void* B, const int32_t* tok_adapter, float scaling,
                                     int r, int n_ad, void* stream);
int mlora_gemv_shrink_rows(int K, int n_proj, int n_ad);
size_t mlora_gemv_ksplit_bytes(int T, int N_total, int ks);
int mlora_gemv_frag_acc_ksplit(float* y, float* y2, float* part, int ks, const void* xf, const void* Wp,
                               int T, int K, int N_main, int N_ext,
                               void* v_part, const void* const* A, int n_proj, const int32_t* tok_adapter, int r, int n_ad,
                               void* stream);
int mlora_rmsnorm_ksplit(void* y, int y_layout, float* resid, const float* part, int ks, int ld_part,
                         const void* w, float eps, int T, int H,
                         const void* v_part, int v_dense, const void* B, const int32_t* tok_adapter, float scaling,
                         int K, int r, int n_ad, void* stream);

/* ---------------------------------------------------------------------------------------------
 * One decode step of the whole model, enqueued by one call.
 * Replaces: the body of the reference's hot loop between kv_state_begin_forward and the argmax
 *   (tvm/llama_auto_batcher/llama_exec_graph.py:110-137): vm["embed"], vm["decode_*"] over all layers
 *   (llama_for_causal_lm.py:79-84,95-100,121-128 with the patched attention of compile_tvm.py:116-160) and
 *   np.argmax.  The host keeps only the integer page bookkeeping (a new page per sequence every 16 steps).
 *
 * All pointers inside the structs are device pointers; the structs themselves and the `layers` array live in
 * host memory and are read during the call only.  Weights are fragment-ordered (mlora_pack_weight), q/k/v and
 * gate/up fused row-wise.  A LoRA projection with A == NULL is not adapted.  One adapter type (rank, scaling)
 * per call; tok_adapter[t] < 0 = no adapter for that sequence.
 * lora_dense != 0: qkv_p, o_p and down_p have the stacked A tables of their adapted projections appended as extra
 * rows (q, k, v slots in that order, n_ad * r rows each, zero rows for a slot that is not adapted), and the shrink
 * is part of the base GEMV; otherwise shrink units ride in the GEMV launch and read the A pointers.
 * lora_dense == 2: as 1, except that o_p is the base weight alone: the attention launch writes the o projection's
 * shrink as one share per head (mlora_rope_attn_decode_oshrink) and riders of the o GEMV launch expand it
 * (mlora_gemv_frag_acc_ksplit_delta).  Needs mlora_rope_attn_oshrink_ok(T, Hq, Hkv, D, r), ks =
 * mlora_gemv_delta_ride_ksplit(T, Hq*D, H, r) > 0, a ksplit_ws of ks slots of [T, H], and Hq * T * r floats in a
 * lora_ws slot.
 * Per step: tokens[t] (in) is embedded, attends at position pos[t] of sequence row rows[t] (ctx[t] = pos[t] + 1
 * positions visible), and tokens[t] (out) receives the greedy next token; pos and ctx are then incremented on the
 * device, so the call can be replayed from a captured graph without host work while no new page is needed.
 * Scratch buffers are caller-owned (sizes in elements):
 *   resid f32 [T*H]; xn, attn: mlora_frag_activation_elems(T, H | Hq*D) f16; qkv f16 [T*(Hq+2Hkv)*D];
 *   gate_up f16 [T*2I]; act: mlora_frag_activation_elems(T, I) f16; logits f32 [T*V];
 *   lora_ws: 5 slots of max(mlora_gather_mm_workspace_bytes(T, max(H, I, Hq*D), r), 4 * T * n_ad * r) bytes;
 *     with lora_dense, (3 * kq + 2) slots for kq = mlora_gemv_split_kq(T, H, (Hq+2Hkv)*D, 3 * n_ad * r) (at most 14).
 * ------------------------------------------------------------------------------------------- */
typedef struct mlora_lora_proj {
  const void* A;   /* [n_ad, r, K] f16 or NULL */
  const void* B;   /* [n_ad, N, r] f16 */
} mlora_lora_proj;

enum { MLORA_Q = 0, MLORA_K = 1, MLORA_V = 2, MLORA_O = 3, MLORA_GATE = 4, MLORA_UP = 5, MLORA_DOWN = 6 };

typedef struct mlora_layer {
  const void* qkv_p;
  const void* o_p;
  const void* gate_up_p;      /* [2I, K]: gate rows then up rows; may be NULL when gate_up_il_p is given and gate/up carry no LoRA */
  const void* gate_up_il_p;   /* the same matrix with 16-row tiles of gate and up interleaved (mlora_gemv_frag_silu), or NULL */
  const void* down_p;
  const void* ln1;
  const void* ln2;
  mlora_lora_proj lora[7];
  void* k_cache;
  void* v_cache;
} mlora_layer;

typedef struct mlora_decode_plan {
  int n_layers, hidden, inter, n_q_heads, n_kv_heads, head_dim, vocab;
  float eps;
  int lora_r, lora_n_ad;
  float lora_scaling;
  int lora_dense;
  const mlora_layer* layers;
  const void* embed;
  const void* norm;
  const void* lm_head_p;
  const float* rope_cos;
  const float* rope_sin;
  int max_pos;
  const int32_t* block_table;
  int max_blocks, n_pages, n_seq;
  int T;
  int32_t* tokens;
  const int32_t* rows;
  int32_t* pos;
  int32_t* ctx;
  const int32_t* tok_adapter;
  float* resid;
  void* xn;
  void* qkv;
  void* attn;
  void* gate_up;
  void* act;
  float* logits;
  void* lora_ws;
  size_t lora_ws_bytes;
  float* ksplit_ws;           /* partials of the K-split o_proj / down_proj GEMVs, or NULL (no split) */
  size_t ksplit_ws_bytes;     /* >= mlora_gemv_ksplit_bytes over both projections (with their appended rows) */
} mlora_decode_plan;

int mlora_decode_step(const mlora_decode_plan* plan, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MLORA_H */
