// One decode step of the whole model enqueued natively: the per-layer launch sequence of the decode hot
// loop without any host work between kernels, so the step can be captured into a graph and replayed.
#include "common.h"

namespace {

__global__ void advance_kernel(int32_t* __restrict__ pos, int32_t* __restrict__ ctx, int T) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < T) {
    pos[t] += 1;
    ctx[t] += 1;
  }
}

#define STEP(call)                   \
  do {                               \
    if (int e_ = (call)) return e_;  \
  } while (0)

// The step for more than 64 sequences: the same operator sequence with one launch per operator (the fused forms above
// are built around a token block that fits one wave).  Activations stay in fragment order, the linears run on the
// matrix-core kernel for mid-size token blocks, the two narrow accumulating ones split over K slices whose partials
// the next RMSNorm adds, and the adapter deltas are matrix-core gather-matmuls (q, k, v and gate, up grouped).
int decode_step_wide(const mlora_decode_plan* p, void* stream) {
  const int T = p->T, H = p->hidden, I = p->inter, Hq = p->n_q_heads, Hkv = p->n_kv_heads, D = p->head_dim;
  const int q_sz = Hq * D, kv_sz = Hkv * D, qkv_sz = q_sz + 2 * kv_sz;
  MLORA_CHECK(H % 32 == 0 && I % 32 == 0 && q_sz % 32 == 0, MLORA_ERR_UNSUPPORTED,
              "decode_step: more than 64 sequences need hidden, intermediate and q sizes that are multiples of 32");
  const bool lora = p->tok_adapter != nullptr && p->lora_r > 0;
  const int r = p->lora_r, n_ad = p->lora_n_ad;
  const float sc = p->lora_scaling;
  f16* qkv = (f16*)p->qkv;
  f16* gu = (f16*)p->gate_up;
  const int Kmax = H > I ? (H > q_sz ? H : q_sz) : (I > q_sz ? I : q_sz);
  MLORA_CHECK(!lora || (p->lora_ws && p->lora_ws_bytes >= 3 * mlora_gather_mm_workspace_bytes(T, Kmax, r)), MLORA_ERR_WORKSPACE,
              "decode_step: lora_ws of %zu bytes given, %zu needed", p->lora_ws_bytes, 3 * mlora_gather_mm_workspace_bytes(T, Kmax, r));
  // adapter deltas of the projections lp[0..n) that read x and write column ranges of y: two or more go out as one group
  auto deltas = [&](void* y, int y_dtype, int ldy, const void* x, int K, const mlora_lora_proj* const* lp, const int32_t* col,
                    const int32_t* ncol, int n) -> int {
    if (!lora) return MLORA_OK;
    mlora_lora_bucket bk[3];
    int32_t c[3], nc[3];
    int live = 0;
    for (int i = 0; i < n; ++i)
      if (lp[i]->A) {
        bk[live] = mlora_lora_bucket{lp[i]->A, lp[i]->B, r, n_ad, sc};
        c[live] = col[i];
        nc[live] = ncol[i];
        ++live;
      }
    if (live >= 2)
      return mlora_gather_mm_multi_proj(y, y_dtype, ldy, x, MLORA_FRAG, bk, 1, live, c, nc, nullptr, p->tok_adapter, T, K, p->lora_ws,
                                        p->lora_ws_bytes, stream);
    const size_t esz = y_dtype == MLORA_F16 ? 2 : 4;
    for (int i = 0; i < live; ++i)
      STEP(mlora_gather_mm((char*)y + (size_t)c[i] * esz, y_dtype, ldy, x, MLORA_FRAG, bk[i].A, bk[i].B, p->tok_adapter, sc, T, K, nc[i], r,
                           n_ad, p->lora_ws, p->lora_ws_bytes, stream));
    return MLORA_OK;
  };
  auto ksplit_of = [&](int K) -> int {
    const int ks = p->ksplit_ws ? mlora_gemv_ksplit(T, K, H) : 1;
    return ks > 1 && mlora_gemv_ksplit_bytes(T, H, ks) <= p->ksplit_ws_bytes ? ks : 1;
  };
  auto norm = [&](const void* w, int ks) -> int {
    if (ks > 1)
      return mlora_rmsnorm_ksplit(p->xn, MLORA_FRAG, p->resid, p->ksplit_ws, ks, H, w, p->eps, T, H, nullptr, 0, nullptr, nullptr, 0.f, 0,
                                  0, 0, stream);
    return mlora_rmsnorm(p->xn, MLORA_FRAG, p->resid, MLORA_F32, w, p->eps, T, H, stream);
  };
  // An adapted o projection: the attention launch leaves the shrink as one share per head, and a launch of expand
  // workgroups adds the deltas to the residual behind the base linear - instead of a shrink pass over the attention
  // output and an expand pass (where the shapes allow it; the per-operator Python path takes the same decision).
  const bool o_shares = lora && mlora_rope_attn_oshrink_ok(T, Hq, Hkv, D, r) && mlora_lora_expand_shares_ok(H, r) &&
                        p->lora_ws_bytes >= (size_t)Hq * T * r * sizeof(float);
  int pending_ks = 1;
  STEP(mlora_embed(p->resid, MLORA_F32, p->embed, p->tokens, T, H, p->vocab, stream));
  for (int l = 0; l < p->n_layers; ++l) {
    const mlora_layer& L = p->layers[l];
    STEP(norm(L.ln1, pending_ks));
    STEP(mlora_linear_frag(qkv, MLORA_F16, MLORA_STORE, p->xn, L.qkv_p, T, H, qkv_sz, stream));
    {
      const mlora_lora_proj* lp[3] = {&L.lora[MLORA_Q], &L.lora[MLORA_K], &L.lora[MLORA_V]};
      const int32_t col[3] = {0, q_sz, q_sz + kv_sz}, ncol[3] = {q_sz, kv_sz, kv_sz};
      STEP(deltas(qkv, MLORA_F16, qkv_sz, p->xn, H, lp, col, ncol, 3));
    }
    STEP(mlora_rope_kv_append(qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows, p->pos, p->rope_cos, p->rope_sin,
                              p->max_pos, T, Hq, Hkv, D, p->n_pages, p->n_seq, stream));
    const bool o_by_shares = o_shares && L.lora[MLORA_O].A;
    if (o_by_shares)
      STEP(mlora_paged_attn_decode_oshrink(p->attn, MLORA_FRAG, qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows, p->ctx,
                                           T, Hq, Hkv, D, p->n_pages, p->n_seq, p->tok_adapter, r, n_ad, L.lora[MLORA_O].A, p->lora_ws,
                                           stream));
    else
      STEP(mlora_paged_attn_decode(p->attn, MLORA_FRAG, qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows, p->ctx, T, Hq,
                                   Hkv, D, p->n_pages, p->n_seq, stream));
    const int ks_o = ksplit_of(q_sz);
    STEP(mlora_gemv_frag_acc_ksplit(p->resid, nullptr, p->ksplit_ws, ks_o, p->attn, L.o_p, T, q_sz, H, 0, nullptr, nullptr, 0, nullptr, 0, 0,
                                    stream));
    if (o_by_shares) {
      STEP(mlora_lora_expand_shares(p->resid, (const float*)p->lora_ws, Hq, L.lora[MLORA_O].B, p->tok_adapter, sc, T, H, r, n_ad, stream));
    } else {
      const mlora_lora_proj* lp[1] = {&L.lora[MLORA_O]};
      const int32_t col[1] = {0}, ncol[1] = {H};
      STEP(deltas(p->resid, MLORA_F32, H, p->attn, q_sz, lp, col, ncol, 1));
    }
    STEP(norm(L.ln2, ks_o));
    STEP(mlora_linear_frag(gu, MLORA_F16, MLORA_STORE, p->xn, L.gate_up_p, T, H, 2 * I, stream));
    {
      const mlora_lora_proj* lp[2] = {&L.lora[MLORA_GATE], &L.lora[MLORA_UP]};
      const int32_t col[2] = {0, I}, ncol[2] = {I, I};
      STEP(deltas(gu, MLORA_F16, 2 * I, p->xn, H, lp, col, ncol, 2));
    }
    STEP(mlora_silu_mul(p->act, MLORA_FRAG, gu, gu + I, 2 * I, T, I, stream));
    pending_ks = ksplit_of(I);
    STEP(mlora_gemv_frag_acc_ksplit(p->resid, nullptr, p->ksplit_ws, pending_ks, p->act, L.down_p, T, I, H, 0, nullptr, nullptr, 0, nullptr, 0,
                                    0, stream));
    {
      const mlora_lora_proj* lp[1] = {&L.lora[MLORA_DOWN]};
      const int32_t col[1] = {0}, ncol[1] = {H};
      STEP(deltas(p->resid, MLORA_F32, H, p->act, I, lp, col, ncol, 1));
    }
  }
  STEP(norm(p->norm, pending_ks));
  STEP(mlora_linear_frag(p->logits, MLORA_F32, MLORA_STORE, p->xn, p->lm_head_p, T, H, p->vocab, stream));
  STEP(mlora_argmax(p->tokens, p->logits, T, p->vocab, stream));
  hipLaunchKernelGGL(advance_kernel, dim3((T + 63) / 64), dim3(64), 0, (hipStream_t)stream, p->pos, p->ctx, T);
  return mlora_launch_status("decode_step");
}

}  // namespace

extern "C" int mlora_decode_step(const mlora_decode_plan* p, void* stream) {
  MLORA_CHECK(p && p->layers, MLORA_ERR_INVALID, "decode_step: null plan");
  const int T = p->T, H = p->hidden, I = p->inter, Hq = p->n_q_heads, Hkv = p->n_kv_heads, D = p->head_dim;
  MLORA_CHECK(T > 0 && T <= 65535, MLORA_ERR_UNSUPPORTED, "decode_step: T=%d outside 1..65535", T);
  MLORA_CHECK(p->tokens && p->rows && p->pos && p->ctx && p->resid && p->xn && p->qkv && p->attn && p->gate_up && p->act &&
                  p->logits && p->embed && p->norm && p->lm_head_p && p->block_table && p->rope_cos && p->rope_sin,
              MLORA_ERR_INVALID, "decode_step: null buffer");
  // every layer of the plan is looked at before the first launch: a rejected call enqueues nothing
  {
    const bool any_lora = p->tok_adapter != nullptr && p->lora_r > 0;
    for (int l = 0; l < p->n_layers; ++l) {
      const mlora_layer& L = p->layers[l];
      MLORA_CHECK(L.ln1 && L.ln2 && L.qkv_p && L.o_p && L.down_p && L.k_cache && L.v_cache, MLORA_ERR_INVALID,
                  "decode_step: layer %d has a null weight, norm or cache pointer", l);
      const bool gu_lora = any_lora && (L.lora[MLORA_GATE].A || L.lora[MLORA_UP].A);
      MLORA_CHECK(L.gate_up_p || (T <= 64 && L.gate_up_il_p && !gu_lora), MLORA_ERR_INVALID, "decode_step: layer %d needs gate_up_p", l);
      if (any_lora)
        for (int j = 0; j < 7; ++j)
          MLORA_CHECK(!L.lora[j].A || L.lora[j].B, MLORA_ERR_INVALID, "decode_step: layer %d projection %d has A but no B table", l, j);
    }
  }
  if (T > 64) {
    MLORA_CHECK(!(p->tok_adapter != nullptr && p->lora_r > 0 && p->lora_dense != 0), MLORA_ERR_UNSUPPORTED,
                "decode_step: the dense shrink (adapter rows appended to the base weights) serves at most 64 sequences (T=%d)", T);
    return decode_step_wide(p, stream);
  }
  const int q_sz = Hq * D, kv_sz = Hkv * D, qkv_sz = q_sz + 2 * kv_sz;
  const bool lora = p->tok_adapter != nullptr && p->lora_r > 0;
  const bool dense = lora && p->lora_dense != 0;
  const int r = p->lora_r, n_ad = p->lora_n_ad;
  const float sc = p->lora_scaling;
  // the o projection's delta from riders of its GEMV launch (o_p is then the base weight alone)
  const bool o_ride = dense && p->lora_dense == 2;
  const int ks_ride = o_ride ? mlora_gemv_delta_ride_ksplit(T, q_sz, H, r) : 0;
  MLORA_CHECK(!o_ride || (ks_ride > 0 && mlora_rope_attn_oshrink_ok(T, Hq, Hkv, D, r) && p->ksplit_ws &&
                          mlora_gemv_ksplit_bytes(T, H, ks_ride + 1) <= p->ksplit_ws_bytes),
              MLORA_ERR_UNSUPPORTED, "decode_step: lora_dense = 2 is not served for T=%d, rank %d, or ksplit_ws is too small", T, r);
  f16* qkv = (f16*)p->qkv;
  f16* gu = (f16*)p->gate_up;
  // LoRA scratch: slots 0-2 q/k/v partials, slot 3 o_proj, slot 4 down_proj / stand-alone calls
  const int Kmax = H > I ? (H > q_sz ? H : q_sz) : (I > q_sz ? I : q_sz);
  size_t slot = lora ? mlora_gather_mm_workspace_bytes(T, Kmax, r) : 0;
  if (dense && slot < (size_t)T * n_ad * r * sizeof(float)) slot = (size_t)T * n_ad * r * sizeof(float);
  if (o_ride && slot < (size_t)Hq * T * r * sizeof(float)) slot = (size_t)Hq * T * r * sizeof(float);   // the o shrink's head shares
  // dense q/k/v shrink rows may come as kq blocks of K-range partials (one-workgroup-per-unit GEMV): 3 kq slots
  const int kq = dense ? mlora_gemv_split_kq(T, H, qkv_sz, 3 * n_ad * r) : 1;
  const size_t ws_need = (size_t)(3 * kq + 2) * slot;
  MLORA_CHECK(!lora || (p->lora_ws && p->lora_ws_bytes >= ws_need), MLORA_ERR_WORKSPACE,
              "decode_step: lora_ws of %zu bytes given, %zu needed", p->lora_ws_bytes, ws_need);
  char* ws = (char*)p->lora_ws;
  void* ws_qkv = ws;
  void* ws_o = ws + (size_t)3 * kq * slot;
  void* ws_down = ws + (size_t)(3 * kq + 1) * slot;
  auto delta = [&](void* y, int y_dtype, int ldy, const void* x, const mlora_lora_proj& lp, int K, int N) -> int {
    if (!lora || !lp.A) return MLORA_OK;
    return mlora_gather_mm(y, y_dtype, ldy, x, MLORA_FRAG, lp.A, lp.B, p->tok_adapter, sc, T, K, N, r, n_ad, ws_down, slot, stream);
  };
  // K split of the two narrow accumulating GEMVs: the slices' partials are summed by the RMSNorm that reads the
  // residual next.  N_total counts the appended adapter rows of the dense shrink.
  // Shrink units that ride in the launch count as the workgroups they are (a launch of more workgroups than compute
  // units ends with a second round on a few of them).
  auto ksplit_of = [&](int K, bool has_lora) -> int {
    const int ld_part = H + (dense && has_lora ? n_ad * r : 0);
    const int n_total = ld_part + (!dense && has_lora ? mlora_gemv_shrink_rows(K, 1, n_ad) : 0);
    const int ks = p->ksplit_ws ? mlora_gemv_ksplit(T, K, n_total) : 1;
    return ks > 1 && mlora_gemv_ksplit_bytes(T, ld_part, ks) <= p->ksplit_ws_bytes ? ks : 1;
  };
  // o_proj / down_proj: resid += x . W^T with the adapter's shrink riding along (dense: appended rows; else shrink units)
  auto acc_gemv = [&](const void* x, const void* Wp, int K, const mlora_lora_proj& lp, void* v_ws, int ks) -> int {
    const bool has = lora && lp.A;
    const void* A1[1] = {lp.A};
    if (has && dense)
      return mlora_gemv_frag_acc_ksplit(p->resid, (float*)v_ws, p->ksplit_ws, ks, x, Wp, T, K, H, n_ad * r, nullptr, nullptr, 0,
                                        nullptr, 0, 0, stream);
    if (has)
      return mlora_gemv_frag_acc_ksplit(p->resid, nullptr, p->ksplit_ws, ks, x, Wp, T, K, H, 0, v_ws, A1, 1, p->tok_adapter, r, n_ad,
                                        stream);
    return mlora_gemv_frag_acc_ksplit(p->resid, nullptr, p->ksplit_ws, ks, x, Wp, T, K, H, 0, nullptr, nullptr, 0, nullptr, 0, 0, stream);
  };
  // RMSNorm of the residual stream, first applying the pending expand and K-split partials of the GEMV before it
  auto norm = [&](const void* w, const void* B, const void* v_ws, int K, int ks) -> int {
    const int ld_part = H + (dense && B ? n_ad * r : 0);
    if (B || ks > 1)
      return mlora_rmsnorm_ksplit(p->xn, MLORA_FRAG, p->resid, p->ksplit_ws, ks, ld_part, w, p->eps, T, H, B ? v_ws : nullptr, dense, B,
                                  p->tok_adapter, sc, K, r, n_ad, stream);
    return mlora_rmsnorm(p->xn, MLORA_FRAG, p->resid, MLORA_F32, w, p->eps, T, H, stream);
  };
  const void* pending_B = nullptr;    // down_proj expand and partials of the previous layer
  int pending_ks = 1;
  STEP(mlora_embed(p->resid, MLORA_F32, p->embed, p->tokens, T, H, p->vocab, stream));
  for (int l = 0; l < p->n_layers; ++l) {
    const mlora_layer& L = p->layers[l];
    STEP(norm(L.ln1, pending_B, ws_down, I, pending_ks));
    const bool qkv_lora = lora && (L.lora[MLORA_Q].A || L.lora[MLORA_K].A || L.lora[MLORA_V].A);
    const bool o_lora = lora && L.lora[MLORA_O].A;
    const bool o_via_ride = o_lora && o_ride;   // the attention launch writes the o shrink's head shares, riders of the o GEMV expand them
    if (qkv_lora) {
      const void* A3[3] = {L.lora[MLORA_Q].A, L.lora[MLORA_K].A, L.lora[MLORA_V].A};
      const void* B3[3] = {L.lora[MLORA_Q].A ? L.lora[MLORA_Q].B : nullptr, L.lora[MLORA_K].A ? L.lora[MLORA_K].B : nullptr,
                           L.lora[MLORA_V].A ? L.lora[MLORA_V].B : nullptr};
      if (dense) STEP(mlora_gemv_frag_split_kq(qkv, (float*)ws_qkv, kq, p->xn, L.qkv_p, T, H, qkv_sz, 3 * n_ad * r, stream));
      else STEP(mlora_gemv_frag_lora(qkv, MLORA_F16, MLORA_STORE, p->xn, L.qkv_p, T, H, qkv_sz, ws_qkv, A3, 3, p->tok_adapter, r, n_ad, stream));
      if (o_via_ride)
        STEP(mlora_rope_attn_decode_oshrink(p->attn, MLORA_FRAG, qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows,
                                            p->pos, p->ctx, p->rope_cos, p->rope_sin, p->max_pos, T, Hq, Hkv, D, p->n_pages, p->n_seq,
                                            ws_qkv, dense ? kq : 0, B3, p->tok_adapter, sc, H, r, n_ad, L.lora[MLORA_O].A, ws_o, stream));
      else
        STEP(mlora_rope_attn_decode(p->attn, MLORA_FRAG, qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows, p->pos,
                                    p->ctx, p->rope_cos, p->rope_sin, p->max_pos, T, Hq, Hkv, D, p->n_pages, p->n_seq, ws_qkv,
                                    dense ? kq : 0, B3, p->tok_adapter, sc, H, r, n_ad, stream));
    } else {
      STEP(mlora_gemv_frag(qkv, MLORA_F16, MLORA_STORE, p->xn, L.qkv_p, T, H, qkv_sz, stream));
      if (o_via_ride)
        STEP(mlora_rope_attn_decode_oshrink(p->attn, MLORA_FRAG, qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows,
                                            p->pos, p->ctx, p->rope_cos, p->rope_sin, p->max_pos, T, Hq, Hkv, D, p->n_pages, p->n_seq,
                                            nullptr, 0, nullptr, p->tok_adapter, sc, H, r, n_ad, L.lora[MLORA_O].A, ws_o, stream));
      else
        STEP(mlora_rope_attn_decode(p->attn, MLORA_FRAG, qkv, L.k_cache, L.v_cache, p->block_table, p->max_blocks, p->rows, p->pos,
                                    p->ctx, p->rope_cos, p->rope_sin, p->max_pos, T, Hq, Hkv, D, p->n_pages, p->n_seq, nullptr, 0,
                                    nullptr, nullptr, 0.f, 0, 0, 0, stream));
    }
    if (o_via_ride) {
      // base GEMV + riders; the delta rows are one more slot of partials for the norm, which has no table to stream
      STEP(mlora_gemv_frag_acc_ksplit_delta(p->resid, p->ksplit_ws, ks_ride, p->attn, L.o_p, T, q_sz, H, (const float*)ws_o, Hq,
                                            L.lora[MLORA_O].B, p->tok_adapter, sc, r, n_ad, stream));
      STEP(mlora_rmsnorm_ksplit(p->xn, MLORA_FRAG, p->resid, p->ksplit_ws, ks_ride + 1, H, L.ln2, p->eps, T, H, nullptr, 0, nullptr, nullptr,
                                0.f, 0, 0, 0, stream));
    } else {
      const int ks_o = ksplit_of(q_sz, o_lora);
      STEP(acc_gemv(p->attn, L.o_p, q_sz, L.lora[MLORA_O], ws_o, ks_o));
      STEP(norm(L.ln2, o_lora ? L.lora[MLORA_O].B : nullptr, ws_o, q_sz, ks_o));
    }
    const bool gu_lora = lora && (L.lora[MLORA_GATE].A || L.lora[MLORA_UP].A);
    if (L.gate_up_il_p && !gu_lora) {
      STEP(mlora_gemv_frag_silu(p->act, p->xn, L.gate_up_il_p, T, H, I, stream));
    } else {
      STEP(mlora_gemv_frag(gu, MLORA_F16, MLORA_STORE, p->xn, L.gate_up_p, T, H, 2 * I, stream));
      STEP(delta(gu, MLORA_F16, 2 * I, p->xn, L.lora[MLORA_GATE], H, I));
      STEP(delta(gu + I, MLORA_F16, 2 * I, p->xn, L.lora[MLORA_UP], H, I));
      STEP(mlora_silu_mul(p->act, MLORA_FRAG, gu, gu + I, 2 * I, T, I, stream));
    }
    const bool down_lora = lora && L.lora[MLORA_DOWN].A;
    pending_ks = ksplit_of(I, down_lora);
    STEP(acc_gemv(p->act, L.down_p, I, L.lora[MLORA_DOWN], ws_down, pending_ks));
    pending_B = down_lora ? L.lora[MLORA_DOWN].B : nullptr;   // expanded inside the next RMSNorm launch
  }
  STEP(norm(p->norm, pending_B, ws_down, I, pending_ks));
  STEP(mlora_gemv_frag(p->logits, MLORA_F32, MLORA_STORE, p->xn, p->lm_head_p, T, H, p->vocab, stream));
  STEP(mlora_argmax(p->tokens, p->logits, T, p->vocab, stream));
  hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, p->pos, p->ctx, T);
  return mlora_launch_status("decode_step");
}
