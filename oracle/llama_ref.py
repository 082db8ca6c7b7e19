"""CPU oracle for the per-layer operators and the greedy decode loop (test infrastructure only).

Follows the graph of `tvm/llama_auto_batcher/llama_for_causal_lm.py` (layer wiring `:79-84`,
final norm `:99`, last-token index at prefill `:131-136`, fp32 logits `:124-128`), the patched
attention of `tvm/llama_auto_batcher/compile_tvm.py:116-160` (LoRA delta added to the projection
outputs before attention) and the loop of `tvm/llama_auto_batcher/llama_exec_graph.py:58-141`.

Two precision modes:
  * "fp32"  - every intermediate stays float32 (softmax / norm statistics in float64).  This is the
              reference CPU path the kernel tolerances (max relative error 2e-3) are quoted against.
  * "mixed" - the same arithmetic, but tensors are rounded to fp16 exactly where the HIP path stores
              fp16 (normed activations, q/k/v, attention output, gate/up, SiLU product); the residual
              stream and the logits stay fp32.  The HIP path then differs only in fp32 summation
              order - which still flips an fp16 rounding on a fraction of a percent of the stored
              elements, so token identity is tested where the top-2 logit margin is decided.
"""
from __future__ import annotations

import numpy as np

from .lora_ref import gather_mm_ref


def f16(x):
    """Round to fp16 storage and come back to float32."""
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def rmsnorm_ref(x, w, eps):
    """x * rsqrt(mean(x^2) + eps) * w   (`nn.RMSNorm(hidden, -1, eps, bias=False)`,
    `llama_for_causal_lm.py:76-77,93`); statistics in float64, result float32."""
    x64 = np.asarray(x, dtype=np.float64)
    inv = 1.0 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + eps)
    return (x64 * inv * np.asarray(w, dtype=np.float64)).astype(np.float32)


def silu_mul_ref(gate, up):
    """silu(gate) * up  (`llama_for_causal_lm.py:35-36`)."""
    g = np.asarray(gate, dtype=np.float64)
    return (g / (1.0 + np.exp(-g)) * np.asarray(up, dtype=np.float64)).astype(np.float32)


def rope_tables(head_dim: int, theta: float, max_pos: int):
    """cos/sin [max_pos, head_dim/2] float32; inv_freq_i = theta^(-2i/d), angle = pos * inv_freq
    (rotary_dim = head_dim, scale 1: `llama_for_causal_lm.py:166-172`)."""
    inv_freq = theta ** (-(np.arange(0, head_dim, 2, dtype=np.float64) / head_dim))
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv_freq[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def rope_ref(x, pos, cos, sin):
    """Rotate-half RoPE on x [T, H, D] at integer positions pos [T]: element i pairs with i + D/2."""
    x = np.asarray(x, dtype=np.float32)
    half = x.shape[-1] // 2
    c = cos[np.asarray(pos)][:, None, :]
    s = sin[np.asarray(pos)][:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1)


def attention_dense_ref(q, K, V, q_pos):
    """Causal softmax(q K^T / sqrt(d)) V for one sequence on contiguous K/V.
    q [n, Hq, D] at absolute positions q_pos [n]; K, V [ctx, Hkv, D]; key j is visible to query i
    iff j <= q_pos[i].  Grouped-query heads: q head h reads kv head h // (Hq // Hkv)."""
    q = np.asarray(q, dtype=np.float64)
    K = np.asarray(K, dtype=np.float64)
    V = np.asarray(V, dtype=np.float64)
    n, Hq, D = q.shape
    ctx, Hkv, _ = K.shape
    g = Hq // Hkv
    mask = np.arange(ctx)[None, :] <= np.asarray(q_pos)[:, None]          # [n, ctx]
    # all heads at once as batched matrix products: [Hkv, g, n, D] x [Hkv, 1, D, ctx]
    qh = q.reshape(n, Hkv, g, D).transpose(1, 2, 0, 3)
    Kh = K.transpose(1, 2, 0)[:, None]                                     # [Hkv, 1, D, ctx]
    Vh = V.transpose(1, 0, 2)[:, None]                                     # [Hkv, 1, ctx, D]
    s = np.matmul(qh, Kh) / np.sqrt(D)                                     # [Hkv, g, n, ctx]
    s = np.where(mask[None, None], s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    out = np.matmul(p, Vh)                                                 # [Hkv, g, n, D]
    return out.transpose(2, 0, 1, 3).reshape(n, Hq, D).astype(np.float32)


class PagedKVRef:
    """Paged KV cache with the host protocol of `llama_exec_graph.py:41-46,66,75-79,85,121-127`:
    add_sequence / begin_forward(seq_ids, append_lens) / attention_with_fused_qkv / end_forward.

    Pages hold `page_size` tokens; physical page ids are handed out from `free_pages` front to back
    (pass a permutation to scatter a sequence over the pool).  K is stored already rotated."""

    def __init__(self, n_layers, n_pages, page_size, n_kv_heads, head_dim, cos, sin, free_pages=None,
                 round_fp16=False):
        self.page_size = page_size
        self.k = np.zeros((n_layers, n_pages, n_kv_heads, page_size, head_dim), dtype=np.float32)
        self.v = np.zeros_like(self.k)
        self.free = list(range(n_pages)) if free_pages is None else [int(p) for p in free_pages]
        self.tables = {}
        self.lens = {}
        self.cos, self.sin = cos, sin
        self.round = f16 if round_fp16 else (lambda a: np.asarray(a, dtype=np.float32))
        self._cur = None

    def add_sequence(self, sid):
        assert sid not in self.tables, f"sequence {sid} already added"
        self.tables[sid] = []
        self.lens[sid] = 0

    def begin_forward(self, seq_ids, append_lens):
        assert self._cur is None, "begin_forward called twice without end_forward"
        assert len(seq_ids) == len(append_lens)
        for sid, n in zip(seq_ids, append_lens):
            need = -(-(self.lens[sid] + n) // self.page_size)
            while len(self.tables[sid]) < need:
                assert self.free, "paged KV cache out of pages"
                self.tables[sid].append(self.free.pop(0))
        self._cur = (list(seq_ids), list(append_lens))

    def end_forward(self):
        seq_ids, append_lens = self._cur
        for sid, n in zip(seq_ids, append_lens):
            self.lens[sid] += n
        self._cur = None

    def gather(self, layer, sid, length):
        """Walk the block table: logical K/V [length, Hkv, D] of a sequence."""
        pos = np.arange(length)
        pages = np.asarray(self.tables[sid], dtype=np.int64)[pos // self.page_size]
        off = pos % self.page_size
        return self.k[layer, pages, :, off, :], self.v[layer, pages, :, off, :]

    def attention_with_fused_qkv(self, layer, qkv, n_q_heads):
        """qkv [T, Hq + 2 Hkv, D] for the tokens announced by begin_forward (sequence-major);
        appends rotated K and V, attends causally, returns [T, Hq * D]
        (`llama_for_causal_lm.py:55-64`)."""
        seq_ids, append_lens = self._cur
        qkv = np.asarray(qkv, dtype=np.float32)
        T, Hall, D = qkv.shape
        Hkv = (Hall - n_q_heads) // 2
        out = np.empty((T, n_q_heads, D), dtype=np.float32)
        t0 = 0
        for sid, n in zip(seq_ids, append_lens):
            base = self.lens[sid]
            pos = base + np.arange(n)
            blk = qkv[t0:t0 + n]
            q = self.round(rope_ref(blk[:, :n_q_heads], pos, self.cos, self.sin))
            k = self.round(rope_ref(blk[:, n_q_heads:n_q_heads + Hkv], pos, self.cos, self.sin))
            v = self.round(blk[:, n_q_heads + Hkv:])
            pages = np.asarray(self.tables[sid], dtype=np.int64)[pos // self.page_size]
            self.k[layer, pages, :, pos % self.page_size, :] = k
            self.v[layer, pages, :, pos % self.page_size, :] = v
            Kc, Vc = self.gather(layer, sid, base + n)
            out[t0:t0 + n] = attention_dense_ref(q, Kc, Vc, pos)
            t0 += n
        assert t0 == T
        return self.round(out.reshape(T, n_q_heads * D))


class LlamaRef:
    """Llama-style decoder with per-token adapter-indexed LoRA on any subset of the 7 linears.

    weights: dict name -> float32 array (fp16-rounded values when the HIP path runs fp16):
      embed_tokens [V,H], lm_head [V,H], norm [H], layers.{l}.{q,k,v,o,gate,up,down}_proj [N,K],
      layers.{l}.{input,post_attention}_layernorm [H].
    lora: dict 'layers.{l}.{proj}.lora_A.{tag}' -> [n_ad, r, K], '...lora_B.{tag}' -> [n_ad, N, r];
      `scaling[tag]` the alpha/r of that adapter type.
    """

    def __init__(self, shape, weights, lora=None, scaling=None, mode="fp32"):
        assert mode in ("fp32", "mixed")
        self.shape = shape
        self.w = weights
        self.lora = lora or {}
        self.scaling = scaling or {}
        self.mode = mode
        self.rnd = f16 if mode == "mixed" else (lambda a: a)

    def new_cache(self, n_pages, page_size, max_pos, free_pages=None):
        s = self.shape
        cos, sin = rope_tables(s.head_dim, s.rope_theta, max_pos)
        return PagedKVRef(s.num_hidden_layers, n_pages, page_size, s.num_key_value_heads, s.head_dim,
                          cos, sin, free_pages, round_fp16=(self.mode == "mixed"))

    def _delta_into(self, y, x, l, proj, tok_adapter):
        """y += LoRA delta of every adapter type that targets this projection.
        tok_adapter: dict tag -> ids [T] (-1 = token does not use this type)."""
        for tag, ids in (tok_adapter or {}).items():
            ka = f"layers.{l}.{proj}.lora_A.{tag}"
            if ka in self.lora:
                y = gather_mm_ref(y, x, self.lora[ka], self.lora[f"layers.{l}.{proj}.lora_B.{tag}"],
                                  ids, self.scaling[tag])
        return y

    def _proj(self, x, l, proj, tok_adapter):
        """Projection whose output is stored (fp16 in mixed mode): base rounded, then delta added and rounded.
        With `fuse_blocks` = n set (the HIP prefill carries the delta inside the base GEMM for every n-token block whose
        tokens all name one adapter of the pass's single adapter type): base + delta rounded ONCE for those tokens."""
        base = x @ self.w[f"layers.{l}.{proj}"].T
        y = self.rnd(base)
        y2 = self._delta_into(y, x, l, proj, tok_adapter)
        if y2 is y:
            return y
        out = self.rnd(y2)
        once = self._rounded_once(tok_adapter, x.shape[0])
        if once is not None and once.any():
            delta = self._delta_into(np.zeros_like(base), x, l, proj, tok_adapter)
            out = np.array(out)
            out[once] = self.rnd(base[once] + delta[once])
        return out

    def _rounded_once(self, tok_adapter, T):
        n = getattr(self, "fuse_blocks", None)
        if not n or self.mode != "mixed" or not tok_adapter or len(tok_adapter) != 1:
            return None
        ids = np.asarray(next(iter(tok_adapter.values())))
        once = np.zeros(T, dtype=bool)
        for t0 in range(0, T, n):
            blk = ids[t0:t0 + n]
            once[t0:t0 + n] = blk[0] >= 0 and bool((blk == blk[0]).all())
        return once

    def _proj_residual(self, resid, x, l, proj, tok_adapter):
        """Projection accumulated into the fp32 residual stream: resid + base, then + delta."""
        resid = resid + x @ self.w[f"layers.{l}.{proj}"].T
        return self._delta_into(resid, x, l, proj, tok_adapter)

    def forward(self, tokens, kv, tok_adapter=None, logits_rows=None, tap_depths=()):
        """tokens [T] (sequence-major, as announced to kv.begin_forward) -> logits [T or len(rows), V] float32.
        tap_depths: layer counts d at which the logits of the model cut off after d layers (final norm and head on
        the residual stream as it stands there) are kept in self.taps[d] - what a pass of a d-layer model over the
        same weights returns, without a second pass."""
        s = self.shape
        eps = s.rms_norm_eps
        self.taps = {}
        resid = np.asarray(self.w["embed_tokens"], dtype=np.float32)[np.asarray(tokens)]
        T = resid.shape[0]
        for l in range(s.num_hidden_layers):
            xn = self.rnd(rmsnorm_ref(resid, self.w[f"layers.{l}.input_layernorm"], eps))
            q = self._proj(xn, l, "q_proj", tok_adapter)
            k = self._proj(xn, l, "k_proj", tok_adapter)
            v = self._proj(xn, l, "v_proj", tok_adapter)
            qkv = np.concatenate([q, k, v], axis=-1).reshape(T, -1, s.head_dim)
            attn = kv.attention_with_fused_qkv(l, qkv, s.num_attention_heads)
            resid = self._proj_residual(resid, attn, l, "o_proj", tok_adapter)
            xn = self.rnd(rmsnorm_ref(resid, self.w[f"layers.{l}.post_attention_layernorm"], eps))
            g = self._proj(xn, l, "gate_proj", tok_adapter)
            u = self._proj(xn, l, "up_proj", tok_adapter)
            act = self.rnd(silu_mul_ref(g, u))
            resid = self._proj_residual(resid, act, l, "down_proj", tok_adapter)
            if l + 1 in tap_depths and l + 1 < s.num_hidden_layers:
                self.taps[l + 1] = self._head(resid, logits_rows)
        return self._head(resid, logits_rows)

    def _head(self, resid, logits_rows):
        if logits_rows is not None:
            resid = resid[np.asarray(logits_rows)]
        xn = self.rnd(rmsnorm_ref(resid, self.w["norm"], self.shape.rms_norm_eps))
        return (xn @ self.w["lm_head"].T).astype(np.float32)


def greedy_generate_ref(model, prompts, tok_adapter, max_gen_len, n_pages, page_size=16, free_pages=None,
                        eos_token_id=None, return_logits=False):
    """Prefill each sequence, then batched greedy decode (`llama_exec_graph.py:58-141`).

    The first generated token is the prefill argmax (`:92`); decoding continues while the last token
    is not EOS and fewer than `max_gen_len` tokens have been produced (`:94-100`); that rule is first
    applied after a decode step (`:110-138`), so every sequence decodes at least once; the batch shrinks
    as sequences finish.  `tok_adapter`: dict tag -> per-request adapter ids [B] (-1 = none).
    np.argmax breaks ties towards the lowest index (`:92,137`).
    Returns a list of B lists of token ids (each of length <= max_gen_len); with return_logits=True also
    the top-1 minus top-2 logit margin of every generated token, in the same nesting, and the logit
    standard deviation of each token's row (the scale against which a margin is small or large)."""
    B = len(prompts)
    max_pos = max(len(p) for p in prompts) + max_gen_len + 1
    kv = model.new_cache(n_pages, page_size, max_pos, free_pages)
    outputs = {}
    margins = {sid: [] for sid in range(B)}
    scales = {sid: [] for sid in range(B)}
    for sid in range(B):
        kv.add_sequence(sid)
        n = len(prompts[sid])
        kv.begin_forward([sid], [n])
        ta = {tag: np.full(n, ids[sid], dtype=np.int32) for tag, ids in (tok_adapter or {}).items()}
        logits = model.forward(np.asarray(prompts[sid]), kv, ta, logits_rows=[n - 1])
        kv.end_forward()
        outputs[sid] = [int(np.argmax(logits[0]))]
        margins[sid].append(_margin(logits[0]))
        scales[sid].append(float(logits[0].std()))
    live = list(range(B))
    while live:
        toks = np.asarray([outputs[sid][-1] for sid in live])
        kv.begin_forward(live, [1] * len(live))
        ta = {tag: np.asarray([ids[sid] for sid in live], dtype=np.int32) for tag, ids in (tok_adapter or {}).items()}
        logits = model.forward(toks, kv, ta)
        kv.end_forward()
        for i, sid in enumerate(live):
            outputs[sid].append(int(np.argmax(logits[i])))
            margins[sid].append(_margin(logits[i]))
            scales[sid].append(float(logits[i].std()))
        live = [sid for sid in live if _alive(outputs[sid], max_gen_len, eos_token_id)]
    out = [outputs[sid] for sid in range(B)]
    if return_logits:
        return out, [margins[sid] for sid in range(B)], [scales[sid] for sid in range(B)]
    return out


def _alive(out, max_gen_len, eos):
    return (eos is None or out[-1] != eos) and len(out) < max_gen_len


def _margin(row):
    top2 = np.partition(row, -2)[-2:]
    return float(top2[1] - top2[0])
