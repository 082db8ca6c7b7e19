"""Llama-style decoder on the HIP operator set, with per-token adapter-indexed LoRA.

Keeps the entry points the reference compiles into its VM (`tvm/llama_auto_batcher/compile_tvm.py:163-285`):
    embed(input_ids) ; prefill_no_adapter(h, kv) ; prefill_a{i}(h, kv, wids) ;
    decode_no_adapter(h, kv) ; decode_a{i}(h, kv, wids) ; mixed_decode_a{i}_a{j}...(h, kv, sids_i, wids_i, ...)
each returning fp32 logits, reachable by name through `model[name]` the way the reference calls `vm[name]`.
The layer graph follows `tvm/llama_auto_batcher/llama_for_causal_lm.py:79-84,95-100,121-144` and the
patched attention of `compile_tvm.py:116-160`; the reference adds LoRA to q and v only (`:180-181`), here
any subset of the seven linears can carry adapters, of several adapter types (rank / alpha) at once.

Precision contract: fp16 weights and stored activations, fp32 accumulation everywhere, fp32 residual
stream (the o_proj / down_proj kernels accumulate straight into it), fp32 logits.
"""
from __future__ import annotations

import re

import numpy as np
import torch

from . import ops
from .kv_cache import PagedKVCache
from .synth import LINEARS, LlamaShape, linear_dims


class LoraType:
    """One adapter type (rank, alpha): stacked tables per (layer, projection)."""

    def __init__(self, r: int, scaling: float, n_adapters: int):
        self.r, self.scaling, self.n_adapters = r, float(scaling), n_adapters
        self.tables = {}     # (layer, proj) -> (A [n_ad, r, K], B [n_ad, N, r])
        self.row_of = None   # weight id -> table row when the two differ (adapters loaded from files), else None

    def rows(self, wids: np.ndarray) -> np.ndarray:
        """Table rows of the weight ids `wids` (-1 stays -1); raises on an id that is not loaded."""
        if self.row_of is None:
            if wids.size and (wids.min() < -1 or wids.max() >= self.n_adapters):
                raise ValueError(f"adapter weight id out of range: {wids.min()}..{wids.max()} of {self.n_adapters}")
            return wids
        out = np.full(wids.shape, -1, dtype=np.int32)
        for i, w in enumerate(wids.tolist()):
            if w >= 0:
                if w not in self.row_of:
                    raise ValueError(f"adapter weight id {w} is not loaded (loaded: {sorted(self.row_of)})")
                out[i] = self.row_of[w]
            elif w != -1:
                raise ValueError(f"bad adapter weight id {w}")
        return out

    def add(self, layer: int, proj: str, A: torch.Tensor, B: torch.Tensor):
        if A.shape[0] != self.n_adapters or A.shape[1] != self.r or B.shape[0] != self.n_adapters or B.shape[2] != self.r:
            raise ValueError(f"LoRA table shape mismatch at layer {layer} {proj}: A{tuple(A.shape)} B{tuple(B.shape)}")
        self.tables[(layer, proj)] = (A.contiguous(), B.contiguous())


class LlamaForCausalLM:
    def __init__(self, shape: LlamaShape, device="cuda:0"):
        self.shape = shape
        self.device = torch.device(device)
        self.layers = []          # per layer dict: qkv, o, gate_up, down (PackedWeight), ln1, ln2 (fp16 [H])
        self.embed_tokens = None
        self.lm_head = None
        self.norm = None
        self.lora_types = []      # index = adapter type id
        self._ws = None

    # ------------------------------------------------------------------ weights
    def load_layer(self, l: int, w: dict):
        """w: the seven projection weights [N, K] fp16 and the two norm weights of layer l
        (keys 'q_proj', ..., 'input_layernorm', 'post_attention_layernorm').  q/k/v and gate/up are fused
        row-wise and stored in matrix-core fragment order."""
        assert l == len(self.layers), "layers must be loaded in order"
        dev = self.device
        qkv = torch.cat([w["q_proj"], w["k_proj"], w["v_proj"]], 0).to(dev, torch.float16)
        gu = torch.cat([w["gate_proj"], w["up_proj"]], 0).to(dev, torch.float16)
        self.layers.append({
            "qkv": ops.PackedWeight(qkv), "o": ops.PackedWeight(w["o_proj"].to(dev, torch.float16)),
            "gate_up": ops.PackedWeight(gu), "down": ops.PackedWeight(w["down_proj"].to(dev, torch.float16)),
            "ln1": w["input_layernorm"].to(dev, torch.float16).contiguous(),
            "ln2": w["post_attention_layernorm"].to(dev, torch.float16).contiguous(),
        })

    def load_head(self, embed_tokens, lm_head, norm):
        dev = self.device
        self.embed_tokens = embed_tokens.to(dev, torch.float16).contiguous()
        self.lm_head = ops.PackedWeight(lm_head.to(dev, torch.float16))
        self.norm = norm.to(dev, torch.float16).contiguous()

    def add_lora_type(self, lora_type: LoraType) -> int:
        self.lora_types.append(lora_type)
        return len(self.lora_types) - 1

    @classmethod
    def from_synthetic(cls, seed: int, shape: LlamaShape, lora_specs=(), device="cuda:0", synth=None):
        """Random-init model generated on the device (bit-identical to the CPU generation of the same seed)."""
        from . import synth as S
        m = cls(shape, device)
        for l in range(shape.num_hidden_layers):
            w = S.layer_weights(seed, shape, l, torch.float16, device)
            m.load_layer(l, {k.split(".", 2)[2]: v for k, v in w.items()})
            del w
        m.load_head(S.normal(seed, "embed_tokens", (shape.vocab_size, shape.hidden_size), 0.02, torch.float16, device),
                    S.normal(seed, "lm_head", (shape.vocab_size, shape.hidden_size), 0.02, torch.float16, device),
                    torch.ones(shape.hidden_size, dtype=torch.float16, device=device))
        for tid, spec in enumerate(lora_specs):
            lt = LoraType(spec.r, spec.scaling, spec.n_adapters)
            lw = S.lora_weights(seed, shape, spec, torch.float16, device, tag=f"a{tid}")
            for l in range(shape.num_hidden_layers):
                for proj in spec.targets:
                    lt.add(l, proj, lw[f"layers.{l}.{proj}.lora_A.a{tid}"], lw[f"layers.{l}.{proj}.lora_B.a{tid}"])
            m.add_lora_type(lt)
        return m

    def interleaved_gate_up(self):
        """Per layer, the gate/up matrix with 16-row tiles of gate and up alternating (for the GEMV whose epilogue
        is the SiLU product).  Cached; one more copy of that matrix."""
        cache = getattr(self, "_il_cache", None)
        if cache is None:
            cache = [ops.interleave_gate_up(L["gate_up"].unpack()) for L in self.layers]
            self._il_cache = cache
        return cache

    def lora_union(self, tids):
        """-> (type, {tid: first table row}): one set of tables that serves the adapter types `tids` in one launch.
        For a single type that is the type itself.  For several, the ranks are zero-padded to the largest (the
        reference's padded strategy, `tvm/lora_only/case_study/multiple_ranks.py:66-95`) and the adapters of all
        types are stacked, type after type; projections a type does not adapt are zero tables.  Zero rows of A give
        v = 0 exactly and zero columns of B add 0 to every sum, so each token gets the delta of its own unpadded
        adapter bit for bit.  The types must share one scaling (alpha / r).  Cached; costs a copy of the tables."""
        tids = tuple(int(t) for t in tids)
        if len(tids) == 1:
            return self.lora_types[tids[0]], {tids[0]: 0}
        cache = getattr(self, "_union_cache", None)
        if cache is None:
            cache = self._union_cache = {}
        if tids in cache:
            return cache[tids]
        types = [self.lora_types[t] for t in tids]
        if any(lt.scaling != types[0].scaling for lt in types):
            raise ValueError("lora_union: the adapter types differ in scaling")
        rmax = max(lt.r for lt in types)
        base, n = {}, 0
        for t, lt in zip(tids, types):
            base[t] = n
            n += lt.n_adapters
        union = LoraType(rmax, types[0].scaling, n)
        for key in sorted({k for lt in types for k in lt.tables}):
            ref = next(lt.tables[key] for lt in types if key in lt.tables)
            K, N = ref[0].shape[2], ref[1].shape[1]
            A = torch.zeros((n, rmax, K), dtype=torch.float16, device=self.device)
            B = torch.zeros((n, N, rmax), dtype=torch.float16, device=self.device)
            for t, lt in zip(tids, types):
                tab = lt.tables.get(key)
                if tab is not None:
                    A[base[t]:base[t] + lt.n_adapters, :lt.r] = tab[0]
                    B[base[t]:base[t] + lt.n_adapters, :, :lt.r] = tab[1]
            union.add(key[0], key[1], A, B)
        cache[tids] = (union, base)
        return cache[tids]

    def union_rows(self, tids, T, pairs):
        """Table rows [T] (int32, host) of a batch in the tables of `lora_union(tids)`; `pairs` as for `_ids`."""
        _, base = self.lora_union(tids)
        full = np.full(T, -1, dtype=np.int32)
        for tid, ids in self._ids(T, pairs, host=True).items():
            full = np.where(ids >= 0, ids + base[tid], full)
        return full.astype(np.int32)

    def dense_lora_weights(self, tid=0, with_o=True):
        """Per layer, the qkv / o / down weights with the stacked A tables of adapter type `tid` (or of the union of
        a tuple of types) appended as extra rows ([n_ad * r, K] per adapted projection; q, k, v slots always present
        for qkv, zero when not adapted), in fragment order.  with_o=False leaves o as the base weight (its delta then
        comes from riders of the GEMV launch).  Cached; costs one more copy of those matrices."""
        cache = getattr(self, "_dense_cache", None)
        if cache is None:
            cache = self._dense_cache = {}
        if isinstance(tid, tuple) and len(tid) == 1:
            tid = tid[0]
        ck = (tid, bool(with_o))
        if ck in cache:
            return cache[ck]
        lt = self.lora_union(tid)[0] if isinstance(tid, tuple) else self.lora_types[tid]
        out = []
        for l, L in enumerate(self.layers):
            ent = {}
            def slot(proj, K):
                tab = lt.tables.get((l, proj))
                if tab is None:
                    return torch.zeros((lt.n_adapters * lt.r, K), dtype=torch.float16, device=self.device)
                return tab[0].reshape(lt.n_adapters * lt.r, K)
            H, I = self.shape.hidden_size, self.shape.intermediate_size
            if any((l, p) in lt.tables for p in ("q_proj", "k_proj", "v_proj")):
                ent["qkv"] = ops.PackedWeight(torch.cat([L["qkv"].unpack()] + [slot(p, H) for p in ("q_proj", "k_proj", "v_proj")]))
            else:
                ent["qkv"] = L["qkv"]
            for key, proj, K in (("o", "o_proj", self.shape.q_size), ("down", "down_proj", I)):
                if (l, proj) in lt.tables and (with_o or key != "o"):
                    ent[key] = ops.PackedWeight(torch.cat([L[key].unpack(), slot(proj, K)]))
                else:
                    ent[key] = L[key]
            out.append(ent)
        cache[ck] = out
        return out

    def create_paged_kv_cache(self, max_batch_size, max_total_seq_len, prefill_chunk_size, page_size,
                              free_pages=None, max_seq_len=None):
        """Same arguments as the reference's VM function (`llama_for_causal_lm.py:148-174`).  The pool holds
        ceil(max_total_seq_len / page_size) + max_batch_size pages (one partial page per sequence)."""
        s = self.shape
        n_pages = -(-max_total_seq_len // page_size) + max_batch_size
        if free_pages is not None:
            n_pages = len(free_pages)
        max_seq_len = max_seq_len or min(max_total_seq_len, n_pages * page_size)
        max_blocks = -(-max_seq_len // page_size)
        return PagedKVCache(s.num_hidden_layers, n_pages, s.num_key_value_heads, s.head_dim, max_seqs=max_batch_size,
                            max_blocks=max_blocks, rope_theta=s.rope_theta, max_pos=max_blocks * page_size,
                            device=self.device, free_pages=free_pages, page_size=page_size)

    # ------------------------------------------------------------------ forward
    def embed(self, input_ids: torch.Tensor) -> torch.Tensor:
        """input_ids [T] or [b, s] int32 -> hidden [T, H] fp32 (the residual stream)."""
        ids = input_ids.reshape(-1).to(self.device, torch.int32).contiguous()
        return ops.embed(self.embed_tokens, ids, out_dtype=torch.float32)

    def _workspace(self, T, K, r):
        # three slices: projections that share an input (q, k, v) keep their shrink results side by side
        need = 3 * (ops.lib().mlora_gather_mm_workspace_bytes(T, K, r) // 4) + 4
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.float32, device=self.device)
        return self._ws

    def _lora(self, y, x, l, proj, tok_adapter):
        """y += delta for every adapter type that targets (l, proj); tok_adapter: {tid: ids [T] int32}, or the merged
        form {"multi": (tok_bucket, tok_adapter)} in which a token names its adapter type and weight row."""
        if "multi" in tok_adapter:
            tb, ta = tok_adapter["multi"]
            buckets = []
            for lt in self.lora_types:
                tab = lt.tables.get((l, proj))
                buckets.append(None if tab is None else (tab[0], tab[1], lt.scaling))
            if any(b is not None for b in buckets):
                rmax = max(lt.r for lt in self.lora_types)
                ops.gather_mm_multi(y, x, buckets, tb, ta, self._workspace(x.shape[0], x.shape[1], rmax))
            return
        for tid, ids in tok_adapter.items():
            lt = self.lora_types[tid]
            tab = lt.tables.get((l, proj))
            if tab is not None:
                ops.gather_mm(y, x, tab[0], tab[1], ids, lt.scaling, self._workspace(x.shape[0], x.shape[1], lt.r))

    def _targets(self, l, *projs):
        """Does any loaded adapter type carry tables for one of these projections of layer l?"""
        return any(lt.tables.get((l, p)) is not None for lt in self.lora_types for p in projs)

    def _lora_group(self, y, x, l, projs, tok_adapter):
        """The deltas of projections that read the same x and own column ranges of one fused output row:
        projs = ((name, first column, columns), ...).  Batches that mix adapter types issue one call for the group."""
        if "multi" in tok_adapter:
            tb, ta = tok_adapter["multi"]
            live, offs, cols = [], [], []
            for proj, c0, n in projs:
                buckets = []
                for lt in self.lora_types:
                    tab = lt.tables.get((l, proj))
                    buckets.append(None if tab is None else (tab[0], tab[1], lt.scaling))
                if any(b is not None for b in buckets):
                    live.append(buckets)
                    offs.append(c0)
                    cols.append(n)
            if live:
                rmax = max(lt.r for lt in self.lora_types)
                ops.gather_mm_multi_proj(y, x, live, offs, cols, tb, ta, self._workspace(x.shape[0], x.shape[1], rmax))
            return
        (tid, ids), = tok_adapter.items()            # one adapter type: a single bucket that every token names
        lt = self.lora_types[tid]
        live = [(lt.tables.get((l, proj)), c0, n) for proj, c0, n in projs]
        live = [(tab, c0, n) for tab, c0, n in live if tab is not None]
        if len(live) >= 2:
            zeros = getattr(self, "_zero_bucket", None)
            if zeros is None or zeros.numel() < ids.numel():
                zeros = self._zero_bucket = torch.zeros(max(ids.numel(), 64), dtype=torch.int32, device=self.device)
            ops.gather_mm_multi_proj(y, x, [[(tab[0], tab[1], lt.scaling)] for tab, _, _ in live], [c0 for _, c0, _ in live],
                                     [n for _, _, n in live], zeros[:ids.numel()], ids, self._workspace(x.shape[0], x.shape[1], lt.r))
            return
        for proj, c0, n in projs:
            self._lora(y[:, c0:c0 + n], x, l, proj, tok_adapter)

    @staticmethod
    def _merge_types(tok_adapter):
        """{tid: ids} with at most one adapter per token -> per-token (type, weight row) arrays for the multi-rank call."""
        tids = sorted(tok_adapter)
        first = tok_adapter[tids[0]]
        tb = torch.full_like(first, -1)
        ta = torch.full_like(first, -1)
        taken = torch.zeros_like(first, dtype=torch.bool)
        for tid in tids:
            has = tok_adapter[tid] >= 0
            if bool((has & taken).any()):
                raise ValueError("a token is bound to adapters of two types")
            taken |= has
            tb = torch.where(has, torch.full_like(tb, tid), tb)
            ta = torch.where(has, tok_adapter[tid], ta)
        return {"multi": (tb, ta)}

    def forward(self, hidden: torch.Tensor, kv: PagedKVCache, tok_adapter=None, logits_rows=None) -> torch.Tensor:
        """hidden [T, H] fp32 (updated in place), tokens in kv.begin_forward order -> logits fp32."""
        s = self.shape
        tok_adapter = tok_adapter or {}
        # the adapter types of this pass (a batch merged beforehand may name any loaded type)
        lora_tids = tuple(range(len(self.lora_types))) if "multi" in tok_adapter else tuple(tok_adapter)
        if len(tok_adapter) > 1:            # several adapter types (ranks) in the batch: one multi-rank call per projection
            tok_adapter = self._merge_types(tok_adapter)
        T = hidden.shape[0]
        H, I = s.hidden_size, s.intermediate_size
        q_sz, kv_sz = s.q_size, s.kv_size
        resid = hidden
        # a decode step (one token per sequence, T <= 64) keeps its activations in fragment order
        dec_frag = T <= 64 and kv._cur is not None and kv._cur[2]
        # so does every larger pass: the operand loads of the matrix-core linears are then plain copies (norm, attention
        # and SiLU write the order the matrix cores read)
        frag = dec_frag or (T > 64 and H % 32 == 0 and q_sz % 32 == 0 and I % 32 == 0)
        is_decode = kv._cur is not None and bool(kv._cur[2])
        # a decode step (of any number of sequences) and a short prefill split K of the two narrow accumulating linears;
        # the RMSNorm that reads the residual next adds the partial results (the same kernels and slice counts as the
        # native decode step)
        ks_ws = self._ksplit_ws(T) if dec_frag or (frag and (T <= 256 or is_decode)) else None
        # a prefill-sized pass of one adapter type of rank 32 or 64: where a 256-token block agrees on one adapter its
        # deltas ride in the base GEMM as extra k-steps; `rest` names the tokens that still need the separate call
        # (a prefill pass only: the choice needs one read-back, which a decode step recorded into a graph cannot make)
        fuse = None
        if (tok_adapter and "multi" not in tok_adapter and frag and T > 64 and not is_decode
                and not torch.cuda.is_current_stream_capturing() and ops.gemm_frag_preferred(T, H, H)):
            (tid, ids), = tok_adapter.items()
            lt = self.lora_types[tid]
            if lt.r in (32, 64):
                blk, rest = ops.lora_block_adapters(ids, lt.n_adapters)
                fuse = (lt, ids, blk, {tid: rest} if bool((rest >= 0).any()) else None)     # one read-back per pass
        o_shares = None
        if tok_adapter and "multi" not in tok_adapter and len(tok_adapter) == 1 and is_decode and T > 64 and frag:
            (tid, ids), = tok_adapter.items()
            lt = self.lora_types[tid]
            if ops.o_shrink_served(T, s.num_attention_heads, s.num_key_value_heads, s.head_dim, H, lt.r):
                o_shares = (lt, ids)
        parts = None
        for l, L in enumerate(self.layers):
            xn = ops.rmsnorm(resid, L["ln1"], s.rms_norm_eps, frag=frag, parts=parts)
            qkv_projs = (("q_proj", 0, q_sz), ("k_proj", q_sz, kv_sz), ("v_proj", q_sz + kv_sz, kv_sz))
            qkv = self._fused_linear(fuse, xn, L["qkv"], l, qkv_projs) if fuse else None
            if qkv is None:
                qkv = ops.linear(xn, L["qkv"])
                if tok_adapter:
                    self._lora_group(qkv, xn, l, qkv_projs, tok_adapter)
            # a decode step of more than 64 sequences of one adapter type: the o projection's shrink comes off the
            # attention launch in head shares and a launch of expand workgroups adds the deltas behind the base linear
            # (what the native step does for such a batch; same kernels, same order)
            o_sh = None
            if o_shares is not None and (l, "o_proj") in o_shares[0].tables:
                o_sh = o_shares[0].tables[(l, "o_proj")]
            if o_sh is not None:
                attn, vpart = kv.attention_with_fused_qkv(l, qkv, s.num_attention_heads, frag=frag, o_shrink=(o_sh[0], o_shares[1]))
                parts = self._linear_acc(attn, L["o"], resid, ks_ws, self._riding_rows(l, "o_proj", lora_tids, T, q_sz))
                ops.lora_expand_shares(resid, vpart, o_sh[1], o_shares[1], o_shares[0].scaling)
            else:
                attn = kv.attention_with_fused_qkv(l, qkv, s.num_attention_heads, frag=frag)
                if fuse and self._fused_linear(fuse, attn, L["o"], l, (("o_proj", 0, H),), resid=resid) is not None:
                    parts = None
                else:
                    parts = self._linear_acc(attn, L["o"], resid, ks_ws, self._riding_rows(l, "o_proj", lora_tids, T, q_sz))
                    if tok_adapter:
                        self._lora(resid, attn, l, "o_proj", tok_adapter)
            xn = ops.rmsnorm(resid, L["ln2"], s.rms_norm_eps, frag=frag, parts=parts)
            if dec_frag and I % 32 == 0 and not (tok_adapter and self._targets(l, "gate_proj", "up_proj")):
                # decode step without an adapter on gate / up: the SiLU product is the epilogue of the GEMV (same bits)
                act = ops.gate_up_silu(xn, self.interleaved_gate_up()[l])
            else:
                gu_projs = (("gate_proj", 0, I), ("up_proj", I, I))
                # a prefill-sized pass: the SiLU product leaves the GEMM itself wherever no token needs a separate delta
                act = self._gate_up_silu(fuse, xn, L["gate_up"], l, gu_projs, bool(tok_adapter)) if frag and T > 64 else None
                if act is None:
                    gu = self._fused_linear(fuse, xn, L["gate_up"], l, gu_projs) if fuse else None
                    if gu is None:
                        gu = ops.linear(xn, L["gate_up"])
                        if tok_adapter:
                            self._lora_group(gu, xn, l, gu_projs, tok_adapter)
                    act = ops.silu_mul(gu, frag=frag)
            if fuse and self._fused_linear(fuse, act, L["down"], l, (("down_proj", 0, H),), resid=resid) is not None:
                parts = None
            else:
                parts = self._linear_acc(act, L["down"], resid, ks_ws, self._riding_rows(l, "down_proj", lora_tids, T, I))
                if tok_adapter:
                    self._lora(resid, act, l, "down_proj", tok_adapter)
        if logits_rows is not None:
            if parts is not None:                         # pending K-slice partials of the last down_proj, in slice order
                pv = parts.part[: (parts.ks - 1) * T * parts.ld].view(parts.ks - 1, T, parts.ld)
                for q in range(parts.ks - 1):
                    resid += pv[q, :, :H]
                parts = None
            resid = resid[logits_rows].contiguous()
        xn = ops.rmsnorm(resid, self.norm, s.rms_norm_eps, frag=resid.shape[0] <= 64 or frag, parts=parts)
        return ops.linear(xn, self.lm_head, out_dtype=torch.float32)

    def _fused_linear(self, fuse, x, W, l, projs, resid=None):
        """The base linear of `projs` = ((name, first row, rows), ...) with the adapter deltas as extra k-steps of the
        GEMM, then the separate gather-matmul for the tokens whose 256-token block mixes adapters.  resid: accumulate
        into it (o_proj, down_proj).  Returns None when the shape or the row ranges do not allow it."""
        lt, ids, blk, rest = fuse
        T, K = x.shape
        N = W.shape[0]
        live = [(proj, c0, n, lt.tables.get((l, proj))) for proj, c0, n in projs]
        live = [e for e in live if e[3] is not None]
        if not live or not ops.gemm_frag_preferred(T, K, N) or any(c0 % 256 or (n % 256 and c0 + n != N) for _, c0, n, _ in live):
            return None
        vs = ops.lora_shrink_split(x, [tab[0] for *_, tab in live], ids, lt.scaling, self._workspace(T, K, lt.r), out=self._v_split_bufs(T, lt.r)[:len(live)])
        fused = [(tab[1], vh, vl, c0, n) for (_, c0, n, tab), (vh, vl) in zip(live, vs)]
        if resid is not None:
            y = ops.linear_frag_lora(x, W, fused, blk, lt.r, out=resid, accumulate=True)
        else:
            y = ops.linear_frag_lora(x, W, fused, blk, lt.r)
        if rest is not None:
            if resid is not None:
                self._lora(y, x, l, projs[0][0], rest)
            else:
                self._lora_group(y, x, l, projs, rest)
        return y

    def _gate_up_silu(self, fuse, x, W, l, projs, adapters):
        """silu(gate) * up in fragment order out of the persistent GEMM of the fused gate/up projection: without
        adapters on these projections, or with their deltas as extra k-steps when every 256-token block of the pass
        agrees on one adapter.  Returns None where that does not apply (shape, a block that mixes adapters, a rank
        or a mix of adapter types that the extra k-steps do not take)."""
        T, K = x.shape
        N = W.shape[0]
        if not isinstance(x, ops.FragActivation) or not isinstance(W, ops.PackedWeight) or (N // 2) % 32 or not ops.gemm_frag_preferred(T, K, N):
            return None
        if not adapters or not self._targets(l, *(p for p, _, _ in projs)):
            return ops.linear_frag_silu(x, W)
        if fuse is None or fuse[3] is not None:
            return None
        lt, ids, blk, _ = fuse
        live = [(c0, n, lt.tables.get((l, proj))) for proj, c0, n in projs]
        live = [e for e in live if e[2] is not None]
        if not live:                                     # the tables belong to an adapter type that is not in this pass
            return ops.linear_frag_silu(x, W)
        vs = ops.lora_shrink_split(x, [tab[0] for *_, tab in live], ids, lt.scaling, self._workspace(T, K, lt.r), out=self._v_split_bufs(T, lt.r)[:len(live)])
        return ops.linear_frag_silu(x, W, [(tab[1], vh, vl, c0, n) for (c0, n, tab), (vh, vl) in zip(live, vs)], blk, lt.r)

    def _v_split_bufs(self, T, r):
        """fp16 hi / lo halves of the shrink results of up to three projections (reused from call to call)."""
        key = (T, r)
        if getattr(self, "_v_split_key", None) != key:
            self._v_split = [tuple(torch.empty((T, r), dtype=torch.float16, device=self.device) for _ in range(2)) for _ in range(3)]
            self._v_split_key = key
        return self._v_split

    def _ksplit_ws(self, T):
        """fp32 scratch for the K-split partials of o_proj / down_proj at T tokens (grown on demand, reused)."""
        s = self.shape
        need = 3 * T * s.hidden_size
        ws = getattr(self, "_ksplit_buf", None)
        if ws is None or ws.numel() < need:
            ws = self._ksplit_buf = torch.empty(need, dtype=torch.float32, device=self.device)
        return ws

    def _riding_rows(self, l, proj, tids, T, K):
        """What the shrink units of an adapted o_proj / down_proj weigh in the K-split rule of a decode step (the native
        step launches them with the GEMV; this path keeps the same slice count, hence the same sums).  tids: the
        adapter types of the pass."""
        if T > 64 or not any(self.lora_types[t].tables.get((l, proj)) is not None for t in tids):
            return 0
        return ops.lib().mlora_gemv_shrink_rows(K, 1, 1)

    @staticmethod
    def _linear_acc(x, W, resid, ks_ws, riding_rows=0):
        if isinstance(x, ops.FragActivation) and isinstance(W, ops.PackedWeight) and ks_ws is not None:
            return ops.linear_acc_ksplit(x, W, resid, ks_ws, riding_rows)
        ops.linear(x, W, out=resid, accumulate=True)
        return None

    # ------------------------------------------------------------------ reference entry points
    def _ids(self, T, pairs, host=False):
        """{tid: (positions | None, wids)} -> {tid: ids [T] int32 on device (host: numpy), -1 where the type is absent}."""
        out = {}
        for tid, (sids, wids) in pairs.items():
            full = np.full(T, -1, dtype=np.int32)
            w = self.lora_types[tid].rows(_host_i32(wids))      # -1 = no adapter for that row
            if sids is None:
                full[:] = np.broadcast_to(w, (T,)) if w.size in (1, T) else _bad(T, w)
            else:
                p = _host_i32(sids)
                if p.size != w.size or (p.size and (p.min() < 0 or p.max() >= T)):
                    raise ValueError("sids / wids mismatch")
                full[p] = w
            out[tid] = full if host else torch.from_numpy(full).to(self.device)
        return out

    def _last_rows(self, kv):
        lens = kv._cur[1]
        return torch.from_numpy(np.cumsum(lens).astype(np.int64) - 1).to(self.device)

    def prefill_no_adapter(self, h, kv):
        return self.forward(h, kv, None, self._last_rows(kv)), kv

    def decode_no_adapter(self, h, kv):
        return self.forward(h, kv, None), kv

    def prefill_a(self, tid, h, kv, wids):
        """Prefill of the sequences announced to kv.begin_forward; wids: one weight id per sequence
        (the reference prefills one sequence per call: wids [1])."""
        lens = kv._cur[1]
        w = np.repeat(_host_i32(wids), lens)
        return self.forward(h, kv, self._ids(h.shape[0], {tid: (None, w)}), self._last_rows(kv)), kv

    def decode_a(self, tid, h, kv, wids):
        return self.forward(h, kv, self._ids(h.shape[0], {tid: (None, wids)})), kv

    def mixed_decode(self, tids, h, kv, *params):
        """params = sids_i, wids_i, sids_j, wids_j, ... for the adapter types in `tids`
        (`compile_tvm.py:135-155`: rows `sids` of the batch use that type with weight ids `wids`)."""
        if len(params) != 2 * len(tids):
            raise ValueError(f"mixed decode over {len(tids)} adapter types needs {2 * len(tids)} id arrays")
        pairs = {tid: (params[2 * i], params[2 * i + 1]) for i, tid in enumerate(tids)}
        return self.forward(h, kv, self._ids(h.shape[0], pairs)), kv

    def __getitem__(self, name: str):
        """Entry points by the reference's VM function names."""
        if name in ("embed", "create_paged_kv_cache", "prefill_no_adapter", "decode_no_adapter"):
            return getattr(self, name)
        m = re.fullmatch(r"(prefill|decode)_a(\d+)", name)
        if m:
            tid = int(m.group(2))
            self._check_tid(tid)
            fn = self.prefill_a if m.group(1) == "prefill" else self.decode_a
            return lambda h, kv, wids: fn(tid, h, kv, wids)
        m = re.fullmatch(r"mixed_decode((?:_a\d+)+)", name)
        if m:
            tids = [int(t) for t in re.findall(r"_a(\d+)", m.group(1))]
            for t in tids:
                self._check_tid(t)
            return lambda h, kv, *params: self.mixed_decode(tids, h, kv, *params)
        raise KeyError(f"unknown entry point {name}")

    def _check_tid(self, tid):
        if not 0 <= tid < len(self.lora_types):
            raise KeyError(f"adapter type a{tid} not loaded")

    def weight_bytes_per_step(self):
        """Algorithmic fp16 weight bytes one decode step streams (all layers + lm_head)."""
        s = self.shape
        per_layer = sum(np.prod(linear_dims(s, p)) for p in LINEARS)
        return int(2 * (per_layer * s.num_hidden_layers + s.vocab_size * s.hidden_size))


def _host_i32(a):
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu().numpy()
    return np.asarray(a, dtype=np.int32).reshape(-1)


def _bad(T, w):
    raise ValueError(f"expected 1 or {T} weight ids, got {w.size}")
