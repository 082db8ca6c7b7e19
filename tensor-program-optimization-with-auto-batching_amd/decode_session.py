"""A fixed batch of sequences decoding greedily with no host round trip per step.

The reference's loop copies the logits to the host, takes np.argmax there and uploads the next tokens
(`tvm/llama_auto_batcher/llama_exec_graph.py:110-137`).  Here the argmax output stays on the device and
feeds the next embedding lookup; positions and context lengths are device counters; the host only does
the integer page bookkeeping (a new page every 16 steps per sequence).
"""
from __future__ import annotations

import numpy as np
import torch

from . import ops


class DecodeSession:
    """Fixed-batch greedy decode through the per-operator path (any mix of adapter types and ranks).  With
    use_graph the launch sequence of a step is captured once - after one eager step, which also sizes the model's
    scratch buffers outside the graph's memory pool - and replayed, so the interpreter is out of the loop; the
    kernels and their order are those of the eager step, hence the same tokens bit for bit."""

    def __init__(self, model, kv, seq_ids, tok_adapter, first_tokens, use_graph=False, longest_first=False):
        """seq_ids: sequences already prefilled in `kv`; tok_adapter: {tid: ids [B] int32 (host or device), -1 = the
        row does not use that type}; first_tokens [B]: the tokens produced by prefill.
        longest_first: run the batch internally in order of decreasing context length, so that the attention
        workgroups of the longest sequences start first and the short ones fill the tail of the launch (every
        operator treats rows independently: a sequence's results do not depend on its row); step() still returns
        the tokens in the caller's order."""
        self.model, self.kv = model, kv
        B = len(seq_ids)
        dev = model.device
        i32 = lambda a: (a if isinstance(a, torch.Tensor) else torch.as_tensor(np.asarray(a, dtype=np.int32))).to(dev, torch.int32)
        self._inv = None
        if longest_first and B > 1:
            order = np.argsort(-np.asarray([kv.lens[s] for s in seq_ids], dtype=np.int64), kind="stable")
            od = torch.from_numpy(order).to(dev)
            seq_ids = [seq_ids[i] for i in order]
            tok_adapter = {tid: i32(ids).index_select(0, od) for tid, ids in tok_adapter.items()}
            first_tokens = i32(first_tokens).index_select(0, od)
            self._inv = torch.from_numpy(np.argsort(order)).to(dev)
        self.seq_ids = list(seq_ids)
        self.tok_adapter = {tid: i32(ids) for tid, ids in tok_adapter.items()}
        if len(self.tok_adapter) > 1:         # several adapter types: merged once here (the check reads back to the host)
            self.tok_adapter = model._merge_types(self.tok_adapter)
        self.tokens = i32(first_tokens).clone()
        self.rows = i32([kv.slot[s] for s in self.seq_ids])
        self.pos = i32([kv.lens[s] for s in self.seq_ids])
        self.ctx = self.pos + 1
        self.use_graph = use_graph
        self.graph = None
        self._eager_steps = 0
        self.history = []

    def _enqueue(self):
        m = self.model
        logits = m.forward(m.embed(self.tokens), self.kv, self.tok_adapter)
        self.tokens.copy_(ops.argmax(logits))
        self.pos.add_(1)
        self.ctx.add_(1)

    def step(self, keep_history=False):
        """One decode step for the whole batch; returns the device tensor of new token ids (updated in place)."""
        kv = self.kv
        kv.begin_forward(self.seq_ids, [1] * len(self.seq_ids), device_meta=(self.rows, self.pos, self.ctx))
        if self.use_graph and self._eager_steps >= 1:
            if self.graph is None:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):         # records, does not run
                    self._enqueue()
                self.graph = g
            self.graph.replay()
        else:
            self._enqueue()
            self._eager_steps += 1
        kv.end_forward()
        out = self.tokens if self._inv is None else self.tokens.index_select(0, self._inv)
        if keep_history:
            self.history.append(out.clone() if self._inv is None else out)
        return out


class NativeDecodeSession:
    """The same fixed-batch greedy decode, one `mlora_decode_step` call per step, optionally replayed from a
    captured graph.  The graph is re-used as long as the batch does not change; the host only grows the block table
    when a sequence crosses a page boundary.  `tid` names one adapter type (`adapter_ids` = weight ids, -1 = none) or,
    as a tuple, several types of equal scaling served from their padded union (`adapter_ids` = rows of
    `model.lora_union(tid)`, see `model.union_rows`)."""

    def __init__(self, model, kv, seq_ids, adapter_ids, first_tokens, tid=0, use_graph=True, dense_lora=None, fuse_silu=True, ksplit=True,
                 longest_first=False):
        """longest_first: as in DecodeSession - the batch runs internally in order of decreasing context length and
        step() returns the tokens in the caller's order (`tokens` and `buf` stay in the internal order)."""
        import ctypes as C
        from . import _lib
        self.model, self.kv = model, kv
        self.seq_ids = list(seq_ids)
        s = model.shape
        dev = model.device
        T = len(self.seq_ids)
        self._inv = None
        if longest_first and T > 1:
            order = np.argsort(-np.asarray([kv.lens[q] for q in self.seq_ids], dtype=np.int64), kind="stable")
            self.seq_ids = [self.seq_ids[i] for i in order]
            if adapter_ids is not None:
                adapter_ids = np.asarray(adapter_ids, dtype=np.int32).reshape(-1)[order]
            first_tokens = torch.as_tensor(first_tokens).cpu().numpy().reshape(-1)[order]
            self._inv = torch.from_numpy(np.argsort(order)).to(dev)
        lt = None
        if adapter_ids is not None and model.lora_types:
            lt = model.lora_union(tid)[0] if isinstance(tid, tuple) else model.lora_types[tid]
        i32 = lambda a: torch.as_tensor(np.asarray(a, dtype=np.int32)).to(dev)
        self.tokens = i32(first_tokens)
        self.rows = i32([kv.slot[q] for q in self.seq_ids])
        self.pos = i32([kv.lens[q] for q in self.seq_ids])
        self.ctx = self.pos + 1
        self.tok_adapter = None
        if lt is not None:
            ids = np.asarray(adapter_ids, dtype=np.int32).reshape(-1)
            if not isinstance(tid, tuple):
                ids = lt.rows(ids)                       # weight ids -> table rows
            elif ids.size != T or (ids.size and (ids.min() < -1 or ids.max() >= lt.n_adapters)):
                raise ValueError("NativeDecodeSession: bad union rows")
            self.tok_adapter = i32(ids)
        H, I, V = s.hidden_size, s.intermediate_size, s.vocab_size
        f16, f32 = torch.float16, torch.float32
        fe = _lib.lib().mlora_frag_activation_elems
        self.buf = {
            "resid": torch.empty(T * H, dtype=f32, device=dev), "xn": torch.empty(fe(T, H), dtype=f16, device=dev),
            "qkv": torch.empty(T * (s.q_size + 2 * s.kv_size), dtype=f16, device=dev),
            "attn": torch.empty(fe(T, s.q_size), dtype=f16, device=dev),
            "gate_up": torch.empty(T * 2 * I, dtype=f16, device=dev), "act": torch.empty(fe(T, I), dtype=f16, device=dev),
            "logits": torch.empty(T * V, dtype=f32, device=dev),
        }
        r = lt.r if lt is not None else 0
        # five slots (q, k, v, o, down); the dense q/k/v shrink may come as up to four K-range blocks of three slots
        # (a slot also holds the o shrink's head shares, [heads, T, r] fp32)
        ws_bytes = 14 * max(_lib.lib().mlora_gather_mm_workspace_bytes(T, max(H, I, s.q_size), max(r, 8)),
                            4 * T * (lt.n_adapters if lt is not None else 0) * max(r, 8), 4 * s.num_attention_heads * T * max(r, 8))
        self.buf["lora_ws"] = torch.empty(ws_bytes // 4, dtype=f32, device=dev)
        # partials of the K-split o_proj / down_proj GEMVs (up to 3 slices of [T, H + appended adapter rows])
        ks_elems = 3 * T * (H + (lt.n_adapters * r if lt is not None else 0)) if ksplit else 0
        self.buf["ksplit_ws"] = torch.empty(max(ks_elems, 1), dtype=f32, device=dev)
        layers = (_lib.Layer * s.num_hidden_layers)()
        order = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")
        # Dense shrink: the stacked A tables become extra weight rows of the base GEMV.  Worth it while the tables
        # are small next to the base weight and most adapters are in use (the extra rows are read whether or not
        # an adapter has a token in the batch).
        if dense_lora is None:
            dense_lora = lt is not None and lt.n_adapters <= 2 * T and T <= 64
        if dense_lora and T > 64:
            raise ValueError("NativeDecodeSession: the dense shrink serves at most 64 sequences per step")
        self.dense_lora = bool(dense_lora and lt is not None)
        # the o projection without appended rows: the attention launch writes its shrink as one share per head and riders
        # of the o GEMV launch expand it (base weight alone, no table for the norm to stream) - where the library serves
        # the shape that way and there is room for the delta rows behind the slice partials
        ks_ride = _lib.lib().mlora_gemv_delta_ride_ksplit(T, s.q_size, H, r) if (self.dense_lora and ksplit) else 0
        self.o_delta_ride = bool(ks_ride > 0 and 4 * ks_elems >= _lib.lib().mlora_gemv_ksplit_bytes(T, H, ks_ride + 1) and
                                 _lib.lib().mlora_rope_attn_oshrink_ok(T, s.num_attention_heads, s.num_key_value_heads, s.head_dim, r))
        ext = model.dense_lora_weights(tid, with_o=not self.o_delta_ride) if self.dense_lora else None
        il = model.interleaved_gate_up() if (fuse_silu and s.intermediate_size % 32 == 0) else None
        for l, L in enumerate(model.layers):
            if il is not None:
                layers[l].gate_up_il_p = il[l].data.data_ptr()
            W = ext[l] if ext is not None else L
            layers[l].qkv_p, layers[l].o_p = W["qkv"].data.data_ptr(), W["o"].data.data_ptr()
            layers[l].gate_up_p, layers[l].down_p = L["gate_up"].data.data_ptr(), W["down"].data.data_ptr()
            layers[l].ln1, layers[l].ln2 = L["ln1"].data_ptr(), L["ln2"].data_ptr()
            layers[l].k_cache, layers[l].v_cache = kv.k[l].data_ptr(), kv.v[l].data_ptr()
            for j, proj in enumerate(order):
                tab = lt.tables.get((l, proj)) if lt is not None else None
                if tab is not None:
                    layers[l].lora[j].A, layers[l].lora[j].B = tab[0].data_ptr(), tab[1].data_ptr()
        p = _lib.DecodePlan()
        p.n_layers, p.hidden, p.inter = s.num_hidden_layers, H, I
        p.n_q_heads, p.n_kv_heads, p.head_dim, p.vocab, p.eps = s.num_attention_heads, s.num_key_value_heads, s.head_dim, V, s.rms_norm_eps
        if lt is not None:
            p.lora_r, p.lora_n_ad, p.lora_scaling = lt.r, lt.n_adapters, lt.scaling
            p.lora_dense = (2 if self.o_delta_ride else 1) if self.dense_lora else 0
        p.layers = C.cast(layers, C.POINTER(_lib.Layer))
        p.embed, p.norm, p.lm_head_p = model.embed_tokens.data_ptr(), model.norm.data_ptr(), model.lm_head.data.data_ptr()
        p.rope_cos, p.rope_sin, p.max_pos = kv.rope_cos.data_ptr(), kv.rope_sin.data_ptr(), kv.max_pos
        p.block_table, p.max_blocks, p.n_pages, p.n_seq = kv.block_table.data_ptr(), kv.max_blocks, kv.n_pages, kv.max_seqs
        p.T = T
        p.tokens, p.rows, p.pos, p.ctx = self.tokens.data_ptr(), self.rows.data_ptr(), self.pos.data_ptr(), self.ctx.data_ptr()
        p.tok_adapter = self.tok_adapter.data_ptr() if self.tok_adapter is not None else None
        for k in ("resid", "xn", "qkv", "attn", "gate_up", "act", "logits", "lora_ws"):
            setattr(p, k, self.buf[k].data_ptr())
        p.lora_ws_bytes = ws_bytes
        if ksplit:
            p.ksplit_ws, p.ksplit_ws_bytes = self.buf["ksplit_ws"].data_ptr(), 4 * ks_elems
        self._layers, self.plan = layers, p
        self._lib = _lib
        self.use_graph = use_graph
        self.graph = None
        self.history = []

    def _enqueue(self):
        import ctypes as C
        self._lib.check(self._lib.lib().mlora_decode_step(C.byref(self.plan), torch.cuda.current_stream().cuda_stream))

    def step(self, keep_history=False):
        kv = self.kv
        # integer page bookkeeping on the host; copies the block table only when a page was added
        kv.begin_forward(self.seq_ids, [1] * len(self.seq_ids), device_meta=(self.rows, self.pos, self.ctx))
        if self.use_graph:
            if self.graph is None:
                # warm-up launch outside capture is not needed: kernels are plain launches; capture directly
                g = torch.cuda.CUDAGraph()
                snap = (self.tokens.clone(), self.pos.clone(), self.ctx.clone())
                with torch.cuda.graph(g):
                    self._enqueue()
                # capture does not execute: restore nothing, just replay once for this step
                self.tokens.copy_(snap[0]); self.pos.copy_(snap[1]); self.ctx.copy_(snap[2])
                self.graph = g
            self.graph.replay()
        else:
            self._enqueue()
        kv.end_forward()
        out = self.tokens if self._inv is None else self.tokens.index_select(0, self._inv)
        if keep_history:
            self.history.append(out.clone() if self._inv is None else out)
        return out
