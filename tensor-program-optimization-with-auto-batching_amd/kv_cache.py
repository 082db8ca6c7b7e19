"""Paged KV cache: host-side page bookkeeping around the HIP attention kernels.

Keeps the host protocol of the reference's cache object
(`tvm/llama_auto_batcher/llama_exec_graph.py:41-46,66,75-79,85,121-127`):
    add_sequence(sid) ; begin_forward(seq_ids, append_lens) ; attention_with_fused_qkv(layer, qkv, n_q_heads) ;
    end_forward()
with RoPE applied inside the cache operator (`llama_for_causal_lm.py:148-174`: rotary_dim = head_dim,
scale 1, no sliding window).  Keys are stored already rotated, which is equivalent to rotating them at
read time and saves the per-step re-rotation of the whole context.

Device layout per layer: k [n_pages, Hkv, 16, D], v [n_pages, Hkv, D, 16] (fp16), one int32 block table
[max_seqs, max_blocks], fp32 RoPE tables [max_pos, D/2].
"""
from __future__ import annotations

import numpy as np
import torch

from . import ops

PAGE = 16


def rope_tables(head_dim: int, theta: float, max_pos: int):
    """cos/sin [max_pos, head_dim/2] float32 (float64 math, rounded once)."""
    inv_freq = theta ** (-(np.arange(0, head_dim, 2, dtype=np.float64) / head_dim))
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv_freq[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


class PagedKVCache:
    def __init__(self, n_layers, n_pages, n_kv_heads, head_dim, max_seqs, max_blocks, rope_theta, max_pos,
                 device="cuda:0", free_pages=None, page_size=PAGE):
        if page_size != PAGE:
            raise ValueError(f"page_size must be {PAGE}")
        self.n_layers, self.n_pages, self.Hkv, self.D = n_layers, n_pages, n_kv_heads, head_dim
        self.max_seqs, self.max_blocks, self.max_pos = max_seqs, max_blocks, max_pos
        self.device = torch.device(device)
        if head_dim % 32:
            raise ValueError("head_dim must be a multiple of 32")
        # keys in matrix-core fragment order: element (token, d) of a page at [d // 32, (d % 32) // 8, token, d % 8]
        self.k = torch.zeros((n_layers, n_pages, n_kv_heads, head_dim // 32, 4, PAGE, 8), dtype=torch.float16, device=self.device)
        self.v = torch.zeros((n_layers, n_pages, n_kv_heads, head_dim, PAGE), dtype=torch.float16, device=self.device)
        cos, sin = rope_tables(head_dim, rope_theta, max_pos)
        self.rope_cos = torch.from_numpy(cos).to(self.device)
        self.rope_sin = torch.from_numpy(sin).to(self.device)
        self.free = list(range(n_pages)) if free_pages is None else [int(p) for p in free_pages]
        if sorted(self.free) != list(range(n_pages)):
            raise ValueError("free_pages must be a permutation of range(n_pages)")
        # host mirrors (integer bookkeeping is host logic, as in the reference's runtime)
        self.table_h = np.full((max_seqs, max_blocks), -1, dtype=np.int32)
        self.lens = {}          # sid -> committed length
        self.slot = {}          # sid -> row of the block table
        self.block_table = torch.from_numpy(self.table_h.copy()).to(self.device)
        self._dirty = False
        self._cur = None

    def k_rowmajor(self, layer: int) -> torch.Tensor:
        """The layer's rotated keys as [n_pages, Hkv, 16, D] (a copy, for inspection)."""
        k = self.k[layer]
        return k.permute(0, 1, 4, 2, 3, 5).reshape(self.n_pages, self.Hkv, PAGE, self.D).contiguous()

    # ------------------------------------------------------------------ protocol
    def add_sequence(self, sid):
        if sid in self.slot:
            raise ValueError(f"sequence with id {sid} has already been added")
        if len(self.slot) >= self.max_seqs:
            raise RuntimeError("paged KV cache: no sequence slot left")
        self.slot[sid] = len(self.slot)
        self.lens[sid] = 0

    def begin_forward(self, seq_ids, append_lens, device_meta=None):
        """Reserve pages for the appended tokens and stage the per-token (sequence, position) arrays."""
        if self._cur is not None:
            raise RuntimeError("begin_forward called twice without end_forward")
        if len(seq_ids) != len(append_lens):
            raise ValueError("seq_ids and append_lens differ in length")
        for sid, n in zip(seq_ids, append_lens):
            row = self.slot[sid]
            new_len = self.lens[sid] + n
            if new_len > self.max_pos or -(-new_len // PAGE) > self.max_blocks:
                raise RuntimeError(f"sequence {sid}: length {new_len} exceeds the cache geometry")
            have = int((self.table_h[row] >= 0).sum())
            need = -(-new_len // PAGE)
            for j in range(have, need):
                if not self.free:
                    raise RuntimeError("paged KV cache out of pages")
                self.table_h[row, j] = self.free.pop(0)
                self._dirty = True
        if self._dirty:
            self.block_table.copy_(torch.from_numpy(self.table_h), non_blocking=False)
            self._dirty = False
        decode = all(n == 1 for n in append_lens)
        rows = np.asarray([self.slot[s] for s in seq_ids], dtype=np.int32)
        base = np.asarray([self.lens[s] for s in seq_ids], dtype=np.int32)
        if device_meta is not None:
            tok_seq, tok_pos, ctx = device_meta
        elif decode:
            tok_seq = torch.from_numpy(rows).to(self.device)
            tok_pos = torch.from_numpy(base).to(self.device)
            ctx = torch.from_numpy(base + 1).to(self.device)
        else:
            ts = np.repeat(rows, append_lens).astype(np.int32)
            tp = np.concatenate([b + np.arange(n, dtype=np.int32) for b, n in zip(base, append_lens)]).astype(np.int32)
            tok_seq = torch.from_numpy(ts).to(self.device)
            tok_pos = torch.from_numpy(tp).to(self.device)
            ctx = None
        self._cur = (list(seq_ids), list(append_lens), decode, tok_seq, tok_pos, ctx)

    def attention_with_fused_qkv(self, layer, qkv, n_q_heads, out=None, frag=False, o_shrink=None):
        """qkv [T, Hq + 2 Hkv, D] (or [T, (Hq + 2 Hkv) * D]) fp16, token-major in begin_forward order.
        Rotates q in place, appends rotated k and v, attends causally; returns [T, Hq * D] fp16
        (frag=True: as a FragActivation ready for the o_proj product).  o_shrink (a decode step only): see
        ops.paged_attn_decode - the call then returns (attention output, head shares of the o projection's shrink)."""
        if self._cur is None:
            raise RuntimeError("attention_with_fused_qkv outside begin_forward/end_forward")
        _, append_lens, decode, tok_seq, tok_pos, ctx = self._cur
        T = sum(append_lens)
        qkv = qkv.view(T, n_q_heads + 2 * self.Hkv, self.D)
        ops.rope_kv_append(qkv, self.k[layer], self.v[layer], self.block_table, tok_seq, tok_pos,
                           self.rope_cos, self.rope_sin, n_q_heads, self.Hkv, self.D)
        if decode:
            return ops.paged_attn_decode(qkv, self.k[layer], self.v[layer], self.block_table, tok_seq, ctx,
                                         n_q_heads, self.Hkv, self.D, out=out, frag=frag, o_shrink=o_shrink)
        if o_shrink is not None:
            raise ValueError("attention_with_fused_qkv: o_shrink is for decode steps")
        return ops.paged_attn_prefill(qkv, self.k[layer], self.v[layer], self.block_table, tok_seq, tok_pos,
                                      n_q_heads, self.Hkv, self.D, out=out, frag=frag)

    def end_forward(self):
        seq_ids, append_lens = self._cur[0], self._cur[1]
        for sid, n in zip(seq_ids, append_lens):
            self.lens[sid] += n
        self._cur = None

    # ------------------------------------------------------------------ helpers
    def pages_of(self, sid):
        row = self.table_h[self.slot[sid]]
        return row[row >= 0].tolist()

    def kv_bytes_read_per_step(self, seq_ids):
        """Algorithmic K+V bytes one decode step reads for these sequences, all layers."""
        per_pos = self.n_layers * 2 * self.Hkv * self.D * 2
        return int(sum(self.lens[s] + 1 for s in seq_ids)) * per_pos
