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
    def __init__(self, model, kv, seq_ids, tok_adapter, first_tokens):
        """seq_ids: sequences already prefilled in `kv`; tok_adapter: {tid: ids [B] int32 (host)};
        first_tokens [B]: the tokens produced by prefill."""
        self.model, self.kv = model, kv
        self.seq_ids = list(seq_ids)
        B = len(self.seq_ids)
        dev = model.device
        self.tok_adapter = {tid: torch.as_tensor(np.asarray(ids, dtype=np.int32)).to(dev) for tid, ids in tok_adapter.items()}
        self.tokens = torch.as_tensor(np.asarray(first_tokens, dtype=np.int32)).to(dev)
        self.rows = torch.as_tensor(np.asarray([kv.slot[s] for s in self.seq_ids], dtype=np.int32)).to(dev)
        self.pos = torch.as_tensor(np.asarray([kv.lens[s] for s in self.seq_ids], dtype=np.int32)).to(dev)
        self.ctx = self.pos + 1
        self.history = []

    def step(self, keep_history=False):
        """One decode step for the whole batch; returns the device tensor of new token ids."""
        m, kv = self.model, self.kv
        hidden = m.embed(self.tokens)
        kv.begin_forward(self.seq_ids, [1] * len(self.seq_ids), device_meta=(self.rows, self.pos, self.ctx))
        logits = m.forward(hidden, kv, self.tok_adapter)
        kv.end_forward()
        nxt = ops.argmax(logits)
        self.tokens = nxt
        self.pos += 1
        self.ctx += 1
        if keep_history:
            self.history.append(nxt)
        return nxt
