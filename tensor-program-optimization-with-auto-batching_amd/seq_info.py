"""What the front end knows about each request: its adapter (type and weight id) and its generation limit; and,
from that, the order of a decode batch and the entry point that serves it.  Integer host logic only.

Behaviour of `tvm/llama_auto_batcher/llama_seq_info.py:1-104`:
  * an adapter *type* is a distinct `LoraConfig` (rank, alpha); types are numbered in the order they are first seen;
  * a decode batch is ordered by (has an adapter, type, weight id), stably, so adapter-less requests come first and
    the rows of one type are contiguous;
  * the entry point is `decode_no_adapter`, `decode_a{t}` (one type, every row adapted: parameter = weight ids) or
    `mixed_decode_a{i}_a{j}...` (parameters per present type: row positions inside the batch, weight ids).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple


@dataclass
class _Request:
    max_gen_len: int
    tid: Optional[int] = None     # adapter type, None = no adapter
    wid: Optional[int] = None     # weight id inside the type


class LlamaSeqInfo:
    def __init__(self, max_gen_len: int):
        self.max_gen_len = max_gen_len
        self._requests: Dict[int, _Request] = {}
        self._types: list = []                    # LoraConfig of type t at index t

    # ------------------------------------------------------------------ registration
    def add_sequence(self, sid: int) -> None:
        assert sid not in self._requests, f"sequence with id {sid} has already been added"
        self._requests[sid] = _Request(self.max_gen_len)

    def update_max_gen_len(self, max_gen_len: int) -> None:
        self.max_gen_len = max_gen_len

    def set_max_gen_len(self, sid: int, max_gen_len: Optional[int]) -> None:
        """Per-request limit, clipped to the global one (None = the global one)."""
        limit = self.max_gen_len if max_gen_len is None else max_gen_len
        if limit > self.max_gen_len:
            print(f"[WARN] max_gen_len {limit} requested for sequence {sid} exceeds the maximum {self.max_gen_len}; "
                  f"using {self.max_gen_len}.")
            limit = self.max_gen_len
        self._requests[sid].max_gen_len = limit

    def set_adapter(self, sid: int, config, wid: int) -> None:
        try:
            tid = self._types.index(config)
        except ValueError:
            tid = len(self._types)
            self._types.append(config)
        req = self._requests[sid]
        if req.tid is not None:
            print(f"[WARN] sequence {sid} already has adapter {self.get_adapter_info(sid)}; replacing it with "
                  f"{{'tid': {tid}, 'wid': {int(wid)}}}")
        req.tid, req.wid = tid, int(wid)

    # ------------------------------------------------------------------ queries
    def get_num_sequences(self) -> int:
        return len(self._requests)

    def get_max_gen_len(self, sid: int) -> int:
        return self._requests[sid].max_gen_len

    def get_adapter_info(self, sid: int) -> Optional[dict]:
        req = self._requests[sid]
        return None if req.tid is None else {"tid": req.tid, "wid": req.wid}

    def get_adapter_configs(self) -> list:
        return self._types

    def get_wids_per_type(self) -> List[set]:
        """The weight ids in use, per adapter type."""
        used: List[set] = [set() for _ in self._types]
        for req in self._requests.values():
            if req.tid is not None:
                used[req.tid].add(req.wid)
        return used

    def get_num_adapters_per_type(self) -> List[int]:
        return [len(w) for w in self.get_wids_per_type()]

    # ------------------------------------------------------------------ batch order and entry point
    def order_seqs(self, sids: Sequence[int]) -> Tuple[List[int], List[int]]:
        """-> (the sequence ids in batch order, for each of them its position in `sids`)."""
        positions = list(range(len(sids)))
        if self._types:
            def rank(pos: int):
                req = self._requests[sids[pos]]
                return (0, 0, 0) if req.tid is None else (1, req.tid, req.wid)
            positions.sort(key=rank)                  # list.sort is stable: ties keep the caller's order
        return [sids[p] for p in positions], positions

    def get_decode_method(self, sids: Sequence[int]) -> Tuple[str, list]:
        """-> (entry-point name, parameter lists) for a batch whose rows are `sids` in this order."""
        rows_of: Dict[int, List[int]] = {}            # type -> rows of the batch that use it
        bare = 0
        for row, sid in enumerate(sids):
            tid = self._requests[sid].tid
            if tid is None:
                bare += 1
            else:
                rows_of.setdefault(tid, []).append(row)
        present = sorted(rows_of)
        wids = {t: [self._requests[sids[row]].wid for row in rows_of[t]] for t in present}
        if not present:
            return "decode_no_adapter", []
        if len(present) == 1 and bare == 0:
            return f"decode_a{present[0]}", [wids[present[0]]]
        params: list = []
        for t in present:
            params.extend((rows_of[t], wids[t]))
        return "mixed_decode_" + "_".join(f"a{t}" for t in present), params
