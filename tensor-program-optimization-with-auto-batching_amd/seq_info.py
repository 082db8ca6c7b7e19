"""Per-sequence adapter bookkeeping and decode-method selection (integer host logic).

Restates `tvm/llama_auto_batcher/llama_seq_info.py:1-104`: adapter *types* are distinct `LoraConfig`s in
first-seen order; `order_seqs` is a stable sort by (has adapter, type id, weight id) so that sequences
without adapter come first; `get_decode_method` names the compiled entry point and builds the per-type
position / weight-id lists.
"""
from __future__ import annotations


class LlamaSeqInfo:
    def __init__(self, max_gen_len):
        self.sid_2_info = {}      # sid -> {"adapter": {"tid", "wid"} | None, "max_gen_len": int}
        self.adapter_types = []
        self.max_gen_len = max_gen_len

    def add_sequence(self, sid):
        assert sid not in self.sid_2_info, f"sequence with id {sid} has already been added"
        self.sid_2_info[sid] = {"adapter": None, "max_gen_len": self.max_gen_len}

    def set_max_gen_len(self, sid, max_gen_len):
        if max_gen_len is None:
            max_gen_len = self.max_gen_len
        if max_gen_len > self.max_gen_len:
            print(f"[WARN] you are trying to set a max_gen_len of {max_gen_len} for sequence {sid} which is bigger "
                  f"than the maximum {self.max_gen_len}. Setting max_gen_len to {self.max_gen_len}.")
            max_gen_len = self.max_gen_len
        self.sid_2_info[sid]["max_gen_len"] = max_gen_len

    def set_adapter(self, sid, config, wid):
        if config in self.adapter_types:
            tid = self.adapter_types.index(config)
        else:
            tid = len(self.adapter_types)
            self.adapter_types.append(config)
        adapter = {"tid": tid, "wid": int(wid)}
        prev = self.sid_2_info[sid]["adapter"]
        if prev is not None:
            print(f"[WARN] you are setting adapter {adapter} for sequence {sid} but it has already been set to {prev}")
        self.sid_2_info[sid]["adapter"] = adapter

    def get_adapter_configs(self):
        return self.adapter_types

    def get_wids_per_type(self):
        out = [set() for _ in self.adapter_types]
        for info in self.sid_2_info.values():
            if info["adapter"] is not None:
                out[info["adapter"]["tid"]].add(info["adapter"]["wid"])
        return out

    def get_num_adapters_per_type(self):
        return [len(s) for s in self.get_wids_per_type()]

    def get_num_sequences(self):
        return len(self.sid_2_info)

    def update_max_gen_len(self, max_gen_len):
        self.max_gen_len = max_gen_len

    def get_max_gen_len(self, sid):
        return self.sid_2_info[sid]["max_gen_len"]

    def get_adapter_info(self, sid):
        return self.sid_2_info[sid]["adapter"]

    def order_seqs(self, sids):
        """-> (ordered sids, original position of each ordered sid)."""
        if not self.adapter_types:
            return list(sids), list(range(len(sids)))
        inf = float("inf")

        def key(item):
            ad = self.sid_2_info[item[1]]["adapter"]
            return (ad is not None, ad["tid"] if ad else inf, ad["wid"] if ad else inf)

        ordered = sorted(enumerate(sids), key=key)      # sorted() is stable
        return [sid for _, sid in ordered], [pos for pos, _ in ordered]

    def get_decode_method(self, sids):
        """-> (entry-point name, parameter lists).  `decode_a{t}` takes [wids]; `mixed_decode_a{i}_a{j}...`
        takes [sids_i, wids_i, sids_j, wids_j, ...] where sids are positions inside this batch."""
        no_adapter = False
        a_sids = [[] for _ in self.adapter_types]
        a_wids = [[] for _ in self.adapter_types]
        for i, sid in enumerate(sids):
            ad = self.sid_2_info[sid]["adapter"]
            if ad is None:
                no_adapter = True
                continue
            a_sids[ad["tid"]].append(i)
            a_wids[ad["tid"]].append(ad["wid"])
        present = [t for t, lst in enumerate(a_sids) if lst]
        if no_adapter and not present:
            return "decode_no_adapter", []
        if not no_adapter and len(present) == 1:
            return f"decode_a{present[0]}", [a_wids[present[0]]]
        name = "mixed_decode_" + "_".join(f"a{t}" for t in present)
        params = []
        for t in present:
            params += [a_sids[t], a_wids[t]]
        return name, params
