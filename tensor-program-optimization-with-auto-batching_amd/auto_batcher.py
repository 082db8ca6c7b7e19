"""User-facing auto-batching front end: create_var / set_adapter / generate / print / compile / execute.

Restates `tvm/llama_auto_batcher/llama_auto_batcher.py:11-138`.  The reference object is a module-level
singleton that loads a tokenizer and Llama-3.1-8B weights by name at import; here the model is handed in
(`set_model`), and `compile()` only fuses the graph and binds the model - there is nothing to compile.
"""
from __future__ import annotations

from .llama_exec_graph import LlamaExecConfig, LlamaExecGraph
from .seq_info import LlamaSeqInfo


class LlamaAutoBatcherClass:
    def __init__(self):
        self.graph = LlamaExecGraph()
        self.current = {"sid": -1, "generated": True}
        self.model = None
        self.tokenizer = None
        self.eos_token_id = None
        self.free_pages = None
        self.exec_config = LlamaExecConfig(max_prompt_len=512, max_gen_len=32, page_size=16)
        self.seq_info = LlamaSeqInfo(self.exec_config.max_gen_len)
        self.warmup_trials = 3
        self.measurement_trials = 0
        self.measurements_dest = "measure.txt"

    def set_model(self, model):
        self.model = model

    def set_tokenizer(self, tokenizer):
        self.tokenizer = tokenizer

    def set_eos_token_id(self, eos_token_id):
        self.eos_token_id = eos_token_id

    def set_free_pages(self, free_pages):
        self.free_pages = free_pages

    def set_exec_config(self, exec_config):
        self.seq_info.update_max_gen_len(exec_config.max_gen_len)
        self.exec_config = exec_config

    def set_measurement_vars(self, trials, dest, warmup_trials=3):
        self.measurement_trials = trials
        self.measurements_dest = dest
        self.warmup_trials = warmup_trials

    def create_var(self, var, source=True):
        return self.graph.variable(var, source)

    def _new_sequence_if_needed(self):
        if self.current["generated"]:
            self.current["sid"] += 1
            self.seq_info.add_sequence(self.current["sid"])

    def generate(self, input_var, max_gen_len=None):
        self._new_sequence_if_needed()
        self.current["generated"] = True
        sid = self.current["sid"]
        self.seq_info.set_max_gen_len(sid, max_gen_len)
        enc = self.create_var(None, False)
        self.graph.operation(input_var, "encode_prompt", seqid=sid, output_var=enc)
        pre = self.create_var(None, False)
        self.graph.operation(enc, "prefill", seqid=sid, output_var=pre)
        dec = self.create_var(None, False)
        self.graph.operation(pre, "decode", seqid=sid, output_var=dec)
        ans = self.create_var(None, False)
        self.graph.operation(dec, "decode_answer", seqid=sid, output_var=ans)
        return ans

    def print(self, var):
        self.graph.operation(var, "print", seqid=self.current["sid"])

    def set_adapter(self, config, wid):
        if self.current["generated"]:
            self.current["sid"] += 1
            self.seq_info.add_sequence(self.current["sid"])
            self.current["generated"] = False
        self.seq_info.set_adapter(self.current["sid"], config, wid)

    def load_adapters(self, cache_dir):
        """Load the adapter types the registered requests use from `{cache_dir}/lora_adapters/r{rank}_a{wid}.safetensors`
        (`compile_tvm.py:296-314`); call after the requests are registered and before compile()."""
        from .adapter_files import load_adapters_for
        if self.model is None:
            raise RuntimeError("set_model() must be called before load_adapters()")
        load_adapters_for(self.seq_info, self.model, cache_dir)

    def compile(self, fuse_decode=True):
        if fuse_decode:
            self.graph.fuse_batchable_ops()
        if self.model is None:
            raise RuntimeError("set_model() must be called before compile()")
        for tid, cfg in enumerate(self.seq_info.get_adapter_configs()):
            if tid >= len(self.model.lora_types) or self.model.lora_types[tid].r != cfg.r or \
                    abs(self.model.lora_types[tid].scaling - cfg.alpha / cfg.r) > 1e-12:
                raise RuntimeError(f"adapter type a{tid} ({cfg}) is not loaded in the model")
        self.graph.set_exec_vars(self.model, self.model.device, None, self.tokenizer, self.seq_info,
                                 self.exec_config, eos_token_id=self.eos_token_id, free_pages=self.free_pages)

    def execute(self):
        if self.measurement_trials:
            for i in range(self.warmup_trials):
                if i != 0:
                    self.graph.set_kv_cache()
                self.graph.execute()
            self.graph.set_measuring(self.measurements_dest)
            for _ in range(self.measurement_trials):
                self.graph.set_kv_cache()
                self.graph.execute()
        else:
            self.graph.execute()
