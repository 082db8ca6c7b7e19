"""The user-facing front end of auto-batching: requests are written one after the other as if each ran alone
(`create_var`, optionally `set_adapter`, `generate`, `print`), `compile()` folds their decode loops into one batched
loop, `execute()` runs the graph.

Same calls and semantics as `tvm/llama_auto_batcher/llama_auto_batcher.py:11-138`.  The reference object is a
module-level singleton that fetches a tokenizer and Llama-3.1-8B by name when imported and compiles a TVM module in
`compile()`; here the model is handed in with `set_model`, nothing is fetched, and `compile()` has nothing to build:
it fuses the graph, checks that the adapter types the requests name are loaded, and binds model and configuration.
"""
from __future__ import annotations

from .llama_exec_graph import LlamaExecConfig, LlamaExecGraph
from .seq_info import LlamaSeqInfo

# the operations one generate() appends, in order; each reads the previous one's output variable
_REQUEST_CHAIN = ("encode_prompt", "prefill", "decode", "decode_answer")


class LlamaAutoBatcherClass:
    def __init__(self):
        self.exec_config = LlamaExecConfig(max_prompt_len=512, max_gen_len=32, page_size=16)
        self.graph = LlamaExecGraph()
        self.seq_info = LlamaSeqInfo(self.exec_config.max_gen_len)
        self.model = self.tokenizer = self.eos_token_id = self.free_pages = None
        # a request's sequence id is claimed by its first set_adapter() or generate(); `_open` says that the newest
        # id has been claimed by set_adapter() and still waits for its generate()
        self._last_sid = -1
        self._open = False
        self.warmup_trials, self.measurement_trials, self.measurements_dest = 3, 0, "measure.txt"

    # ------------------------------------------------------------------ configuration
    def set_model(self, model):
        self.model = model

    def set_tokenizer(self, tokenizer):
        self.tokenizer = tokenizer

    def set_eos_token_id(self, eos_token_id):
        self.eos_token_id = eos_token_id

    def set_free_pages(self, free_pages):
        self.free_pages = free_pages

    def set_exec_config(self, exec_config):
        self.exec_config = exec_config
        self.seq_info.update_max_gen_len(exec_config.max_gen_len)

    def set_measurement_vars(self, trials, dest, warmup_trials=3):
        """Run the graph `warmup_trials` times untimed, then `trials` times writing one step time (ms) per line to `dest`."""
        self.warmup_trials, self.measurement_trials, self.measurements_dest = warmup_trials, trials, dest

    # ------------------------------------------------------------------ writing requests
    def _claim_sid(self) -> int:
        if not self._open:
            self._last_sid += 1
            self.seq_info.add_sequence(self._last_sid)
        return self._last_sid

    def create_var(self, var, source=True):
        return self.graph.variable(var, source)

    def set_adapter(self, config, wid):
        """The adapter of the request whose generate() comes next."""
        sid = self._claim_sid()
        self._open = True
        self.seq_info.set_adapter(sid, config, wid)

    def generate(self, input_var, max_gen_len=None):
        sid = self._claim_sid()
        self._open = False
        self.seq_info.set_max_gen_len(sid, max_gen_len)
        var = input_var
        for op_type in _REQUEST_CHAIN:
            out = self.create_var(None, False)
            self.graph.operation(var, op_type, seqid=sid, output_var=out)
            var = out
        return var

    def print(self, var):
        self.graph.operation(var, "print", seqid=self._last_sid)

    # ------------------------------------------------------------------ running
    def load_adapters(self, cache_dir):
        """Load the adapter types the registered requests use from `{cache_dir}/lora_adapters/r{rank}_a{wid}.safetensors`
        (`compile_tvm.py:296-314`); call after the requests are registered and before compile()."""
        from .adapter_files import load_adapters_for
        if self.model is None:
            raise RuntimeError("set_model() must be called before load_adapters()")
        load_adapters_for(self.seq_info, self.model, cache_dir)

    def compile(self, fuse_decode=True):
        if self.model is None:
            raise RuntimeError("set_model() must be called before compile()")
        loaded = self.model.lora_types
        for tid, cfg in enumerate(self.seq_info.get_adapter_configs()):
            ok = tid < len(loaded) and loaded[tid].r == cfg.r and abs(loaded[tid].scaling - cfg.alpha / cfg.r) <= 1e-12
            if not ok:
                raise RuntimeError(f"adapter type a{tid} ({cfg}) is not loaded in the model")
        if fuse_decode:
            if getattr(self.exec_config, "batch_prefill", False) and "prefill" not in self.graph.batchable_op_types:
                self.graph.batchable_op_types += ("prefill",)
            self.graph.fuse_batchable_ops()
        self.graph.set_exec_vars(self.model, self.model.device, None, self.tokenizer, self.seq_info,
                                 self.exec_config, eos_token_id=self.eos_token_id, free_pages=self.free_pages)

    def execute(self):
        if not self.measurement_trials:
            self.graph.execute()
            return
        for trial in range(self.warmup_trials + self.measurement_trials):
            if trial == self.warmup_trials:
                self.graph.set_measuring(self.measurements_dest)
            if trial > 0:
                self.graph.set_kv_cache()            # every pass after the first starts from an empty cache
            self.graph.execute()
