"""MI355X-native multi-LoRA decode/prefill hot path: HIP kernels behind a C ABI, Python host on top.

Submodules: `ops` (operator surface over the C ABI), `lora` (LoraConfig, GatherMMLinear), `kv_cache`
(PagedKVCache), `llama` (LlamaForCausalLM with the reference's entry points), `seq_info`, `exec_graph`,
`llama_exec_graph`, `auto_batcher` (the auto-batching front end), `synth` (seeded synthetic inputs),
`build` (compiles libmlora_hip.so).  Importing the package does not load the library; the first operator
call does, and fails loudly if it has not been built.
"""
__all__ = ["ops", "lora", "kv_cache", "llama", "seq_info", "exec_graph", "llama_exec_graph", "auto_batcher",
           "synth", "build"]
