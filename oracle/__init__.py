"""CPU oracle for the multi-LoRA decode/prefill hot path.

TEST INFRASTRUCTURE ONLY.  This package is a numpy restatement of the reference's
algorithms, used as the checker by `tests/`, by `__graft_entry__.smoke()` and by the
`cpu_baseline` leg of `bench.py`.  The product (the HIP library and the Python host
around it) never imports it and has no CPU fallback.

The reference cannot be imported in this environment (it needs `peft` and `tvm`, which
are not installed, and fetches model files by name), and it ships no golden vectors,
so every function here is pinned by checks that the mathematics fixes (see
`tests/test_oracle_*.py`): per-token brute force in float64, equivalence of the
reference's own batching strategies (`tvm/lora_only/single_rank.py:254`,
`tvm/lora_only/case_study/multiple_ranks.py:382-383`), dense-library special cases,
invariance under page permutation, cache-vs-recompute identity, and enumeration of the
integer host logic on the request mix of `tvm/llama_auto_batcher/user_example.py:7-39`.

Parity unpinned (third-party code that is neither vendored nor installed, so nothing in
the reference pins it): PEFT `_mixed_batch_forward` accumulation order, HF `generate`
EOS/pad handling, TVM `PagedKVCache` page-allocation order and its attention
accumulation order.  The oracle defines those by the published algorithm (causal
softmax attention, rotate-half RoPE) and documents its own page allocator.
"""
from .lora_ref import (  # noqa: F401
    gather_mm_ref, gather_bmm_hf_ref, lora_sequential_ref, take_matmul_ref,
    write_tensor_part_ref, mixed_delta_ref, max_rel_err, combined_tables_ref, lora_combined_ref,
)
from .llama_ref import (  # noqa: F401
    rmsnorm_ref, rope_tables, rope_ref, silu_mul_ref, PagedKVRef, attention_dense_ref,
    LlamaRef, greedy_generate_ref, f16,
)
