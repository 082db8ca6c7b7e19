"""Shared test helpers: build the CPU oracle and the HIP model from the same seeded synthetic weights."""
import numpy as np
import torch

import oracle
from conftest import load_pkg


def oracle_model(wl, mode="mixed", lora_specs=None):
    """LlamaRef on CPU-generated weights (bit-identical to the device generation of the same seed)."""
    synth = load_pkg("synth")
    specs = [wl.lora] if lora_specs is None else lora_specs
    w = {k: v.float().numpy() for k, v in synth.base_weights(wl.seed, wl.shape, torch.float16, "cpu").items()}
    lora, scaling = {}, {}
    for tid, spec in enumerate(specs):
        lw = synth.lora_weights(wl.seed, wl.shape, spec, torch.float16, "cpu", tag=f"a{tid}")
        lora.update({k: v.float().numpy() for k, v in lw.items()})
        scaling[f"a{tid}"] = spec.scaling
    return oracle.LlamaRef(wl.shape, w, lora, scaling, mode=mode)


def hip_model(wl, lora_specs=None, device="cuda:0"):
    llama = load_pkg("llama")
    specs = [wl.lora] if lora_specs is None else lora_specs
    return llama.LlamaForCausalLM.from_synthetic(wl.seed, wl.shape, specs, device)


def n_pages_for(wl, max_gen_len):
    return wl.batch * (-(-(wl.prompt_len + max_gen_len) // wl.page_size) + 1)


def run_hip_generate(model, wl, prompts, adapter_ids, max_gen_len, free_pages, tids=None, max_gen_lens=None,
                     eos_token_id=None, native_decode=True, dense_lora=False, batch_prefill=False):
    """Drive the auto-batching front end the way `tvm/llama_auto_batcher/main.py:37-44` does."""
    ab = load_pkg("auto_batcher")
    lora = load_pkg("lora")
    xg = load_pkg("llama_exec_graph")
    batcher = ab.LlamaAutoBatcherClass()
    batcher.set_model(model)
    batcher.set_exec_config(xg.LlamaExecConfig(max_prompt_len=wl.prompt_len, max_gen_len=max_gen_len, page_size=wl.page_size,
                                               native_decode=native_decode, dense_lora=dense_lora,
                                               batch_prefill=batch_prefill))
    batcher.set_free_pages(free_pages)
    batcher.set_eos_token_id(eos_token_id)
    results = []
    for i in range(len(prompts)):
        var = batcher.create_var(np.asarray(prompts[i], dtype=np.int32))
        if adapter_ids[i] >= 0:
            tid = 0 if tids is None else tids[i]
            lt = model.lora_types[tid]
            batcher.set_adapter(lora.LoraConfig(r=lt.r, alpha=lt.scaling * lt.r), wid=int(adapter_ids[i]))
        results.append(batcher.generate(var, max_gen_len=None if max_gen_lens is None else max_gen_lens[i]))
    batcher.compile()
    batcher.execute()
    return [list(map(int, r.var)) for r in results], batcher


NEAR_TIE = 2e-2   # a top-1/top-2 margin below this fraction of the logit std is not numerically decided


def teacher_forced_hip(model, wl, prompts, adapter_ids, tokens, free_pages, tid=0):
    """Run the HIP model along a given token trajectory (tokens[b] = generated ids of request b, all the same
    length) and return its own argmax at every step: out[b][i] is what the HIP path would emit as token i."""
    import torch
    ops = load_pkg("ops")
    B, P = prompts.shape
    n_steps = len(tokens[0])
    kv = model.create_paged_kv_cache(B, B * (P + n_steps + 16), P, wl.page_size, free_pages=free_pages,
                                     max_seq_len=P + n_steps + 1)
    out = [[] for _ in range(B)]
    for b in range(B):
        kv.add_sequence(b)
        kv.begin_forward([b], [P])
        h = model.embed(torch.from_numpy(np.ascontiguousarray(prompts[b])))
        if adapter_ids[b] >= 0:
            logits, _ = model[f"prefill_a{tid}"](h, kv, [int(adapter_ids[b])])
        else:
            logits, _ = model["prefill_no_adapter"](h, kv)
        kv.end_forward()
        out[b].append(int(ops.argmax(logits).cpu()[0]))
    ids = np.asarray(adapter_ids, dtype=np.int32)
    for i in range(1, n_steps):
        forced = torch.tensor([tokens[b][i - 1] for b in range(B)], dtype=torch.int32)
        kv.begin_forward(list(range(B)), [1] * B)
        logits, _ = model[f"decode_a{tid}"](model.embed(forced), kv, ids)
        kv.end_forward()
        nxt = ops.argmax(logits).cpu().numpy()
        for b in range(B):
            out[b].append(int(nxt[b]))
    return out


def check_tokens_against_oracle(got, exp, margins, scales, near_tie=NEAR_TIE):
    """Every token must equal the oracle's, except where the oracle's own decision is a near tie
    (margin < near_tie * logit std).  Returns the list of (request, step) near-tie disagreements."""
    ties = []
    for b in range(len(exp)):
        assert len(got[b]) == len(exp[b]), (b, len(got[b]), len(exp[b]))
        for i in range(len(exp[b])):
            if got[b][i] != exp[b][i]:
                assert margins[b][i] < near_tie * scales[b][i], \
                    f"request {b} step {i}: {got[b][i]} != {exp[b][i]} with oracle margin {margins[b][i]:.4g} " \
                    f"(logit std {scales[b][i]:.3g})"
                ties.append((b, i))
    return ties
