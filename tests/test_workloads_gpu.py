"""Reduced-size versions of the prefill workload (rank-64 adapters on all seven linears, ragged prompts grouped
into adapter segments) and of the auto-batching decode stress (more than 64 concurrent requests, Zipf adapter
popularity, ragged context lengths, shuffled block table), against the CPU oracle.

The full-size workloads differ from these only in dimensions; every code path they take (segment LoRA on all
linears, prefill attention over ragged sequences, the T > 64 decode path with row-major activations) is the
one exercised here at sizes the numpy oracle finishes in seconds.
"""
import numpy as np
import pytest
import torch

from conftest import load_pkg
from helpers import NEAR_TIE, hip_model, oracle_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _err(g, r):
    """max abs error against the logit scale (a logit is a long sum with cancellation)."""
    return float(np.abs(g - r).max() / r.std())


def _small_shape(synth, layers=2):
    return synth.LlamaShape(hidden_size=512, intermediate_size=1408, num_attention_heads=8, num_key_value_heads=8,
                            num_hidden_layers=layers, head_dim=64, vocab_size=4096)


def _oracle_prefill(ref, prompts, tok_ids, n_pages, page_size, perm, max_len):
    kv = ref.new_cache(n_pages, page_size, max_len, perm)
    lens = [len(p) for p in prompts]
    for s in range(len(prompts)):
        kv.add_sequence(s)
    kv.begin_forward(list(range(len(prompts))), lens)
    logits = ref.forward(np.concatenate(prompts), kv, tok_ids, logits_rows=np.cumsum(lens) - 1)
    kv.end_forward()
    return kv, logits


def _hip_prefill(model, prompts, wids, n_pages, page_size, perm, max_len):
    lens = [len(p) for p in prompts]
    kv = model.create_paged_kv_cache(len(prompts), n_pages * page_size, max(lens), page_size, free_pages=perm,
                                     max_seq_len=max_len)
    for s in range(len(prompts)):
        kv.add_sequence(s)
    kv.begin_forward(list(range(len(prompts))), lens)
    h = model.embed(torch.from_numpy(np.concatenate(prompts).astype(np.int32)))
    logits, _ = model["prefill_a0"](h, kv, wids)
    kv.end_forward()
    return kv, logits.cpu().numpy()


def test_prefill_rank64_all_linears_adapter_segments():
    """Five ragged prompts in three adapter segments, rank-64 LoRA on q, k, v, o, gate, up, down (248 tokens)."""
    synth = load_pkg("synth")
    shape = _small_shape(synth)
    lora = synth.LoraSpec(r=64, alpha=32.0, n_adapters=6, targets=synth.LINEARS)
    wl = synth.Workload("c4_small", 3, shape, lora, batch=5, prompt_len=81, gen_len=0,
                        adapter_ids=np.array([0, 0, 3, 3, 5], dtype=np.int32))
    lens = [37, 64, 50, 16, 81]
    prompts = [synth.randint(3, f"c4s.prompt{i}", (n,), shape.vocab_size).numpy() for i, n in enumerate(lens)]
    n_pages = sum(-(-n // 16) for n in lens) + 4
    perm = synth.permutation(3, "c4s.pages", n_pages)
    tok_ids = {"a0": np.repeat(wl.adapter_ids, lens)}
    model = hip_model(wl)
    kvh, got = _hip_prefill(model, prompts, wl.adapter_ids, n_pages, 16, perm, 96)
    for mode, tol in (("mixed", 1e-2), ("fp32", 1.5e-2)):
        kvr, exp = _oracle_prefill(oracle_model(wl, mode), prompts, tok_ids, n_pages, 16, perm, 96)
        e = _err(got, exp)
        print(f"rank-64 / 7 linears prefill logits vs {mode} oracle: {e:.2e} of the logit std")
        assert e <= tol
        if mode == "mixed":
            for s in range(5):
                assert list(kvh.table_h[kvh.slot[s], :len(kvr.tables[s])]) == list(kvr.tables[s])
            margin = np.sort(exp, -1)[:, -1] - np.sort(exp, -1)[:, -2]
            decided = margin >= NEAR_TIE * exp.std(-1)
            assert np.array_equal(got.argmax(-1)[decided], exp.argmax(-1)[decided])
            # the LoRA delta must matter at this rank: without it the logits move by far more than the tolerance
            kv0, base = _oracle_prefill(oracle_model(wl, mode), prompts, {}, n_pages, 16, perm, 96)
            assert _err(base, exp) > 10 * tol


def test_decode_more_than_64_requests_zipf_adapters_ragged_contexts():
    """80 concurrent requests over 40 rank-16 adapters (Zipf popularity, some requests without adapter), context
    lengths 20..200 in a shuffled paged cache; three teacher-forced decode steps."""
    synth = load_pkg("synth")
    ops = load_pkg("ops")
    shape = _small_shape(synth)
    B, n_ad = 80, 40
    lora = synth.LoraSpec(r=16, alpha=8.0, n_adapters=n_ad, targets=("q_proj", "k_proj", "v_proj", "o_proj"))
    ids = synth.zipf_ids(4, "c5s.ids", B, n_ad, 1.1).astype(np.int32)
    ids[[7, 33]] = -1
    wl = synth.Workload("c5_small", 4, shape, lora, batch=B, prompt_len=200, gen_len=3, adapter_ids=ids)
    lens = (20 + synth.randint(4, "c5s.ctx", (B,), 181).numpy()).tolist()
    prompts = [synth.randint(4, f"c5s.prompt{i}", (n,), shape.vocab_size).numpy() for i, n in enumerate(lens)]
    n_pages = sum(-(-(n + 4) // 16) for n in lens) + 8
    perm = synth.permutation(4, "c5s.pages", n_pages)
    steps = 3
    ref = oracle_model(wl, "mixed")
    kvr, l0 = _oracle_prefill(ref, prompts, {"a0": np.repeat(ids, lens)}, n_pages, 16, perm, 208)
    model = hip_model(wl)
    kvh, g0 = _hip_prefill(model, prompts, ids, n_pages, 16, perm, 208)
    assert _err(g0, l0) <= 1e-2
    tok = l0.argmax(-1)
    for i in range(steps):
        kvr.begin_forward(list(range(B)), [1] * B)
        lr = ref.forward(tok, kvr, {"a0": ids})
        kvr.end_forward()
        kvh.begin_forward(list(range(B)), [1] * B)
        lg, _ = model["decode_a0"](model.embed(torch.from_numpy(tok.astype(np.int32))), kvh, ids)
        kvh.end_forward()
        got_tok = ops.argmax(lg).cpu().numpy()
        lg = lg.cpu().numpy()
        e = _err(lg, lr)
        print(f"decode step {i}, 80 requests: logits {e:.2e} of the logit std")
        assert e <= 1e-2
        srt = np.sort(lr, -1)
        decided = (srt[:, -1] - srt[:, -2]) >= NEAR_TIE * lr.std(-1)
        assert np.array_equal(got_tok[decided], lr.argmax(-1)[decided])
        assert np.array_equal(got_tok, lg.argmax(-1))
        tok = lr.argmax(-1)
    # integer bookkeeping: both caches walked the same pages
    for s in range(B):
        n_blk = -(-(lens[s] + steps) // 16)
        assert list(kvh.table_h[kvh.slot[s], :n_blk]) == list(kvr.tables[s])[:n_blk]


@pytest.mark.parametrize("B,use_graph,native", [(70, False, False), (12, True, False), (70, True, True), (12, False, True)])
def test_decode_session_longest_context_first_keeps_tokens_and_request_order(B, use_graph, native):
    """The session may run its batch internally in order of decreasing context length (the long sequences' attention
    workgroups start first); every operator treats rows independently, so each request's tokens and cache pages are
    those of the batch in request order, bit for bit, and come back in request order."""
    synth = load_pkg("synth")
    dsm = load_pkg("decode_session")
    shape = _small_shape(synth)
    n_ad = 6
    lora = synth.LoraSpec(r=16, alpha=8.0, n_adapters=n_ad, targets=("q_proj", "k_proj", "v_proj", "o_proj"))
    ids = synth.randint(6, f"lf.ids{B}", (B,), n_ad + 1).numpy().astype(np.int32) - 1        # -1 = no adapter
    wl = synth.Workload("lf_small", 6, shape, lora, batch=B, prompt_len=90, gen_len=6, adapter_ids=ids)
    lens = (5 + synth.randint(6, f"lf.ctx{B}", (B,), 86).numpy()).tolist()
    prompts = [synth.randint(6, f"lf.prompt{B}.{i}", (n,), shape.vocab_size).numpy() for i, n in enumerate(lens)]
    steps = 6
    n_pages = sum(-(-(n + steps + 1) // 16) for n in lens) + 4
    perm = synth.permutation(6, f"lf.pages{B}", n_pages)
    model = hip_model(wl)
    runs = []
    for longest_first in (False, True):
        kv, logits = _hip_prefill(model, prompts, ids, n_pages, 16, perm, 112)
        first = logits.argmax(-1).astype(np.int32)
        if native:
            sess = dsm.NativeDecodeSession(model, kv, list(range(B)), ids, first, use_graph=use_graph, longest_first=longest_first,
                                           dense_lora=False)
        else:
            sess = dsm.DecodeSession(model, kv, list(range(B)), {0: ids}, first, use_graph=use_graph, longest_first=longest_first)
        toks = np.stack([sess.step().cpu().numpy().copy() for _ in range(steps)])
        rows = [[kv.k[0][p].clone() for p in kv.pages_of(s)] for s in range(B)]
        runs.append((toks, rows, [kv.lens[s] for s in range(B)]))
    (t0, r0, l0), (t1, r1, l1) = runs
    assert np.array_equal(t0, t1)
    assert l0 == l1 == [n + steps for n in lens]
    for s in range(B):
        assert len(r0[s]) == len(r1[s]) and all(torch.equal(a, b) for a, b in zip(r0[s], r1[s])), s
