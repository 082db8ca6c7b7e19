"""The three large configurations at their real layer shapes against the CPU oracle.

* the benchmark model at full depth (32 layers, hidden 4096, 32 requests x 16 rank-16 adapters on q/k/v/o, 512-token
  prompts, shuffled pages): prefill on the HIP path, the cache copied into the oracle (a layout transform only), then
  decode steps of the graph-replayed native step - the path `bench.py` times - beside teacher-forced oracle steps in
  both precision modes;
* the prefill configuration at full layer shape with 2 layers (8 x 512 tokens, 64 rank-64 adapters on all seven
  linears, this package's GEMM);
* the 256-request stress configuration at full layer shape with 2 layers (Zipf over 256 rank-16 adapters, contexts
  128..2048 in shuffled pages, the same fp16 cache contents on both sides).

The oracle's weights are the device-generated tensors copied to the host (the generator gives the same bits on
either side; one tensor is regenerated on the CPU to show it), which spares the host the hash arithmetic for 6.7e9
parameters.
"""
import time

import numpy as np
import pytest
import torch

import oracle
from conftest import load_pkg
from helpers import NEAR_TIE

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _f32(t):
    return t.detach().float().cpu().numpy()


def oracle_from_device(wl, specs, check_key=None):
    """-> (weights, lora, scaling) as float32 numpy dicts, generated on the GPU layer by layer and copied over."""
    synth = load_pkg("synth")
    s = wl.shape
    w = {"embed_tokens": _f32(synth.normal(wl.seed, "embed_tokens", (s.vocab_size, s.hidden_size), 0.02, torch.float16, DEV)),
         "lm_head": _f32(synth.normal(wl.seed, "lm_head", (s.vocab_size, s.hidden_size), 0.02, torch.float16, DEV)),
         "norm": np.ones(s.hidden_size, np.float32)}
    for l in range(s.num_hidden_layers):
        for k, v in synth.layer_weights(wl.seed, s, l, torch.float16, DEV).items():
            w[k] = _f32(v)
    lora, scaling = {}, {}
    for tid, spec in enumerate(specs):
        for l in range(s.num_hidden_layers):
            for k, v in synth.lora_weights(wl.seed, s, spec, torch.float16, DEV, layers=[l], tag=f"a{tid}").items():
                lora[k] = _f32(v)
        scaling[f"a{tid}"] = spec.scaling
    if check_key is not None:                       # one tensor regenerated on the host: same bits
        N, K = w[check_key].shape
        cpu = synth.normal(wl.seed, check_key, (N, K), 0.02, torch.float16, "cpu").float().numpy()
        assert np.array_equal(cpu, w[check_key])
    return w, lora, scaling


def copy_cache_to_oracle(kv, kvr, seq_ids):
    """HIP cache -> oracle cache: keys from fragment order to [page, head, token, dim], values transposed; block
    tables, lengths and the free list as they stand."""
    for l in range(kv.n_layers):
        kvr.k[l] = _f32(kv.k_rowmajor(l))
        kvr.v[l] = _f32(kv.v[l].transpose(-1, -2))
    kvr.tables = {s: list(kv.pages_of(s)) for s in seq_ids}
    kvr.lens = {s: int(kv.lens[s]) for s in seq_ids}
    kvr.free = list(kv.free)


def _margins(logits):
    srt = np.sort(logits, -1)
    return srt[:, -1] - srt[:, -2], logits.std(-1)


def _compare(tag, got, exp, tol, rms_tol=None):
    """logits within tol of the logit std (largest deviation over all rows and vocabulary entries) and within rms_tol in
    the root mean square; argmax equal wherever the oracle's top-2 margin is decided.  Returns (error, rms error,
    decided rows, rows whose argmax differs)."""
    err = float(np.abs(got - exp).max() / exp.std())
    rms = float(np.sqrt(np.mean((got - exp) ** 2)) / exp.std())
    m, sd = _margins(exp)
    decided = m >= NEAR_TIE * sd
    diff = got.argmax(-1) != exp.argmax(-1)
    print(f"{tag}: logits max {err:.2e} / rms {rms:.2e} of the logit std; {int(decided.sum())} of {len(decided)} rows decided, "
          f"{int(diff.sum())} argmax differences ({int((diff & decided).sum())} on decided rows)", flush=True)
    assert err <= tol, (tag, err)
    assert rms_tol is None or rms <= rms_tol, (tag, rms)
    assert not (diff & decided).any(), tag
    return err, rms, int(decided.sum()), int(diff.sum())


def test_c3_full_depth_native_step_against_oracle():
    synth, llama, dsm, ops = (load_pkg(m) for m in ("synth", "llama", "decode_session", "ops"))
    steps = 3
    wl = synth.config3(num_layers=32)
    s = wl.shape
    B, P = wl.batch, wl.prompt_len
    print("building the 32-layer model", flush=True)
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], DEV)
    prompts = synth.prompts(wl)
    blocks = -(-(P + steps + 2) // 16)
    perm = synth.permutation(wl.seed, "c3.full.pages", B * blocks)
    kv = model.create_paged_kv_cache(B, B * blocks * 16, P, 16, free_pages=perm, max_seq_len=blocks * 16)
    seqs = list(range(B))
    for q in seqs:
        kv.add_sequence(q)
    first = np.zeros(B, np.int32)
    for lo in range(0, B, 4):                                 # HIP prefill, four prompts per pass
        sids = seqs[lo:lo + 4]
        kv.begin_forward(sids, [P] * len(sids))
        h = model.embed(torch.from_numpy(np.ascontiguousarray(prompts[sids].reshape(-1))))
        logits, _ = model["prefill_a0"](h, kv, wl.adapter_ids[sids])
        kv.end_forward()
        first[sids] = ops.argmax(logits).cpu().numpy()
    print("copying weights and the cache to the host", flush=True)
    w, lora, scaling = oracle_from_device(wl, [wl.lora], check_key=f"layers.{s.num_hidden_layers - 1}.k_proj")
    ref = {m: oracle.LlamaRef(s, w, lora, scaling, mode=m) for m in ("mixed", "fp32")}
    kvr = ref["mixed"].new_cache(B * blocks, 16, blocks * 16, perm)
    copy_cache_to_oracle(kv, kvr, seqs)

    # (1) the benchmarked path: dense-shrink native step replayed from a graph, free-running
    sess = dsm.NativeDecodeSession(model, kv, seqs, wl.adapter_ids, first, use_graph=True)
    assert sess.dense_lora
    tok_in, hip = [], {"dense": [], "ids": []}
    for i in range(steps):
        tok_in.append(sess.tokens.cpu().numpy().copy())
        out = sess.step().cpu().numpy().copy()
        lg = _f32(sess.buf["logits"].view(B, -1))
        assert np.array_equal(out, lg.argmax(-1))
        hip["dense"].append(lg)
    # (2) the ids-based native step (what the front end runs by default), teacher-forced along the same inputs,
    #     over the same pages (positions P.. are simply written again)
    for q in seqs:
        kv.lens[q] = P
    sess = dsm.NativeDecodeSession(model, kv, seqs, wl.adapter_ids, tok_in[0], use_graph=False, dense_lora=False)
    for i in range(steps):
        sess.tokens.copy_(torch.from_numpy(tok_in[i]))
        sess.step()
        hip["ids"].append(_f32(sess.buf["logits"].view(B, -1)))
    del sess, model
    torch.cuda.empty_cache()

    # (3) the oracle, teacher-forced along the same inputs, in both modes from the same prefilled cache
    ids = {"a0": wl.adapter_ids}
    summary = {}
    # Tolerances: at two layers the logits sit within 5e-3 of the oracle's (largest deviation, in units of the logit
    # std); through 32 layers the fp16 rounding flips of every stored activation (fp32 summation order straddling an
    # fp16 boundary on a fraction of a percent of the elements) add up to what was measured here: 1.7e-2 .. 2.0e-2
    # at the worst of 32 x 32000 logits and 3.4e-3 in the root mean square against the mixed oracle, 2.4e-2 .. 3.0e-2
    # and 5.0e-3 against the all-fp32 oracle, whose own distance to the mixed oracle is of that size.  Bounds = 1.5 x.
    for mode, tol, rms_tol in (("mixed", 3e-2, 5e-3), ("fp32", 4.5e-2, 7.5e-3)):
        for q in seqs:
            kvr.lens[q] = P
        kvr.round = oracle.f16 if mode == "mixed" else (lambda a: np.asarray(a, dtype=np.float32))
        for i in range(steps):
            t0 = time.perf_counter()
            kvr.begin_forward(seqs, [1] * B)
            exp = ref[mode].forward(tok_in[i], kvr, ids)
            kvr.end_forward()
            print(f"oracle {mode} step {i}: {time.perf_counter() - t0:.1f} s", flush=True)
            for kind in ("dense", "ids"):
                summary[(mode, kind, i)] = _compare(f"step {i} {kind}-shrink vs {mode} oracle", hip[kind][i], exp, tol, rms_tol)
    # the page walk: both sides handed the new page of every sequence out of the same free list
    for q in seqs:
        assert list(kv.pages_of(q)) == kvr.tables[q]
    print("summary (max error, rms error, decided rows, argmax differences):", summary, flush=True)
    # measured: 88 of the 96 (request, step) decisions are decided (top-2 margin >= 2 % of the logit std) and the HIP
    # token equals the oracle's on every one of them, in both modes (asserted row by row in _compare).  On the 8 near
    # ties the token follows fp32 summation orders - of the prefill attention and the GEMMs that filled the cache as
    # much as of the step itself - and has differed 1 to 3 times against either oracle from one kernel revision to
    # the next: no more than the near ties there are.
    for mode in ("mixed", "fp32"):
        for kind in ("dense", "ids"):
            undecided = sum(B - summary[(mode, kind, i)][2] for i in range(steps))
            assert sum(summary[(mode, kind, i)][3] for i in range(steps)) <= undecided <= 10, (mode, kind)


def test_c4_prefill_full_layer_shape_against_oracle():
    """8 x 512 tokens in adapter segments, 64 rank-64 adapters on all seven linears, hidden 4096 / 32 x 128 heads /
    intermediate 11008, two layers, base linears on this package's GEMM."""
    synth, llama = load_pkg("synth"), load_pkg("llama")
    wl = synth.config4(num_layers=2)
    s = wl.shape
    B, P = wl.batch, wl.prompt_len
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], DEV)
    prompts = synth.prompts(wl)
    order = np.argsort(wl.adapter_ids, kind="stable")             # requests grouped into adapter segments
    wids = wl.adapter_ids[order]
    tokens = np.ascontiguousarray(prompts[order].reshape(-1))
    blocks = P // 16
    perm = synth.permutation(wl.seed, "c4.full.pages", B * blocks)
    kv = model.create_paged_kv_cache(B, B * P, P, 16, free_pages=perm, max_seq_len=P)
    seqs = list(range(B))
    for q in seqs:
        kv.add_sequence(q)
    kv.begin_forward(seqs, [P] * B)
    got, _ = model["prefill_a0"](model.embed(torch.from_numpy(tokens)), kv, wids)
    kv.end_forward()
    got = _f32(got)
    w, lora, scaling = oracle_from_device(wl, [wl.lora], check_key="layers.1.o_proj")
    rows = np.arange(B) * P + P - 1
    for mode, tol in (("mixed", 1e-2), ("fp32", 1.5e-2)):
        ref = oracle.LlamaRef(s, w, lora, scaling, mode=mode)
        ref.fuse_blocks = 256        # the HIP pass carries the deltas of its adapter-uniform 256-token blocks inside the base GEMM: rounded once
        kvr = ref.new_cache(B * blocks, 16, P, perm)
        for q in seqs:
            kvr.add_sequence(q)
        t0 = time.perf_counter()
        kvr.begin_forward(seqs, [P] * B)
        exp = ref.forward(tokens, kvr, {"a0": np.repeat(wids, P)}, logits_rows=rows)
        kvr.end_forward()
        print(f"oracle {mode} prefill of {B * P} tokens: {time.perf_counter() - t0:.1f} s", flush=True)
        _compare(f"C4 prefill vs {mode} oracle", got, exp, tol)
        if mode == "mixed":
            for q in seqs:
                assert list(kv.pages_of(q)) == kvr.tables[q]
            # cached keys and values of the last layer: fp16 storage on both sides, a few ulps apart at most
            for name, mine, theirs in (("k", _f32(kv.k_rowmajor(1)), kvr.k[1]), ("v", _f32(kv.v[1].transpose(-1, -2)), kvr.v[1])):
                d = float(np.abs(mine - theirs).max())
                print(f"layer-1 {name} cache: max abs difference {d:.3e} (values up to {np.abs(theirs).max():.2f})", flush=True)
                assert d <= 2e-2 * float(np.abs(theirs).max())
            # the adapters matter at this rank: without them the logits move by far more than the tolerance
            kv0 = ref.new_cache(B * blocks, 16, P, perm)
            for q in seqs:
                kv0.add_sequence(q)
            kv0.begin_forward(seqs, [P] * B)
            base = ref.forward(tokens, kv0, {}, logits_rows=rows)
            kv0.end_forward()
            assert float(np.abs(base - exp).max() / exp.std()) > 10 * tol


def test_c5_decode_full_layer_shape_against_oracle():
    """256 requests over 256 rank-16 adapters (Zipf popularity), contexts 128..2048 in shuffled pages pre-filled with
    the same fp16 values on both sides, hidden 4096 / 32 x 128 heads, two layers: two teacher-forced decode steps."""
    synth, llama, ops = load_pkg("synth"), load_pkg("llama"), load_pkg("ops")
    steps = 2
    wl = synth.config5(num_layers=2)
    s = wl.shape
    B = wl.batch
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], DEV)
    order = np.argsort(wl.adapter_ids, kind="stable")             # the front end's order: by adapter
    ids = wl.adapter_ids[order].astype(np.int32)
    ctx = wl.ctx_lens[order].astype(np.int64)
    blocks = [int(-(-(c + steps + 1) // 16)) for c in ctx]
    n_pages = sum(blocks)
    perm = synth.permutation(wl.seed, "c5.full.pages", n_pages)
    kv = model.create_paged_kv_cache(B, n_pages * 16, 1, 16, free_pages=perm, max_seq_len=max(blocks) * 16)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(5)
    for l in range(s.num_hidden_layers):
        kv.k[l].normal_(generator=gen)
        kv.v[l].normal_(generator=gen)
    seqs = list(range(B))
    for q in seqs:
        kv.add_sequence(q)
    kv.begin_forward(seqs, [int(c) for c in ctx])                 # claims the pages of the pre-filled contexts
    kv.end_forward()
    w, lora, scaling = oracle_from_device(wl, [wl.lora], check_key="layers.0.v_proj")
    ref = {m: oracle.LlamaRef(s, w, lora, scaling, mode=m) for m in ("mixed", "fp32")}
    kvr = ref["mixed"].new_cache(n_pages, 16, max(blocks) * 16, perm)
    copy_cache_to_oracle(kv, kvr, seqs)
    tok = synth.randint(wl.seed, "c5.full.first", (B,), s.vocab_size).numpy()
    hip, tok_in = [], []
    for i in range(steps):
        tok_in.append(tok.copy())
        kv.begin_forward(seqs, [1] * B)
        lg, _ = model["decode_a0"](model.embed(torch.from_numpy(tok.astype(np.int32))), kv, ids)
        kv.end_forward()
        assert np.array_equal(ops.argmax(lg).cpu().numpy(), _f32(lg).argmax(-1))
        hip.append(_f32(lg))
        tok = hip[-1].argmax(-1)
    for mode, tol, n in (("mixed", 1e-2, steps), ("fp32", 1.5e-2, 1)):
        for q in seqs:
            kvr.lens[q] = int(ctx[q])
        kvr.round = oracle.f16 if mode == "mixed" else (lambda a: np.asarray(a, dtype=np.float32))
        for i in range(n):
            t0 = time.perf_counter()
            kvr.begin_forward(seqs, [1] * B)
            exp = ref[mode].forward(tok_in[i], kvr, {"a0": ids})
            kvr.end_forward()
            print(f"oracle {mode} step {i} over {int(ctx.sum())} cached positions: {time.perf_counter() - t0:.1f} s", flush=True)
            _compare(f"C5 step {i} vs {mode} oracle", hip[i], exp, tol)
    for q in seqs:
        assert list(kv.pages_of(q)) == kvr.tables[q]
