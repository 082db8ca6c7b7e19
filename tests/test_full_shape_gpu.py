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


def oracle_from_device(wl, specs, check_key=None, adapters=None):
    """-> (weights, lora, scaling) as float32 numpy dicts, generated on the GPU layer by layer and copied over.
    adapters: rows of the adapter tables to keep, in this order (the caller renumbers its ids accordingly) - a pass that
    uses 8 of 64 rank-64 adapters need not hold the other 56 on the host."""
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
                lora[k] = _f32(v if adapters is None else v[torch.as_tensor(adapters, device=v.device)])
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
    decided rows, rows whose argmax differs, the mask of those rows)."""
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
    return err, rms, int(decided.sum()), int(diff.sum()), diff


def test_c3_full_depth_native_step_against_oracle():
    """The benchmarked 32-layer step against the oracle: 18 steps (free-running on the HIP side, the oracle teacher-forced
    along the same inputs - the run crosses the page boundary at position 528 under graph replay) in mixed mode, 3 in fp32
    mode; and the same step cut off after 2, 8 and 16 layers, which gives the error bound of the full depth: rounding
    flips of independent layers add up like a random walk, so the error may grow with the square root of the depth."""
    import dataclasses
    synth, llama, dsm, ops = (load_pkg(m) for m in ("synth", "llama", "decode_session", "ops"))
    steps = {"mixed": 18, "fp32": 3}
    n_steps = max(steps.values())
    wl = synth.config3(num_layers=32)
    s = wl.shape
    B, P = wl.batch, wl.prompt_len
    assert P + n_steps > 528 >= P + 3                          # the long leg allocates a page per sequence on the way
    print("building the 32-layer model", flush=True)
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], DEV)
    prompts = synth.prompts(wl)
    blocks = -(-(P + n_steps + 2) // 16)
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
    assert all(len(kv.pages_of(q)) == P // 16 for q in seqs)

    def rewind():
        """Both caches back to the end of the prefill: positions P.. are simply written again, into the pages that the
        sequences were given for them the first time."""
        for q in seqs:
            kv.lens[q] = P
            kvr.lens[q] = P

    def set_mode(mode):
        kvr.round = oracle.f16 if mode == "mixed" else (lambda a: np.asarray(a, dtype=np.float32))

    # (0) the step cut off after d layers (final norm and head on the residual stream as it stands there), one step each;
    #     the oracle's logits at those depths are taken off its first full-depth step below (`tap_depths`): the error
    #     at depth 2 sets the bound for depth 32
    shallow = (2, 8, 16)
    hip_d = {}
    for d in shallow:
        sess = dsm.NativeDecodeSession(model, kv, seqs, wl.adapter_ids, first, use_graph=False)
        sess.plan.n_layers = d
        sess.step()
        hip_d[d] = _f32(sess.buf["logits"].view(B, -1))
        del sess
        rewind()
    ids = {"a0": wl.adapter_ids}
    depth_err = {}

    # (1) the benchmarked path: dense-shrink native step replayed from a graph, free-running
    sess = dsm.NativeDecodeSession(model, kv, seqs, wl.adapter_ids, first, use_graph=True)
    assert sess.dense_lora
    tok_in, hip = [], {"dense": [], "ids": []}
    for i in range(n_steps):
        tok_in.append(sess.tokens.cpu().numpy().copy())
        out = sess.step().cpu().numpy().copy()
        lg = _f32(sess.buf["logits"].view(B, -1))
        assert np.array_equal(out, lg.argmax(-1))
        hip["dense"].append(lg)
    assert all(len(kv.pages_of(q)) == P // 16 + 2 for q in seqs)      # a page for position 512 and one for position 528
    pages_after = {q: list(kv.pages_of(q)) for q in seqs}
    # (2) the ids-based native step (what the front end runs by default), teacher-forced along the same inputs,
    #     over the same pages
    for q in seqs:
        kv.lens[q] = P
    sess = dsm.NativeDecodeSession(model, kv, seqs, wl.adapter_ids, tok_in[0], use_graph=False, dense_lora=False)
    for i in range(n_steps):
        sess.tokens.copy_(torch.from_numpy(tok_in[i]))
        sess.step()
        hip["ids"].append(_f32(sess.buf["logits"].view(B, -1)))
    assert all(list(kv.pages_of(q)) == pages_after[q] for q in seqs)
    del sess, model
    torch.cuda.empty_cache()

    # (3) the oracle, teacher-forced along the same inputs, in both modes from the same prefilled cache.
    # Bounds: at two layers the error is a few fp16 rounding flips of stored activations (fp32 summation order
    # straddling an fp16 boundary on a fraction of a percent of the elements); flips of different layers are
    # independent, so through L layers the root mean square may grow like sqrt(L / 2) - with half as much again for
    # the later steps, whose inputs already carry the error of the steps before.  The largest of the 32 x 32000
    # deviations of a step sits 5 to 6 root mean squares out (a Gaussian's extreme over 1e6 samples is at 4.9): bound 8.
    summary = {}
    for mode in ("mixed", "fp32"):
        for q in seqs:
            kvr.lens[q] = P
        set_mode(mode)
        for i in range(steps[mode]):
            t0 = time.perf_counter()
            kvr.begin_forward(seqs, [1] * B)
            exp = ref[mode].forward(tok_in[i], kvr, ids, tap_depths=shallow if i == 0 else ())
            kvr.end_forward()
            print(f"oracle {mode} step {i}: {time.perf_counter() - t0:.1f} s", flush=True)
            if i == 0:                                             # tok_in[0] is `first`: the input of the cut-off steps
                assert np.array_equal(tok_in[0], first)
                for d in shallow:
                    exp_d = ref[mode].taps[d]
                    err = float(np.abs(hip_d[d] - exp_d).max() / exp_d.std())
                    rms = float(np.sqrt(np.mean((hip_d[d] - exp_d) ** 2)) / exp_d.std())
                    depth_err[(mode, d)] = (err, rms)
                    print(f"depth {d:2d} vs {mode} oracle: logits max {err:.2e} / rms {rms:.2e} of the logit std", flush=True)
                rms2 = depth_err[(mode, 2)][1]
                assert rms2 <= (1.5e-3 if mode == "mixed" else 2.5e-3), (mode, rms2)   # the two-layer figure itself
                for d in shallow:
                    err, rms = depth_err[(mode, d)]
                    assert rms <= 1.5 * rms2 * np.sqrt(d / 2) and err <= 8 * 1.5 * rms2 * np.sqrt(d / 2), (mode, d, err, rms)
                rms_tol = 1.5 * rms2 * np.sqrt(s.num_hidden_layers / 2)
                tol = 8 * rms_tol
                print(f"{mode}: two-layer rms {rms2:.2e} -> bounds at depth {s.num_hidden_layers}: rms {rms_tol:.2e}, max {tol:.2e}", flush=True)
            for kind in ("dense", "ids"):
                summary[(mode, kind, i)] = _compare(f"step {i} {kind}-shrink vs {mode} oracle", hip[kind][i], exp, tol, rms_tol)
        # the page walk: both sides handed the new page of every sequence out of the same free list
        if steps[mode] == n_steps:
            for q in seqs:
                assert pages_after[q] == kvr.tables[q]
    print("summary (max error, rms error, decided rows, argmax differences):", summary, flush=True)
    # Greedy tokens: on every decided row (top-2 margin of the oracle >= 2 % of the logit std) the HIP token equals the
    # oracle's, in both modes, at every step (asserted row by row in _compare).  On the near ties the token follows fp32
    # summation orders - of the prefill kernels that filled the cache as much as of the step itself: it may differ there,
    # on no more rows than there are near ties, and near ties stay a small part of the decisions.
    for mode in ("mixed", "fp32"):
        for kind in ("dense", "ids"):
            decisions = B * steps[mode]
            undecided = sum(B - summary[(mode, kind, i)][2] for i in range(steps[mode]))
            differing = sum(summary[(mode, kind, i)][3] for i in range(steps[mode]))
            print(f"{mode} / {kind}: {decisions} decisions, {decisions - undecided} decided, {undecided} near ties, {differing} differing tokens (all on near ties)", flush=True)
            assert differing <= undecided <= 0.15 * decisions, (mode, kind, differing, undecided)
    # Free-running trajectories: the dense-shrink session above ran on its own tokens, and the oracle was fed the same
    # inputs - so an oracle running on ITS own tokens produces the same sequence for a request up to the first step at
    # which the two argmax differ, and the whole sequence where they never do.  Every first difference is a near tie
    # (asserted per row above); requests without one have identical free-running trajectories over all steps.
    flips = np.stack([summary[("mixed", "dense", i)][4] for i in range(steps["mixed"])])        # [step, request]
    first_flip = np.where(flips.any(0), flips.argmax(0), steps["mixed"])
    same = int((first_flip == steps["mixed"]).sum())
    print(f"free-running: {same} of {B} requests produce the oracle's {steps['mixed']} tokens one for one; the others part "
          f"at a near tie, at steps {sorted(int(f) for f in first_flip if f < steps['mixed'])}", flush=True)
    assert same >= B - int(flips.any(0).sum()) and same >= B // 2


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


def test_c4_prefill_full_depth_against_oracle():
    """The prefill configuration at its full depth (32 layers, 8 x 512 tokens, 64 rank-64 adapters on all seven linears):
    the pass `bench.py --workload c4_prefill` times, against the mixed-mode oracle.  The same pass cut off after 2 and 8
    layers gives the bound, as for the decode step: rounding flips of independent layers add up like a random walk."""
    synth, llama = load_pkg("synth"), load_pkg("llama")
    wl = synth.config4(num_layers=32)
    s = wl.shape
    B, P = wl.batch, wl.prompt_len
    print("building the 32-layer model with its adapters", flush=True)
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], DEV)
    prompts = synth.prompts(wl)
    order = np.argsort(wl.adapter_ids, kind="stable")
    wids = wl.adapter_ids[order]
    tokens = np.ascontiguousarray(prompts[order].reshape(-1))
    blocks = P // 16
    perm = synth.permutation(wl.seed, "c4.deep.pages", B * blocks)
    seqs = list(range(B))
    layers = model.layers
    depths = (32, 8, 2)                                           # the full pass first: it builds the per-layer caches of the model
    hip, kv_full = {}, None
    for d in depths:
        model.layers = layers[:d]
        kv = model.create_paged_kv_cache(B, B * P, P, 16, free_pages=perm, max_seq_len=P)
        for q in seqs:
            kv.add_sequence(q)
        kv.begin_forward(seqs, [P] * B)
        got, _ = model["prefill_a0"](model.embed(torch.from_numpy(tokens)), kv, wids)
        kv.end_forward()
        hip[d] = _f32(got)
        if d == s.num_hidden_layers:
            kv_full = kv
        else:
            del kv
    model.layers = layers
    used = np.unique(wids)
    print("copying weights to the host", flush=True)
    w, lora, scaling = oracle_from_device(wl, [wl.lora], check_key="layers.31.up_proj", adapters=used)
    rows = np.arange(B) * P + P - 1
    ref = oracle.LlamaRef(s, w, lora, scaling, mode="mixed")
    ref.fuse_blocks = 256
    kvr = ref.new_cache(B * blocks, 16, P, perm)
    for q in seqs:
        kvr.add_sequence(q)
    t0 = time.perf_counter()
    kvr.begin_forward(seqs, [P] * B)
    exp = {32: ref.forward(tokens, kvr, {"a0": np.repeat(np.searchsorted(used, wids), P).astype(np.int32)}, logits_rows=rows,
                           tap_depths=(2, 8))}
    kvr.end_forward()
    exp.update(ref.taps)
    print(f"oracle prefill of {B * P} tokens through 32 layers: {time.perf_counter() - t0:.1f} s", flush=True)
    errs = {}
    for d in sorted(hip):
        errs[d] = (float(np.abs(hip[d] - exp[d]).max() / exp[d].std()), float(np.sqrt(np.mean((hip[d] - exp[d]) ** 2)) / exp[d].std()))
        print(f"depth {d:2d}: logits max {errs[d][0]:.2e} / rms {errs[d][1]:.2e} of the logit std", flush=True)
    rms2 = errs[2][1]
    assert rms2 <= 2e-3, rms2                                     # the two-layer figure itself (measured 9.5e-4)
    for d in sorted(hip):
        rms_tol = 1.5 * rms2 * np.sqrt(d / 2)
        _compare(f"C4 prefill cut off after {d} layers vs mixed oracle", hip[d], exp[d], 8 * rms_tol, rms_tol)
    for q in seqs:
        assert list(kv_full.pages_of(q)) == kvr.tables[q]
    last = s.num_hidden_layers - 1
    for name, mine, theirs in (("k", _f32(kv_full.k_rowmajor(last)), kvr.k[last]), ("v", _f32(kv_full.v[last].transpose(-1, -2)), kvr.v[last])):
        d = float(np.abs(mine - theirs).max())
        print(f"layer-{last} {name} cache: max abs difference {d:.3e} (values up to {np.abs(theirs).max():.2f})", flush=True)
        assert d <= 2e-2 * float(np.abs(theirs).max())


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


def test_reference_default_shape_llama31_8b_two_layers():
    """The reference's own model shape (`tvm/llama_auto_batcher/llama_for_causal_lm.py:10-21`: 8 kv heads under 32
    query heads, intermediate 14336, vocabulary 128256, rope theta 5e5) with the reference's adapter targets (q and v,
    `compile_tvm.py:180-181`), 2 layers, 32 requests x 16 rank-16 adapters, shuffled pages: the HIP prefill and three
    steps of the native decode step (the 384-tile q/k/v GEMV, the 8016-tile head, decode attention with four query
    heads per kv head) against the oracle in both modes, teacher-forced; and the native step, eagerly and replayed from
    a graph, against the per-operator path bit for bit (tokens and the whole K cache)."""
    import dataclasses
    synth, llama, dsm, ops = (load_pkg(m) for m in ("synth", "llama", "decode_session", "ops"))
    steps = 3
    wl = synth.config3(num_layers=2, batch=32, prompt_len=40, gen_len=steps, shape="llama31_8b")
    spec = synth.LoraSpec(r=16, alpha=8.0, n_adapters=16, targets=("q_proj", "v_proj"))
    wl = dataclasses.replace(wl, lora=spec)
    s = wl.shape
    assert (s.num_key_value_heads, s.intermediate_size, s.vocab_size, s.rope_theta) == (8, 14336, 128256, 500000.0)
    B, P = wl.batch, wl.prompt_len
    adapter_ids = wl.adapter_ids.copy()
    adapter_ids[7] = -1                                        # one request without adapter
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [spec], DEV)
    prompts = synth.prompts(wl)
    blocks = -(-(P + steps + 2) // 16)
    perm = synth.permutation(wl.seed, "l31.pages", B * blocks)
    seqs = list(range(B))

    def hip_prefill():
        kv = model.create_paged_kv_cache(B, B * blocks * 16, P, 16, free_pages=perm, max_seq_len=blocks * 16)
        for q in seqs:
            kv.add_sequence(q)
        out = []
        for lo in range(0, B, 8):
            sids = seqs[lo:lo + 8]
            kv.begin_forward(sids, [P] * len(sids))
            h = model.embed(torch.from_numpy(np.ascontiguousarray(prompts[sids].reshape(-1))))
            tok = np.repeat(adapter_ids[sids], P).astype(np.int32)
            out.append(_f32(model.forward(h, kv, model._ids(len(tok), {0: (None, tok)}), model._last_rows(kv))))
            kv.end_forward()
        return kv, np.concatenate(out)

    # (1) native step == per-operator path, bit for bit
    runs = {}
    for kind in ("py", "native", "graph"):
        kv, l0 = hip_prefill()
        first = l0.argmax(-1).astype(np.int32)
        if kind == "py":
            sess = dsm.DecodeSession(model, kv, seqs, {0: adapter_ids}, first)
        else:
            sess = dsm.NativeDecodeSession(model, kv, seqs, adapter_ids, first, use_graph=(kind == "graph"), dense_lora=False)
        toks = [first] + [sess.step().cpu().numpy().copy() for _ in range(steps)]
        runs[kind] = (np.stack(toks), kv.k.clone())
        del sess, kv
    for kind in ("native", "graph"):
        assert np.array_equal(runs["py"][0], runs[kind][0]), kind
        assert torch.equal(runs["py"][1], runs[kind][1]), kind
    del runs
    torch.cuda.empty_cache()

    # (2) prefill and three steps of the dense-shrink native step (graph) and of the ids-based one against the oracle
    kv, l0 = hip_prefill()
    first = l0.argmax(-1).astype(np.int32)
    sess = dsm.NativeDecodeSession(model, kv, seqs, adapter_ids, first, use_graph=True)
    assert sess.dense_lora
    tok_in, hip = [], {"dense": [], "ids": []}
    for i in range(steps):
        tok_in.append(sess.tokens.cpu().numpy().copy())
        sess.step()
        hip["dense"].append(_f32(sess.buf["logits"].view(B, -1)))
    for q in seqs:
        kv.lens[q] = P
    sess = dsm.NativeDecodeSession(model, kv, seqs, adapter_ids, tok_in[0], use_graph=False, dense_lora=False)
    for i in range(steps):
        sess.tokens.copy_(torch.from_numpy(tok_in[i]))
        sess.step()
        hip["ids"].append(_f32(sess.buf["logits"].view(B, -1)))
    pages = {q: list(kv.pages_of(q)) for q in seqs}
    del sess, model, kv
    torch.cuda.empty_cache()
    w, lora, scaling = oracle_from_device(wl, [spec], check_key="layers.1.v_proj")
    ids = {"a0": adapter_ids}
    # bounds as at the Llama-2 two-layer shape (logits within 1e-2 / 1.5e-2 of the logit std against the mixed / fp32
    # oracle, tests/test_model_gpu.py), root mean square a fifth of that
    for mode, tol in (("mixed", 1e-2), ("fp32", 1.5e-2)):
        ref = oracle.LlamaRef(s, w, lora, scaling, mode=mode)
        kvr = ref.new_cache(B * blocks, 16, blocks * 16, perm)
        for q in seqs:
            kvr.add_sequence(q)
        t0 = time.perf_counter()
        kvr.begin_forward(seqs, [P] * B)
        e0 = ref.forward(prompts.reshape(-1), kvr, {"a0": np.repeat(adapter_ids, P)}, logits_rows=np.arange(B) * P + P - 1)
        kvr.end_forward()
        print(f"oracle {mode} prefill: {time.perf_counter() - t0:.1f} s", flush=True)
        _compare(f"prefill vs {mode} oracle", l0, e0, tol, tol / 5)
        for i in range(steps):
            kvr.begin_forward(seqs, [1] * B)
            exp = ref.forward(tok_in[i], kvr, ids)
            kvr.end_forward()
            for kind in ("dense", "ids"):
                _compare(f"step {i} {kind}-shrink vs {mode} oracle", hip[kind][i], exp, tol, tol / 5)
        for q in seqs:
            assert pages[q] == kvr.tables[q]
