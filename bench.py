#!/usr/bin/env python3
"""Headline benchmark: greedy decode of a Llama-2-7B-shape model, 32 requests x 16 rank-16 LoRA adapters
(q/k/v/o), paged KV cache with 16-token pages in random page order, 512-token prompts.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch (32 new tokens).  Inputs are synthetic (seeded, generated on
the device); weights and the KV cache are resident in HBM when the timed region starts.  Prints ONE JSON
line: decode tok/s, the roofline of the dominant kernel (the weight-streaming GEMV, timed with events on
the launch stream), the gather-matmul figures, and a CPU baseline (the numpy oracle on the host cores,
bounded sample).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
PKG = "tensor-program-optimization-with-auto-batching_amd"
HBM_PEAK_GBS = 8000.0


def _mod(name):
    return importlib.import_module(PKG + "." + name)


def prefill_all(model, kv, prompts, adapter_ids, chunk=4):
    """Prefill all sequences, `chunk` at a time; returns the first generated token of each."""
    import torch
    ops = _mod("ops")
    B, P = prompts.shape
    first = np.zeros(B, dtype=np.int32)
    for s in range(B):
        kv.add_sequence(s)
    for lo in range(0, B, chunk):
        sids = list(range(lo, min(B, lo + chunk)))
        kv.begin_forward(sids, [P] * len(sids))
        h = model.embed(torch.from_numpy(np.ascontiguousarray(prompts[sids].reshape(-1))))
        logits, _ = model["prefill_a0"](h, kv, adapter_ids[sids])
        kv.end_forward()
        first[sids] = ops.argmax(logits).cpu().numpy()
    return first


def profiled_gemv_traffic():
    """HBM bytes per GEMV launch from the committed rocprofv3 counter summary (FETCH_SIZE and WRITE_SIZE runs of
    `bench.py --probe`, each scaled by what the counter reads for a plain 256 MiB copy), weighted over the launch
    mix of one decode step; None when the summary is not there."""
    import re
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "gemv_gather_mm_pmc_fetch_write.txt")
    try:
        m = re.search(r"gemv_mix_hbm_bytes_per_launch=(\d+)", open(path).read())
    except OSError:
        return None
    return int(m.group(1)) if m else None


def traffic_from_counters(fetch_csv, write_csv, layers_step=32, layers_probe=2):
    """HBM bytes per GEMV launch, weighted over the launch mix of one decode step, from the two counter runs of
    `bench.py --probe` (rocprofv3 --pmc FETCH_SIZE, then --pmc WRITE_SIZE, --output-format csv): each counter is scaled
    by what it reads for the probe's plain 256 MiB device copy; the probe's GEMV launches come in the order qkv, o,
    gate_up, down per layer and lm_head last (a warm-up pass, then the timed one, over the probe's `layers_probe`
    layers; the GEMV launches of the decode steps at the end of the probe come after them and are not used), and a
    decode step issues each layer kind `layers_step` times and lm_head once.  Needs no GPU."""
    import csv
    per_kind = {}
    scale = {}
    for name, path in (("fetch", fetch_csv), ("write", write_csv)):
        rows = sorted(csv.DictReader(open(path)), key=lambda r: int(r["Dispatch_Id"]))
        copy = max(float(r["Counter_Value"]) for r in rows if "copyBuffer" in r["Kernel_Name"])
        scale[name] = 262144.0 / copy
        gemv = [r for r in rows if "gemv" in r["Kernel_Name"] and "pack" not in r["Kernel_Name"]]
        n_layers = layers_probe
        per_pass = 4 * n_layers + 1
        assert len(gemv) >= 2 * per_pass, (len(gemv), n_layers)
        block = gemv[per_pass:2 * per_pass]             # the second of the two passes over the mix
        kinds = ["qkv", "o", "gate_up", "down"] * n_layers + ["lm_head"]
        for k, r in zip(kinds, block):
            per_kind.setdefault(k, {}).setdefault(name, []).append(float(r["Counter_Value"]))
    out, tot, n = {}, 0.0, 0
    for k, d in per_kind.items():
        kib = sum(d["fetch"]) / len(d["fetch"]) * scale["fetch"] + sum(d["write"]) / len(d["write"]) * scale["write"]
        cnt = 1 if k == "lm_head" else layers_step
        out[k] = {"hbm_bytes_per_launch": kib * 1024, "launches_per_step": cnt}
        tot += cnt * kib * 1024
        n += cnt
    return {"scale_fetch": scale["fetch"], "scale_write": scale["write"], "per_kind": out, "gemv_mix_launches": n,
            "gemv_mix_hbm_bytes_per_launch": tot / n}


def gemv_event_timing(model, T, reps=3, per_kind=True):
    """Average duration of the weight-streaming GEMV over exactly the launches of one decode step (per layer: qkv with
    the adapters' A rows appended, o accumulating into the residual with the riders that expand its adapter delta (or,
    where the library does not serve the shape that way, with A rows appended), gate/up with the SiLU epilogue, down
    accumulating - o and down with their K split; then lm_head: 129 launches on 129 distinct matrices), issued back to
    back as in a decode step and bracketed by one event pair on the launch stream."""
    import torch
    ops, lm = _mod("ops"), _mod("_lib")
    lib = lm.lib()
    s = model.shape
    dev = model.device
    lt = model.lora_types[0]
    ks_ride = lib.mlora_gemv_delta_ride_ksplit(T, s.q_size, s.hidden_size, lt.r)
    ride = ks_ride > 0 and bool(lib.mlora_rope_attn_oshrink_ok(T, s.num_attention_heads, s.num_key_value_heads, s.head_dim, lt.r))
    ext = model.dense_lora_weights(0, with_o=not ride)
    il = model.interleaved_gate_up()
    x_h = ops.FragActivation(T, s.hidden_size, dev)
    x_q = ops.FragActivation(T, s.q_size, dev)
    x_i = ops.FragActivation(T, s.intermediate_size, dev)
    act = ops.FragActivation(T, s.intermediate_size, dev)
    for x in (x_h, x_q, x_i):
        x.data.normal_()                  # (the matrix cores' clock depends on the operand bits: no constant activations)
    n_ext = lt.n_adapters * lt.r
    resid = torch.zeros((T, s.hidden_size), dtype=torch.float32, device=dev)
    qkv = torch.empty((T, s.q_size + 2 * s.kv_size), dtype=torch.float16, device=dev)
    kq = lib.mlora_gemv_split_kq(T, s.hidden_size, s.q_size + 2 * s.kv_size, 3 * n_ext)   # K-range blocks of the appended q/k/v rows
    y2 = torch.empty((kq, T, 3 * n_ext), dtype=torch.float32, device=dev)
    logits = torch.empty((T, s.vocab_size), dtype=torch.float32, device=dev)
    F16, F32, STORE, ACC = lm.F16, lm.F32, lm.STORE, lm.ACCUMULATE
    H, I, Q, QKV = s.hidden_size, s.intermediate_size, s.q_size, s.q_size + 2 * s.kv_size
    launches, total_bytes = [], 0
    st = torch.cuda.current_stream().cuda_stream        # the stream the events below are recorded on
    # o and down split K over several workgroups as in the decode step; the partial results go to `part`
    ks_o, ks_d = lib.mlora_gemv_ksplit(T, Q, H + n_ext), lib.mlora_gemv_ksplit(T, I, H)
    part = torch.empty(3 * T * (H + n_ext), dtype=torch.float32, device=dev)
    # the riders' inputs: the o shrink as one share per attention head, every token on an adapter (T tokens over n_ad adapters)
    ids = (torch.arange(T, device=dev) % lt.n_adapters).to(torch.int32)
    vpart = torch.randn((s.num_attention_heads, T, lt.r), dtype=torch.float32, device=dev)
    used = min(T, lt.n_adapters)

    kinds, nbytes = [], []

    def add(kind, fn, rows, K, out_bytes):
        nonlocal total_bytes
        launches.append(fn)
        kinds.append(kind)
        nbytes.append(rows * K * 2 + T * K * 2 + out_bytes)
        total_bytes += nbytes[-1]

    for l in range(s.num_hidden_layers):
        wq, wo, wd, wg = ext[l]["qkv"], ext[l]["o"], ext[l]["down"], il[l]
        q_ext = wq.N - QKV
        o_ext = wo.N - H
        add("qkv", lambda wq=wq, q_ext=q_ext: lib.mlora_gemv_frag_split_kq(qkv.data_ptr(), y2.data_ptr(), kq, x_h.data.data_ptr(),
                                                                    wq.data.data_ptr(), T, H, QKV, q_ext, st),
            wq.N, H, T * QKV * 2 + kq * T * q_ext * 4)
        tab_o = lt.tables.get((l, "o_proj"))
        if ride and tab_o is not None:
            # base weight + riders: the weight, the token block, the residual read and written, the B rows of the adapters
            # in use and the head shares of the shrink (the slice partials and the delta rows are not counted, as before)
            add("o", lambda wo=wo, Bo=tab_o[1]: lib.mlora_gemv_frag_acc_ksplit_delta(resid.data_ptr(), part.data_ptr(), ks_ride, x_q.data.data_ptr(),
                                                                                 wo.data.data_ptr(), T, Q, H, vpart.data_ptr(), vpart.shape[0],
                                                                                 Bo.data_ptr(), ids.data_ptr(), lt.scaling, lt.r, lt.n_adapters, st),
                wo.N, Q, T * H * 8 + used * H * lt.r * 2 + vpart.numel() * 4)
        else:
            add("o", lambda wo=wo, o_ext=o_ext: lib.mlora_gemv_frag_acc_ksplit(resid.data_ptr(), y2.data_ptr(), part.data_ptr(), ks_o,
                                                                          x_q.data.data_ptr(), wo.data.data_ptr(), T, Q, H, o_ext,
                                                                          None, None, 0, None, 0, 0, st),
                wo.N, Q, T * H * 8 + T * o_ext * 4)
        add("gate_up", lambda wg=wg: lib.mlora_gemv_frag_silu(act.data.data_ptr(), x_h.data.data_ptr(), wg.data.data_ptr(), T, H, I, st),
            2 * I, H, T * I * 2)
        add("down", lambda wd=wd: lib.mlora_gemv_frag_acc_ksplit(resid.data_ptr(), None, part.data_ptr(), ks_d, x_i.data.data_ptr(),
                                                         wd.data.data_ptr(), T, I, H, 0, None, None, 0, None, 0, 0, st),
            H, I, T * H * 8)
    add("lm_head", lambda: lib.mlora_gemv_frag(logits.data_ptr(), F32, STORE, x_h.data.data_ptr(), model.lm_head.data.data_ptr(), T, H,
                                    s.vocab_size, st), s.vocab_size, H, T * s.vocab_size * 4)
    def timed(fns):
        """Median over the timed passes (the first pass is a warm-up and is left out)."""
        times = []
        for i in range(reps + 1):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for fn in fns:
                rc = fn()
                if rc != 0:
                    raise RuntimeError(lib.mlora_last_error().decode())
            e1.record()
            torch.cuda.synchronize()
            if i > 0 or reps == 0:
                times.append(e0.elapsed_time(e1))
        return float(np.median(times))

    best = timed(launches)
    # the same launches one kind at a time (each kind's launches back to back on their distinct matrices)
    per_kernel = {}
    for kind in ("qkv", "o", "gate_up", "down", "lm_head") if per_kind else ():
        idx = [i for i, k in enumerate(kinds) if k == kind]
        ms = timed([launches[i] for i in idx])
        by = sum(nbytes[i] for i in idx)
        per_kernel[kind] = {"launches": len(idx), "avg_us": 1e3 * ms / len(idx), "bytes_per_launch": by / len(idx),
                            "gbs": by / (ms * 1e-3) / 1e9, "frac": by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    return {"launches": len(launches), "avg_us": 1e3 * best / len(launches), "bytes_per_launch": total_bytes / len(launches),
            "gbs": total_bytes / (best * 1e-3) / 1e9, "per_kernel": per_kernel, "kinds": kinds}


def gather_mm_timing(n_sets=128, torch_init=False):
    """Isolated gather-matmul at the decode shape (T=64, K=N=4096, r=16, 32 adapters): n_sets distinct
    operand sets (> 1 GiB, larger than the 256 MB last-level cache) issued back to back.  torch_init fills the
    operands with torch's own generator (two launches per tensor instead of the counter-based generator's two
    dozen: for runs under a counter profiler, which records every launch)."""
    import torch
    ops, synth = _mod("ops"), _mod("synth")
    dev = "cuda:0"
    T, K, N, r, n_ad = 64, 4096, 4096, 16, 32
    ids = synth.randint(1, "gmm.ids", (T,), n_ad, dev)
    U = len(np.unique(ids.cpu().numpy()))
    sets = []
    for j in range(n_sets):
        if torch_init:
            sets.append((torch.randn((T, K), dtype=torch.float16, device=dev),
                         torch.randn((n_ad, r, K), dtype=torch.float16, device=dev) * 0.02,
                         torch.randn((n_ad, N, r), dtype=torch.float16, device=dev) * 0.02,
                         torch.randn((T, N), dtype=torch.float16, device=dev)))
            continue
        sets.append((synth.normal(1, f"b.x{j}", (T, K), 1.0, torch.float16, dev),
                     synth.normal(1, f"b.A{j}", (n_ad, r, K), 0.02, torch.float16, dev),
                     synth.normal(1, f"b.B{j}", (n_ad, N, r), 0.02, torch.float16, dev),
                     synth.normal(1, f"b.y{j}", (T, N), 1.0, torch.float16, dev)))
    ws = ops.gather_mm_workspace(T, K, r, dev)

    def all_calls():
        for x, A, B, y in sets:
            ops.gather_mm(y, x, A, B, ids, 1.0, ws)

    # The n_sets calls are recorded once into a HIP graph and replayed, so that the timed region holds the
    # kernels back to back (one launch per call) and not the Python interpreter between them.
    all_calls()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            all_calls()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 3
    e0.record()
    for _ in range(reps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / reps
    by = 2 * T * K + U * 2 * r * K + U * 2 * N * r + 4 * T * N + 4 * T
    # the same sets in ONE call (mlora_gather_mm_batch): what the op costs when it does not pay a launch per problem -
    # as a shrink pass and an expand pass over all sets (two launches; what the call does when it is given a
    # workspace), and as the single launch whose workgroups shrink into LDS and expand from there
    def batch_time(stream_passes):
        batch = ops.GatherMMBatch([(y, x, A, B) for x, A, B, y in sets], ids, 1.0, stream_passes=stream_passes)
        batch.run()
        torch.cuda.synchronize()
        best = None
        for _ in range(5):
            e0.record()
            batch.run()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3
            best = t if best is None else min(best, t)
        return {"us_per_set": best / n_sets * 1e6, "us_per_call": best * 1e6, "gbs": by * n_sets / best / 1e9,
                "frac_of_hbm_peak": by * n_sets / best / 1e9 / HBM_PEAK_GBS}

    two = batch_time(True)
    two["launches"] = 2
    one = batch_time(False)
    one["launches"] = 1
    return {"workload": "T=64 K=N=4096 r=16 n_ad=32", "distinct_adapters": U, "sets": n_sets,
            "bytes_per_call": by, "single_call_latency_us": sec / n_sets * 1e6,
            "one_call_per_set": {"us_per_call": sec / n_sets * 1e6, "gbs": by * n_sets / sec / 1e9,
                                 "frac_of_hbm_peak": by * n_sets / sec / 1e9 / HBM_PEAK_GBS},
            "one_call_for_all_sets": two, "one_launch_for_all_sets": one}


def gather_mm_cpu_baseline(reps=20):
    """The isolated gather-matmul on the host cores, in the reference's two forms (fp32, the oracle's restatements):
    GatherBMM (stack the per-request A and scaled B, two batched matmuls, add - `lora_gatherbmm_linear_layer.py:14-20`)
    and sequential (requests sorted by adapter, one matmul pair per adapter - `single_rank.py:39-50`)."""
    import torch
    import oracle
    synth = _mod("synth")
    c = synth.gather_mm_case(seed=1, T=64, K=4096, N=4096, r=16, n_ad=32, device="cpu")
    x, A, B, y = (c[k].float().numpy() for k in ("x", "A", "B", "y"))
    ids = c["ids"].numpy()
    order = np.argsort(ids, kind="stable")
    out = {}
    for name, fn in (("gather_bmm", lambda: oracle.gather_bmm_hf_ref(y[:, None, :], x[:, None, :], A, B, ids, 1.0)),
                     ("sequential", lambda: oracle.lora_sequential_ref(y[order], x[order], A, B, ids[order], 1.0))):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        out[name + "_us_per_call"] = (time.perf_counter() - t0) / reps * 1e6
    out["cores"] = os.cpu_count()
    out["kind"] = "port"
    return out


def cpu_baseline(wl, ctx, layers=2, steps=3):
    """The numpy oracle (fp32) on the host cores: `layers` of the 32 layers, `steps` decode steps of the
    whole batch at context `ctx` with a pre-filled cache, plus lm_head; scaled to the full depth."""
    import torch
    import oracle
    synth = _mod("synth")
    shape = synth.LlamaShape(**{**wl.shape.__dict__, "num_hidden_layers": layers})
    w = {k: v.float().numpy() for k, v in synth.base_weights(wl.seed, shape, torch.float16, "cpu").items()}
    lw = {k: v.float().numpy() for k, v in synth.lora_weights(wl.seed, shape, wl.lora, torch.float16, "cpu", tag="a0").items()}
    ref = oracle.LlamaRef(shape, w, lw, {"a0": wl.lora.scaling}, mode="fp32")
    B = wl.batch
    blocks = -(-(ctx + steps + 1) // 16)
    kv = ref.new_cache(B * blocks, 16, ctx + steps + 2)
    rng = np.random.default_rng(0)
    kv.k[:] = rng.standard_normal(kv.k.shape, dtype=np.float32)
    kv.v[:] = rng.standard_normal(kv.v.shape, dtype=np.float32)
    for s in range(B):
        kv.add_sequence(s)
        kv.tables[s] = [kv.free.pop(0) for _ in range(blocks)]
        kv.lens[s] = ctx
    toks = rng.integers(0, shape.vocab_size, B)
    ids = {"a0": wl.adapter_ids}
    t_steps = []
    for _ in range(steps):
        t0 = time.perf_counter()
        kv.begin_forward(list(range(B)), [1] * B)
        logits = ref.forward(toks, kv, ids)
        kv.end_forward()
        toks = logits.argmax(-1)
        t_steps.append(time.perf_counter() - t0)
    # split one step into the per-layer part and the head (embedding + final norm + lm_head)
    t0 = time.perf_counter()
    xn = oracle.rmsnorm_ref(w["embed_tokens"][toks], w["norm"], shape.rms_norm_eps)
    (xn @ w["lm_head"].T).argmax(-1)
    t_head = time.perf_counter() - t0
    t_step = float(np.median(t_steps))
    t_full = (t_step - t_head) * (wl.shape.num_hidden_layers / layers) + t_head
    return {"value": B / t_full, "unit": "tok/s", "cores": os.cpu_count(), "kind": "port",
            "sample": f"numpy fp32 oracle, {layers} of {wl.shape.num_hidden_layers} layers x {steps} decode steps of the "
                      f"32-request batch at context {ctx} (pre-filled cache) + lm_head, per-layer time scaled x"
                      f"{wl.shape.num_hidden_layers // layers}; threads = BLAS default on {os.cpu_count()} cores"}


def bench_c4_prefill(args, synth, llama):
    """The prefill configuration: 8 x 512 tokens grouped in adapter segments, 64 rank-64 adapters on all seven
    linears.  A step = one batched prefill pass over the whole model (fresh cache slots each step)."""
    import torch
    ops = _mod("ops")
    dev = "cuda:0"
    wl = synth.config4(num_layers=args.layers)
    s = wl.shape
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], dev)
    prompts = synth.prompts(wl)
    B, P = prompts.shape
    order = np.argsort(wl.adapter_ids, kind="stable")             # requests grouped into adapter segments
    tokens = torch.from_numpy(np.ascontiguousarray(prompts[order].reshape(-1)))
    wids = wl.adapter_ids[order]
    blocks = -(-P // wl.page_size)
    n_steps = args.warmup + args.steps
    kv = model.create_paged_kv_cache(B, B * blocks * wl.page_size, P, wl.page_size,
                                     free_pages=synth.permutation(wl.seed, "c4.pages", B * blocks), max_seq_len=blocks * wl.page_size)
    for b in range(B):
        kv.add_sequence(b)

    def step():
        for b in range(B):                                          # same pages again: every pass starts from empty sequences
            kv.lens[b] = 0
        kv.begin_forward(list(range(B)), [P] * B)
        logits, _ = model["prefill_a0"](model.embed(tokens), kv, wids)
        kv.end_forward()
        return logits

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    T = B * P
    L = s.num_hidden_layers
    per_layer = sum(int(np.prod(synth.linear_dims(s, p))) for p in synth.LINEARS)
    flops_base = 2.0 * T * per_layer * L
    flops_lora = sum(2.0 * T * wl.lora.r * sum(synth.linear_dims(s, p)) for p in wl.lora.targets) * L
    flops_attn = 2.0 * 2 * P * P / 2 * s.q_size * B * L            # causal QK^T and PV
    flops = flops_base + flops_lora + flops_attn + 2.0 * B * s.hidden_size * s.vocab_size
    print(json.dumps({
        "metric": "prefill tok/s, Llama-7B-shape 8x512 tokens, 64 rank-64 adapters on 7 linears", "value": T / dt, "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": wl.name, "layers": L, "tokens": T, "segments": int(len(np.unique(wids))), "rank": wl.lora.r,
                   "lora_targets": list(wl.lora.targets),
                   "base_gemm": "gemm_pp_kernel (this package), activations in fragment order"},
        "roofline": {"kernel": "whole prefill pass (base GEMMs 97 % of the flops)", "bound": "mfma", "achieved": flops / dt / 1e12,
                     "peak": 2500.0, "unit": "TFLOP/s", "frac": flops / dt / 1e12 / 2500.0, "traffic": None,
                     "flops_base": flops_base, "flops_lora": flops_lora, "flops_attention": flops_attn}}))


def bench_c5_decode(args, synth, llama):
    """The auto-batching stress configuration: 256 concurrent requests, Zipf(1.1) over 256 rank-16 adapters, context lengths uniform in
    128..2048 in a shuffled paged cache pre-filled with N(0,1) values; a step = one decode step of all 256 requests
    through the native step (one launch per operator beyond 64 sequences), replayed from a captured graph."""
    import torch
    dsm = _mod("decode_session")
    dev = "cuda:0"
    wl = synth.config5(num_layers=args.layers)
    s = wl.shape
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], dev)
    B = wl.batch
    n_steps = args.warmup + args.steps
    # requests in adapter order, as the front end batches them (`llama_seq_info.py:61-75` sorts by adapter type and weight id)
    order = np.argsort(wl.adapter_ids, kind="stable")
    adapter_ids = wl.adapter_ids[order]
    ctx = wl.ctx_lens[order].astype(np.int64)
    blocks = [int(-(-(c + n_steps + 1) // wl.page_size)) for c in ctx]
    n_pages = sum(blocks)
    kv = model.create_paged_kv_cache(B, n_pages * wl.page_size, 1, wl.page_size,
                                     free_pages=synth.permutation(wl.seed, "c5.pages", n_pages), max_seq_len=max(blocks) * wl.page_size)
    for l in range(s.num_hidden_layers):
        kv.k[l].normal_()
        kv.v[l].normal_()
    for b in range(B):
        kv.add_sequence(b)
    kv.begin_forward(list(range(B)), [int(c) for c in ctx])          # claims the pages of the pre-filled contexts
    kv.end_forward()
    first = synth.randint(wl.seed, "c5.first", (B,), s.vocab_size).numpy()
    if args.python_loop:
        sess = dsm.DecodeSession(model, kv, list(range(B)), {0: adapter_ids}, first, longest_first=not args.batch_order)
    else:
        sess = dsm.NativeDecodeSession(model, kv, list(range(B)), adapter_ids, first, use_graph=not args.no_graph,
                                       longest_first=not args.batch_order)
    for _ in range(args.warmup):
        sess.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sess.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    mean_ctx = float(ctx.sum()) + B * (args.warmup + (args.steps + 1) / 2.0)
    kv_bytes = mean_ctx * s.num_hidden_layers * 2 * s.kv_size * 2
    used = len(np.unique(wl.adapter_ids))
    lora_bytes = s.num_hidden_layers * len(wl.lora.targets) * used * 2 * wl.lora.r * (2 * 4096)
    step_bytes = model.weight_bytes_per_step() + kv_bytes + lora_bytes
    print(json.dumps({
        "metric": "decode tok/s, Llama-7B-shape 256 requests, Zipf over 256 rank-16 adapters, ctx 128-2048", "value": B / dt,
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": wl.name, "layers": s.num_hidden_layers, "batch": B, "adapters_in_use": used,
                   "total_context": int(ctx.sum()),
                   "host_loop": "python" if args.python_loop else ("mlora_decode_step" if args.no_graph else "hipGraph replay of mlora_decode_step"),
                   "base_gemm": "this package's kernels"},
        "roofline": {"kernel": "whole decode step (paged attention 91 % of the bytes)", "bound": "hbm",
                     "achieved": step_bytes / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": step_bytes / dt / 1e9 / HBM_PEAK_GBS, "traffic": None, "step_algorithmic_gb": step_bytes / 1e9}}))


def bench_c1_generate(args, synth, llama):
    """The reference's own CPU-runnable case, end to end through the auto-batching front end: 4 requests, each with
    its own rank-8 adapter, 128-token prompts, 32 greedy tokens per request (per-request prefill, batched decode).
    A step = one whole generate pass (requests registered, graph fused and executed).  The CPU baseline is the
    numpy oracle's `greedy_generate_ref` on the same prompts, timed once; the token ids of both are compared."""
    import torch
    ab, xg, lora = _mod("auto_batcher"), _mod("llama_exec_graph"), _mod("lora")
    dev = "cuda:0"
    wl = synth.config1()
    s = wl.shape
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, s, [wl.lora], dev)
    prompts = synth.prompts(wl)
    prompts = prompts.numpy() if hasattr(prompts, "numpy") else np.asarray(prompts)
    B, G = wl.batch, wl.gen_len
    n_pages = B * (-(-(wl.prompt_len + G) // wl.page_size) + 1)
    perm = synth.permutation(wl.seed, "c1.bench.pages", n_pages)

    def one_pass():
        b = ab.LlamaAutoBatcherClass()
        b.set_model(model)
        b.set_exec_config(xg.LlamaExecConfig(max_prompt_len=wl.prompt_len, max_gen_len=G, page_size=wl.page_size,
                                             dense_lora=not args.ids_lora, batch_prefill=args.batch_prefill))
        b.set_free_pages(perm)
        b.set_eos_token_id(None)
        outs = []
        for i in range(B):
            v = b.create_var(np.asarray(prompts[i], dtype=np.int32))
            b.set_adapter(lora.LoraConfig(r=wl.lora.r, alpha=wl.lora.scaling * wl.lora.r), wid=int(wl.adapter_ids[i]))
            outs.append(b.generate(v, max_gen_len=G))
        b.compile()
        b.execute()
        return [list(map(int, o.var)) for o in outs]

    warm = min(args.warmup, 3)
    steps = min(args.steps, 20)
    for _ in range(warm):
        got = one_pass()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        got = one_pass()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    out = {
        "metric": "end-to-end generate tok/s, 2-layer plumbing model, 4 requests x 4 rank-8 adapters, 128-token prompts, 32 greedy tokens",
        "value": B * G / dt, "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": wl.name, "layers": s.num_hidden_layers, "hidden": s.hidden_size, "batch": B,
                   "prompt_len": wl.prompt_len, "gen_len": G, "host_loop": "auto-batching front end, native decode step",
                   "dense_lora": not args.ids_lora, "batch_prefill": args.batch_prefill},
        "roofline": {"kernel": "whole generate pass (4 prefills + 31 decode steps; launch- and host-bound at this size)", "bound": "hbm",
                     "achieved": model.weight_bytes_per_step() * (B + G - 1) / dt / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": model.weight_bytes_per_step() * (B + G - 1) / dt / 1e9 / HBM_PEAK_GBS, "traffic": None}}
    if not args.no_cpu_baseline:
        import oracle
        w = {k: v.float().numpy() for k, v in synth.base_weights(wl.seed, s, torch.float16, "cpu").items()}
        lw = {k: v.float().numpy() for k, v in synth.lora_weights(wl.seed, s, wl.lora, torch.float16, "cpu", tag="a0").items()}
        ref = oracle.LlamaRef(s, w, lw, {"a0": wl.lora.scaling}, mode="mixed")
        t0 = time.perf_counter()
        exp = oracle.greedy_generate_ref(ref, prompts, {"a0": wl.adapter_ids}, G, n_pages, wl.page_size, perm)
        t_cpu = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": B * G / t_cpu, "unit": "tok/s", "cores": os.cpu_count(), "kind": "port",
                               "sample": "numpy oracle greedy_generate_ref, the whole workload once (fp32 arithmetic with fp16 "
                                         f"rounding where the HIP path stores fp16); threads = BLAS default on {os.cpu_count()} cores"}
        out["tokens_equal_oracle"] = bool(got == [list(map(int, e)) for e in exp])
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=32, help="model depth (32 = the benchmark configuration)")
    ap.add_argument("--batch", type=int, default=32,
                    help="c3_decode: concurrent requests (32 = the benchmark configuration; up to 64 run the native step)")
    ap.add_argument("--workload", default="c3_decode", choices=["c3_decode", "c4_prefill", "c5_decode", "c1_generate"],
                    help="c3_decode is the benchmark the metric is quoted on; the other two time the prefill and the "
                         "256-request stress configurations with the same harness")
    ap.add_argument("--shape", default="llama2_7b", choices=["llama2_7b", "llama31_8b"],
                    help="c3_decode: model shape (llama2_7b = the benchmark configuration; llama31_8b = the reference's default "
                         "model: grouped-query attention, 8 kv heads, vocabulary 128256)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ids-lora", action="store_true",
                    help="c1_generate: LlamaExecConfig.dense_lora = False (the ids-based shrink instead of the default dense one)")
    ap.add_argument("--batch-prefill", action="store_true", help="c1_generate: LlamaExecConfig.batch_prefill")
    ap.add_argument("--batch-order", action="store_true", help="c5_decode: keep the request order inside the batch (default: longest context first)")
    ap.add_argument("--no-extras", action="store_true", help="skip the per-kernel event timing and the gather-matmul stream")
    ap.add_argument("--python-loop", action="store_true", help="issue every kernel from Python instead of mlora_decode_step")
    ap.add_argument("--no-graph", action="store_true", help="call mlora_decode_step every step instead of replaying a captured graph")
    ap.add_argument("--probe", action="store_true",
                    help="counter probe: a few GEMV / gather-matmul launches and a plain 256 MiB copy of known size "
                         "(the calibration for FETCH_SIZE / WRITE_SIZE), no decode loop")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: read the counter CSVs of two `rocprofv3 --pmc` runs of `bench.py --probe` (FETCH_SIZE, "
                         "WRITE_SIZE) and print the HBM bytes per GEMV launch weighted over the launch mix of one decode step")
    args = ap.parse_args()
    if args.traffic_from:
        print(json.dumps(traffic_from_counters(*args.traffic_from)))
        return
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (every box here has one GPU, and the "
              f"path has no collective: requests would simply be partitioned over GPUs).", file=sys.stderr)
        sys.exit(2)

    import torch
    synth, llama, dsm = _mod("synth"), _mod("llama"), _mod("decode_session")
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.workload == "c4_prefill":
        return bench_c4_prefill(args, synth, llama)
    if args.workload == "c5_decode":
        return bench_c5_decode(args, synth, llama)
    if args.workload == "c1_generate":
        return bench_c1_generate(args, synth, llama)
    if args.probe:
        ops = _mod("ops")

        def stage(name):                     # progress on stderr: names the stage a profiler run stopped in
            print(f"[probe] {name}", file=sys.stderr, flush=True)

        stage("model")
        wl = synth.config3(num_layers=2)
        model = llama.LlamaForCausalLM.from_synthetic(wl.seed, wl.shape, [wl.lora], dev)
        src = torch.zeros(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        stage("copy")
        dst.copy_(src)                       # plain copy kernel: reads 256 MiB, writes 256 MiB
        stage("gemv")
        g = gemv_event_timing(model, wl.batch, reps=1, per_kind=False)    # exactly two passes over the mix: warm-up, timed
        stage("gather_mm")
        gm = gather_mm_timing(n_sets=24, torch_init=True)     # enough (set, adapter) pairs for the persistent shrink pass
        # the mid-size linear (gemm_mid_kernel) on a 256-token block: q/k/v and the accumulating o projection with its K slices
        stage("mid-size linears")
        x256 = ops.FragActivation.pack(torch.randn(256, wl.shape.hidden_size, device=dev, dtype=torch.float16))
        r256 = torch.zeros((256, wl.shape.hidden_size), dtype=torch.float32, device=dev)
        for _ in range(2):
            ops.linear(x256, model.layers[0]["qkv"])
            ops.linear(x256, model.layers[1]["gate_up"])
            ops.linear(x256, model.layers[0]["o"], out=r256, accumulate=True)
        # two native decode steps of the 2-layer model at the benchmark's cache geometry (32 sequences at context 520
        # in shuffled pages, cache pre-filled with N(0,1)): the fused RoPE + attention launch at its real shape
        stage("decode steps")
        blocks = -(-(wl.prompt_len + 16) // wl.page_size)
        kv = model.create_paged_kv_cache(wl.batch, wl.batch * blocks * wl.page_size, wl.prompt_len, wl.page_size,
                                         free_pages=synth.permutation(wl.seed, "c3.pages", wl.batch * blocks),
                                         max_seq_len=blocks * wl.page_size)
        for l in range(wl.shape.num_hidden_layers):
            kv.k[l].normal_()
            kv.v[l].normal_()
        for b in range(wl.batch):
            kv.add_sequence(b)
        kv.begin_forward(list(range(wl.batch)), [wl.prompt_len + 8] * wl.batch)
        kv.end_forward()
        sess = dsm.NativeDecodeSession(model, kv, list(range(wl.batch)), wl.adapter_ids, np.arange(wl.batch, dtype=np.int32),
                                       use_graph=False)
        sess.step()
        sess.step()
        torch.cuda.synchronize()
        print(json.dumps({"probe": True, "copy_bytes_each_way": 256 << 20, "gemv": g, "gather_matmul": gm,
                          "attention_kv_bytes_per_launch": int(wl.batch * (wl.prompt_len + 9.5) * 2 * wl.shape.kv_size * 2)}))
        return
    wl = synth.config3(num_layers=args.layers, batch=args.batch, shape=args.shape)
    t_setup = time.perf_counter()
    model = llama.LlamaForCausalLM.from_synthetic(wl.seed, wl.shape, [wl.lora], dev)
    prompts = synth.prompts(wl)
    total_new = args.warmup + args.steps + 1
    max_len = wl.prompt_len + total_new + 1
    blocks = -(-max_len // wl.page_size)
    perm = synth.permutation(wl.seed, "c3.pages", wl.batch * blocks)
    kv = model.create_paged_kv_cache(wl.batch, wl.batch * blocks * wl.page_size, wl.prompt_len, wl.page_size,
                                     free_pages=perm, max_seq_len=blocks * wl.page_size)
    first = prefill_all(model, kv, prompts, wl.adapter_ids)
    if args.python_loop:
        sess = dsm.DecodeSession(model, kv, list(range(wl.batch)), {0: wl.adapter_ids}, first)
    else:
        sess = dsm.NativeDecodeSession(model, kv, list(range(wl.batch)), wl.adapter_ids, first, use_graph=not args.no_graph)
    for _ in range(args.warmup):
        sess.step()
    torch.cuda.synchronize()
    t_setup = time.perf_counter() - t_setup

    ctx0 = wl.prompt_len + args.warmup
    t0 = time.perf_counter()
    for _ in range(args.steps):
        sess.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    tok_s = wl.batch * args.steps / dt
    dense = bool(getattr(sess, "dense_lora", False))
    # The timed session computes the LoRA shrink as extra rows of the base GEMV ("dense": taken while the adapters are
    # few; the session's and the front end's default, LlamaExecConfig.dense_lora).  The ids-based shrink (bit-identical to
    # the per-operator path, LlamaExecConfig.dense_lora = False) runs the same steps over the same pages once more, for the record.
    ids_ms = None
    if not args.python_loop and dense and not args.no_extras:
        for q in range(wl.batch):
            kv.lens[q] = wl.prompt_len
        s2 = dsm.NativeDecodeSession(model, kv, list(range(wl.batch)), wl.adapter_ids, first, use_graph=not args.no_graph, dense_lora=False)
        for _ in range(args.warmup):
            s2.step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            s2.step()
        torch.cuda.synchronize()
        ids_ms = (time.perf_counter() - t1) / args.steps * 1e3
        del s2

    # algorithmic bytes of one step at the mean context of the timed region
    mean_ctx = ctx0 + (args.steps + 1) / 2.0
    kv_bytes = wl.batch * mean_ctx * wl.shape.num_hidden_layers * 2 * wl.shape.kv_size * 2
    lora_bytes = wl.shape.num_hidden_layers * wl.lora.n_adapters * 2 * wl.lora.r * sum(sum(synth.linear_dims(wl.shape, p)) for p in wl.lora.targets)
    step_bytes = model.weight_bytes_per_step() + kv_bytes + lora_bytes

    out = {
        "metric": "decode tok/s, Llama-7B-shape bs32×16 LoRAs; gather-matmul HBM GB/s %peak" if args.shape == "llama2_7b"
                  else f"decode tok/s, Llama-3.1-8B-shape bs{wl.batch}×16 LoRAs",
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": wl.name, "layers": wl.shape.num_hidden_layers, "hidden": wl.shape.hidden_size,
                   "batch": wl.batch, "adapters": wl.lora.n_adapters, "rank": wl.lora.r, "lora_targets": list(wl.lora.targets),
                   "prompt_len": wl.prompt_len, "context_at_start": ctx0, "page_size": wl.page_size, "page_order": "random",
                   "host_loop": "python" if args.python_loop else ("native" if args.no_graph else "native+graph"),
                   "dense_lora": dense},
        "step_algorithmic_gb": step_bytes / 1e9,
        "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "setup_s": t_setup,
    }
    if ids_ms is not None:
        out["ids_shrink_variant"] = {"ms_per_step": ids_ms, "tok_s": wl.batch / (ids_ms * 1e-3), "dense_lora": False}
    if not args.no_extras:
        g = gemv_event_timing(model, wl.batch)
        out["roofline"] = {"kernel": "gemv_kernel / gemv_split_cu_kernel / gemv_silu_cu_kernel (fragment-ordered weights and activations, T=32; the 129 GEMV launches of one decode step: adapter A rows appended to qkv, expand riders in o, K split on o / down, SiLU epilogue on gate/up)", "bound": "hbm", "achieved": g["gbs"],
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": g["gbs"] / HBM_PEAK_GBS, "traffic": profiled_gemv_traffic(),
                           "launches_timed": g["launches"], "avg_launch_us": g["avg_us"],
                           "algorithmic_bytes_per_launch": g["bytes_per_launch"], "per_kernel": g["per_kernel"]}
        del sess, kv
        torch.cuda.empty_cache()
        out["gather_matmul"] = gather_mm_timing()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl, ctx0)
        if "gather_matmul" in out:
            out["gather_matmul"]["cpu_baseline"] = gather_mm_cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
