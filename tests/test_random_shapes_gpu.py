"""Seeded random model shapes and request mixes: the native decode step and the auto-batching front end against the
per-operator path, bit for bit.  The fixed-size tests cover the benchmark shapes; these cover the corners between them
(one kv head, 64-wide heads with a 128-wide q block, 1 to 64 requests, ranks 8 to 64, any subset of the seven
projections, one to seventy adapters, prompts that end on or next to a page boundary)."""
import numpy as np
import pytest
import torch

from conftest import load_pkg

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ALL = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")


def _prefill(model, kv, prompts, ids, ops):
    B, P = prompts.shape
    for s in range(B):
        kv.add_sequence(s)
    kv.begin_forward(list(range(B)), [P] * B)
    h = model.embed(torch.from_numpy(np.ascontiguousarray(prompts.reshape(-1))))
    tok = model._ids(B * P, {0: (None, np.repeat(ids, P).astype(np.int32))}) if model.lora_types else None
    logits = model.forward(h, kv, tok, model._last_rows(kv))
    kv.end_forward()
    return ops.argmax(logits).cpu().numpy()


def test_native_step_on_random_model_shapes():
    """Token ids and the whole K cache of `mlora_decode_step` (called per step and replayed from a graph, ids-based
    LoRA shrink) equal those of the per-operator path on 120 random configurations."""
    _native_step_equals_per_operator_path(20240611, 120, [1, 2, 5, 16, 17, 32, 33, 48, 64], [2, 5, 19])


def test_native_step_on_random_model_shapes_above_64_requests():
    """The same on 60 random configurations of 65 to 520 requests: one launch per operator on fragment-ordered
    activations (one, two or three 256-token blocks), K slices on o_proj and down_proj, grouped-query shapes, ranks 8 to
    64, the o projection's delta from head shares of the attention launch where the shape is served that way."""
    _native_step_equals_per_operator_path(20241126, 60, [65, 66, 80, 128, 129, 200, 256, 257, 300, 520], [2, 4])


def _native_step_equals_per_operator_path(rng_seed, cases, batches, step_counts):
    synth, llama, dsm, ops = load_pkg("synth"), load_pkg("llama"), load_pkg("decode_session"), load_pkg("ops")
    rng = np.random.default_rng(rng_seed)
    for case in range(cases):
        D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4])); Hq = Hkv * int(rng.choice([1, 2, 4]))
        hidden = int(rng.choice([256, 512, 1024])); inter = int(rng.choice([352, 704, 1408, 2816]))
        layers = int(rng.choice([1, 2, 3]))
        B = int(rng.choice(batches)); P = int(rng.choice([3, 15, 16, 30])); steps = int(rng.choice(step_counts))
        r = int(rng.choice([8, 16, 32, 64])); n_ad = int(rng.choice([1, 3, 8, 70])); k = int(rng.integers(0, 8))
        targets = tuple(np.array(ALL)[sorted(rng.choice(7, size=k, replace=False))]) if k else ()
        shape = synth.LlamaShape(hidden_size=hidden, intermediate_size=inter, num_attention_heads=Hq, num_key_value_heads=Hkv,
                                 num_hidden_layers=layers, head_dim=D, vocab_size=int(rng.choice([512, 1000, 4096])))
        seed = int(rng.integers(0, 1000))
        specs = [synth.LoraSpec(r=r, alpha=r / 2, n_adapters=n_ad, targets=targets)] if targets else []
        tag = (f"case {case}: B={B} P={P} steps={steps} hidden={hidden} inter={inter} Hq={Hq} Hkv={Hkv} D={D} L={layers} "
               f"r={r} n_ad={n_ad} targets={targets}")
        print(tag, flush=True)
        model = llama.LlamaForCausalLM.from_synthetic(seed, shape, specs, DEV)
        ids = rng.integers(-1, n_ad, size=B).astype(np.int32) if specs else np.full(B, -1, np.int32)
        prompts = rng.integers(0, shape.vocab_size, size=(B, P)).astype(np.int32)
        blocks = -(-(P + steps + 2) // 16)
        outs = []
        for kind in ("py", "graph", "nograph"):
            perm = np.random.default_rng(seed).permutation(B * blocks)
            kv = model.create_paged_kv_cache(B, B * blocks * 16, P, 16, free_pages=perm, max_seq_len=blocks * 16)
            first = _prefill(model, kv, prompts, ids, ops)
            if kind == "py":
                s = dsm.DecodeSession(model, kv, list(range(B)), {0: ids} if specs else {}, first)
            else:
                s = dsm.NativeDecodeSession(model, kv, list(range(B)), ids if specs else None, first,
                                            use_graph=(kind == "graph"), dense_lora=False)
            toks = np.stack([s.step().cpu().numpy().copy() for _ in range(steps)])
            outs.append((toks, kv.k.clone()))
        for toks, kc in outs[1:]:
            assert np.array_equal(toks, outs[0][0]), tag
            assert torch.equal(kc, outs[0][1]), tag


def test_dense_native_step_on_random_model_shapes():
    """The dense-shrink native step - adapter A rows inside the q/k/v (and down) GEMV, the o projection's shrink taken off
    the attention launch in head shares and expanded by riders of the o GEMV launch where the library serves the shape
    that way, appended A rows and the expand inside the RMSNorm where it does not - against the ids-based native step
    (which is bit-identical to the per-operator path, see above) on 60 random configurations: first-step logits agree to
    rounding-flip noise, tokens on every row whose top-2 margin is decided, cached keys to a few fp16 ulps.  Both forms of
    the o projection must have been drawn."""
    synth, llama, dsm, ops = load_pkg("synth"), load_pkg("llama"), load_pkg("decode_session"), load_pkg("ops")
    rng = np.random.default_rng(20240613)
    ride_seen = {True: 0, False: 0}
    for case in range(60):
        D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4, 8])); Hq = Hkv * int(rng.choice([1, 2, 4]))
        if case % 2 == 0:                                        # wide attention outputs: the o GEMV is K-split there, which is what carries riders
            Hq, Hkv, D = [(16, 4, 128), (16, 8, 128), (32, 8, 128), (16, 16, 128), (32, 8, 64), (32, 32, 64)][int(rng.integers(0, 6))]
        hidden = int(rng.choice([512, 1024, 2048, 4096])); inter = int(rng.choice([704, 1408, 2816]))
        layers = int(rng.choice([1, 2]))
        B = int(rng.choice([1, 3, 16, 17, 32, 33, 64])); P = int(rng.choice([3, 16, 30]))
        r = int(rng.choice([8, 16, 32, 64])); n_ad = int(rng.choice([1, 3, 8, 24]))
        extra = tuple(np.array(ALL)[sorted(rng.choice(7, size=int(rng.integers(0, 5)), replace=False))])
        targets = tuple(t for t in ALL if t == "o_proj" or t in extra)
        shape = synth.LlamaShape(hidden_size=hidden, intermediate_size=inter, num_attention_heads=Hq, num_key_value_heads=Hkv,
                                 num_hidden_layers=layers, head_dim=D, vocab_size=int(rng.choice([512, 1000])))
        seed = int(rng.integers(0, 1000))
        tag = (f"case {case}: B={B} P={P} hidden={hidden} inter={inter} Hq={Hq} Hkv={Hkv} D={D} L={layers} r={r} n_ad={n_ad} "
               f"targets={targets}")
        print(tag, flush=True)
        model = llama.LlamaForCausalLM.from_synthetic(seed, shape, [synth.LoraSpec(r=r, alpha=r / 2, n_adapters=n_ad, targets=targets)], DEV)
        ids = rng.integers(-1, n_ad, size=B).astype(np.int32)
        ids[rng.integers(0, B)] = n_ad - 1                       # at least one adapted row
        prompts = rng.integers(0, shape.vocab_size, size=(B, P)).astype(np.int32)
        blocks = -(-(P + 3) // 16)
        res = {}
        for kind in ("ids", "dense"):
            perm = np.random.default_rng(seed).permutation(B * blocks)
            kv = model.create_paged_kv_cache(B, B * blocks * 16, P, 16, free_pages=perm, max_seq_len=blocks * 16)
            first = _prefill(model, kv, prompts, ids, ops)
            sess = dsm.NativeDecodeSession(model, kv, list(range(B)), ids, first, use_graph=False, dense_lora=(kind == "dense"))
            tok = sess.step().cpu().numpy().copy()
            res[kind] = (tok, sess.buf["logits"].view(B, -1).clone(), kv.k.clone())
            if kind == "dense":
                assert sess.dense_lora, tag
                ride_seen[bool(sess.o_delta_ride)] += 1
        (ti, li, ki), (td, ld, kd) = res["ids"], res["dense"]
        err = float((ld - li).abs().max() / li.std())
        assert err <= 1e-2, (tag, err)
        assert float((ki.float() - kd.float()).abs().max()) <= 2.0 ** -5 * max(1.0, float(ki.float().abs().max())), tag
        top = torch.topk(li, 2, dim=-1).values
        decided = ((top[:, 0] - top[:, 1]) >= 2e-2 * li.std(dim=-1)).cpu().numpy()
        assert np.array_equal(td[decided], ti[decided]), tag
    print("o projection by riders / by appended rows:", ride_seen, flush=True)
    assert ride_seen[True] >= 10 and ride_seen[False] >= 10, ride_seen


def test_front_end_on_random_request_mixes():
    """Up to three adapter types (one scaling) and requests without adapter, per-request length limits and an
    optional EOS id: the front end returns the same token ids whether decode batches take the native / recorded
    step or one call per operator, on 80 random mixes."""
    synth, llama, ab, xg, lora = (load_pkg(m) for m in ("synth", "llama", "auto_batcher", "llama_exec_graph", "lora"))
    rng = np.random.default_rng(20240612)

    def run(model, prompts, req, max_gen, lens, perm, eos, native):
        b = ab.LlamaAutoBatcherClass()
        b.set_model(model)
        b.set_exec_config(xg.LlamaExecConfig(max_prompt_len=max(len(p) for p in prompts), max_gen_len=max_gen, page_size=16,
                                             native_decode=native, dense_lora=False))    # the bit-identical routing
        b.set_free_pages(perm)
        b.set_eos_token_id(eos)
        outs = []
        for p, (tid, wid), mg in zip(prompts, req, lens):
            v = b.create_var(np.asarray(p, dtype=np.int32))
            if tid >= 0:
                lt = model.lora_types[tid]
                b.set_adapter(lora.LoraConfig(lt.r, lt.scaling * lt.r), wid=wid)
            outs.append(b.generate(v, max_gen_len=mg))
        b.compile()
        b.execute()
        return [list(np.asarray(o.var).reshape(-1)) for o in outs]

    done = 0
    while done < 80:
        D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4])); Hq = Hkv * int(rng.choice([1, 2]))
        shape = synth.LlamaShape(hidden_size=int(rng.choice([256, 512])), intermediate_size=int(rng.choice([352, 704])),
                                 num_attention_heads=Hq, num_key_value_heads=Hkv, num_hidden_layers=int(rng.choice([1, 2])),
                                 head_dim=D, vocab_size=int(rng.choice([300, 1000])))
        ntypes = int(rng.choice([0, 1, 2, 3]))
        ranks = [int(x) for x in rng.choice([8, 16, 32, 64], size=ntypes, replace=False)] if ntypes else []
        specs = [synth.LoraSpec(r=r, alpha=r / 2, n_adapters=int(rng.choice([1, 2, 5])),
                                targets=tuple(np.array(ALL)[sorted(rng.choice(7, size=int(rng.integers(1, 8)), replace=False))]))
                 for r in ranks]
        seed = int(rng.integers(0, 1000))
        nreq = int(rng.choice([1, 2, 3, 7, 12, 20])); max_gen = int(rng.choice([1, 3, 10, 20]))
        req = []
        for _ in range(nreq):
            tid = int(rng.integers(-1, ntypes)) if ntypes else -1
            req.append((tid, int(rng.integers(0, specs[tid].n_adapters)) if tid >= 0 else -1))
        seen = []
        for tid, _ in req:
            if tid >= 0 and tid not in seen:
                seen.append(tid)
        if seen != list(range(len(seen))):       # the front end numbers adapter types by first use: keep the model's order
            continue
        model = llama.LlamaForCausalLM.from_synthetic(seed, shape, specs, DEV)
        prompts = [rng.integers(0, shape.vocab_size, size=int(rng.integers(1, 40))).astype(np.int32) for _ in range(nreq)]
        lens = [int(rng.integers(1, max_gen + 1)) for _ in range(nreq)]
        eos = int(rng.integers(0, shape.vocab_size)) if rng.random() < 0.3 else None
        pages = sum(-(-(len(p) + max_gen + 1) // 16) for p in prompts) + 2
        perm = np.random.default_rng(seed).permutation(pages)
        tag = f"mix {done}: nreq={nreq} ranks={ranks} max_gen={max_gen} eos={eos} Hq={Hq} Hkv={Hkv} D={D} req={req}"
        print(tag, flush=True)
        a = run(model, prompts, req, max_gen, lens, perm, eos, True)
        b_ = run(model, prompts, req, max_gen, lens, perm, eos, False)
        assert a == b_, tag
        # a decode step always follows prefill before the finish rule is applied (`llama_exec_graph.py:102-141`)
        assert all(2 <= len(o) <= max(mg, 2) for o, mg in zip(a, lens)), tag
        done += 1


def _rowmajor_caches(k, v, n_pages, Hkv, D):
    """[page, head, slot, d] float64 views of the fragment-ordered K pages and the token-minor V pages."""
    return (k.permute(0, 1, 4, 2, 3, 5).reshape(n_pages, Hkv, 16, D).double().cpu().numpy(),
            v.permute(0, 1, 3, 2).double().cpu().numpy())


def test_decode_attention_on_random_shapes():
    """RoPE + append + decode attention in one launch equals the two separate launches bit for bit (output and both
    caches), and the output equals a dense float64 softmax(q K^T / sqrt(D)) V over each sequence's pages to 3e-3, on
    100 random (batch, heads, group size, head width, context) draws with shuffled pages."""
    ops, kvm = load_pkg("ops"), load_pkg("kv_cache")
    rng = np.random.default_rng(20240613)
    for case in range(100):
        D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4, 8, 16, 32])); G = int(rng.choice([1, 2, 4, 8])); Hq = Hkv * G
        B = int(rng.choice([1, 2, 7, 16, 33, 64, 90])); maxctx = int(rng.choice([1, 17, 100, 300]))
        ctx = rng.integers(1, maxctx + 1, size=B)
        max_blocks = -(-maxctx // 16) + 1
        nb = [-(-int(c) // 16) for c in ctx]
        n_pages = sum(nb) + 3
        perm = rng.permutation(n_pages)
        table = np.full((B, max_blocks), -1, dtype=np.int32)
        o = 0
        for b in range(B):
            table[b, :nb[b]] = perm[o:o + nb[b]]
            o += nb[b]
        tag = f"case {case}: B={B} Hq={Hq} Hkv={Hkv} D={D} maxctx={maxctx}"
        print(tag, flush=True)
        cos, sin = kvm.rope_tables(D, 10000.0, max_blocks * 16)
        cos, sin = torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV)
        tab = torch.tensor(table, device=DEV)
        g = torch.Generator(device="cpu").manual_seed(case)
        k0 = torch.randn((n_pages, Hkv, D // 32, 4, 16, 8), generator=g).half().to(DEV)
        v0 = torch.randn((n_pages, Hkv, D, 16), generator=g).half().to(DEV)
        qkv = torch.randn((B, Hq + 2 * Hkv, D), generator=g).half().to(DEV)
        seqs = torch.arange(B, dtype=torch.int32, device=DEV)
        tpos = torch.tensor(ctx - 1, dtype=torch.int32, device=DEV)
        ctxl = torch.tensor(ctx, dtype=torch.int32, device=DEV)
        k1, v1, q1 = k0.clone(), v0.clone(), qkv.clone()
        ops.rope_kv_append(q1, k1, v1, tab, seqs, tpos, cos, sin, Hq, Hkv, D)
        want = ops.paged_attn_decode(q1, k1, v1, tab, seqs, ctxl, Hq, Hkv, D)
        k2, v2 = k0.clone(), v0.clone()
        got = ops.rope_attn_decode(qkv.clone(), k2, v2, tab, seqs, tpos, ctxl, cos, sin, Hq, Hkv, D)
        assert torch.equal(k1, k2) and torch.equal(v1, v2) and torch.equal(got, want), tag
        krm, vrm = _rowmajor_caches(k1, v1, n_pages, Hkv, D)
        out = want.view(B, Hq, D).double().cpu().numpy()
        qr = q1.double().cpu().numpy()
        for b in range(min(B, 6)):
            pages = table[b, :nb[b]]
            K = krm[pages].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :ctx[b]]
            V = vrm[pages].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :ctx[b]]
            sc = np.einsum("hgd,hkd->hgk", qr[b, :Hq].reshape(Hkv, G, D), K) / np.sqrt(D)
            sc -= sc.max(-1, keepdims=True)
            p = np.exp(sc)
            p /= p.sum(-1, keepdims=True)
            ref = np.einsum("hgk,hkd->hgd", p, V).reshape(Hq, D)
            assert np.abs(out[b] - ref).max() <= 3e-3 * np.abs(ref).max(), (tag, b)


def test_prefill_append_and_attention_on_random_segments():
    """Ragged prompt segments of several sequences in one call, some continuing a prefix that is already cached:
    the append writes exactly the rotated keys and the values of the new tokens into their page slots (bit-exact,
    nothing else touched, q rotated in place), and the causal attention output equals a dense float64 evaluation
    over each token's own sequence to 2e-3, on 80 random draws."""
    ops, kvm = load_pkg("ops"), load_pkg("kv_cache")
    rng = np.random.default_rng(20240614)
    for case in range(80):
        D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4, 8])); G = int(rng.choice([1, 2, 4, 8])); Hq = Hkv * G
        S = int(rng.choice([1, 2, 3, 7, 20])); maxlen = int(rng.choice([1, 5, 16, 17, 40, 130]))
        new = rng.integers(1, maxlen + 1, size=S)
        pre = rng.integers(0, int(rng.choice([1, 20, 70])), size=S)
        total = new + pre
        max_blocks = -(-int(total.max()) // 16) + 1
        nb = [-(-int(c) // 16) for c in total]
        n_pages = sum(nb) + 2
        perm = rng.permutation(n_pages)
        n_seq = S + 2
        rows = rng.permutation(n_seq)[:S]
        table = np.full((n_seq, max_blocks), -1, dtype=np.int32)
        o = 0
        for s in range(S):
            table[rows[s], :nb[s]] = perm[o:o + nb[s]]
            o += nb[s]
        T = int(new.sum())
        tok_seq = np.concatenate([np.full(new[s], rows[s]) for s in range(S)]).astype(np.int32)
        tok_pos = np.concatenate([np.arange(pre[s], total[s]) for s in range(S)]).astype(np.int32)
        tag = f"case {case}: S={S} T={T} Hq={Hq} Hkv={Hkv} D={D} new={new.tolist()} pre={pre.tolist()}"
        print(tag, flush=True)
        cos, sin = kvm.rope_tables(D, 10000.0, max_blocks * 16)
        cosd, sind = torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV)
        tab = torch.tensor(table, device=DEV)
        g = torch.Generator(device="cpu").manual_seed(1000 + case)
        k = torch.randn((n_pages, Hkv, D // 32, 4, 16, 8), generator=g).half().to(DEV)
        v = torch.randn((n_pages, Hkv, D, 16), generator=g).half().to(DEV)
        qkv = torch.randn((T, Hq + 2 * Hkv, D), generator=g).half().to(DEV)
        q_in = qkv.cpu().numpy()
        k0rm, v0rm = (a.astype(np.float16) for a in _rowmajor_caches(k, v, n_pages, Hkv, D))
        ts, tp = torch.tensor(tok_seq, device=DEV), torch.tensor(tok_pos, device=DEV)
        ops.rope_kv_append(qkv, k, v, tab, ts, tp, cosd, sind, Hq, Hkv, D)
        out = ops.paged_attn_prefill(qkv, k, v, tab, ts, tp, Hq, Hkv, D)
        krm, vrm = _rowmajor_caches(k, v, n_pages, Hkv, D)
        q_out = qkv.cpu().numpy()
        half = D // 2

        def rot(x, p):      # fp32 arithmetic on fp16 inputs, rounded once: element i pairs with element i + D/2
            x = x.astype(np.float32)
            c, s_ = cos[p].astype(np.float32), sin[p].astype(np.float32)
            a, b = x[..., :half], x[..., half:]
            return np.concatenate([a * c - b * s_, b * c + a * s_], axis=-1).astype(np.float16)

        kexp, vexp = k0rm.copy(), v0rm.copy()
        for t in range(T):
            pg, sl = table[tok_seq[t], tok_pos[t] // 16], tok_pos[t] % 16
            assert np.array_equal(q_out[t, :Hq], rot(q_in[t, :Hq], tok_pos[t])), (tag, "q", t)
            kexp[pg, :, sl] = rot(q_in[t, Hq:Hq + Hkv], tok_pos[t])
            vexp[pg, :, sl] = q_in[t, Hq + Hkv:]
        assert np.array_equal(kexp, krm.astype(np.float16)) and np.array_equal(vexp, vrm.astype(np.float16)), tag
        assert np.array_equal(q_out[:, Hq:], q_in[:, Hq:]), tag
        got = out.double().cpu().numpy().reshape(T, Hq, D)
        for t in range(T):
            L = tok_pos[t] + 1
            pages = table[tok_seq[t], :-(-L // 16)]
            K = krm[pages].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :L]
            V = vrm[pages].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :L]
            sc = np.einsum("kgd,kld->kgl", q_out[t, :Hq].astype(np.float64).reshape(Hkv, G, D), K) / np.sqrt(D)
            sc -= sc.max(-1, keepdims=True)
            p = np.exp(sc)
            p /= p.sum(-1, keepdims=True)
            ref = np.einsum("kgl,kld->kgd", p, V).reshape(Hq, D)
            assert np.abs(got[t] - ref).max() <= 2e-3 * max(np.abs(ref).max(), 1e-3), (tag, t)


def _rel(got, ref, floor=1e-3):
    scale = ref.abs().max().item()
    return ((got.double() - ref).abs() / torch.clamp(ref.abs(), min=floor * scale)).max().item()


def _gather_mm_float64(y0, x, A, B, ids, s):
    ref = y0.double().clone()
    for t in range(x.shape[0]):
        a = int(ids[t])
        if a >= 0:
            ref[t] += s * (B[a].double() @ (A[a].double() @ x[t].double()))
    return ref


def test_append_of_many_single_tokens_equals_the_small_batch_kernel():
    """A decode step of 65 to 300 sequences appends one token each through the 16-token tile kernel (tokens of a tile in
    different sequences and pages, slots anywhere in a page, a ragged last tile, rows without a valid sequence): the
    rotated q, and every byte of the K and V caches, equal those written by the per-token kernel that serves up to 64
    tokens, called on the same tokens in pieces."""
    ops, kvm = load_pkg("ops"), load_pkg("kv_cache")
    rng = np.random.default_rng(20241125)
    for case in range(12):
        D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 8])); Hq = Hkv * int(rng.choice([1, 4]))
        T = int(rng.choice([65, 96, 129, 200, 256, 300]))
        max_blocks = 6
        pos = rng.integers(0, max_blocks * 16, size=T)
        pos[: min(T, 8)] = [0, 15, 16, 31, 32, 47, 95, 80][: min(T, 8)]
        n_seq = T + 3
        rows = rng.permutation(n_seq)[:T].astype(np.int32)
        bad = rng.choice(T, size=3, replace=False)
        rows[bad[0]] = -1                       # no sequence
        pos[bad[1]] = max_blocks * 16 + 5       # position outside the table
        n_pages = n_seq * max_blocks + 1
        table = rng.permutation(n_pages - 1)[: n_seq * max_blocks].reshape(n_seq, max_blocks).astype(np.int32)
        table[rows[bad[2]], min(pos[bad[2]] // 16, max_blocks - 1)] = -1    # page never assigned
        tag = f"case {case}: T={T} Hq={Hq} Hkv={Hkv} D={D}"
        print(tag, flush=True)
        cos, sin = kvm.rope_tables(D, 10000.0, max_blocks * 16)
        cosd, sind = torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV)
        tab = torch.tensor(table, device=DEV)
        g = torch.Generator(device="cpu").manual_seed(77 + case)
        k0 = torch.randn((n_pages, Hkv, D // 32, 4, 16, 8), generator=g).half().to(DEV)
        v0 = torch.randn((n_pages, Hkv, D, 16), generator=g).half().to(DEV)
        qkv0 = torch.randn((T, Hq + 2 * Hkv, D), generator=g).half().to(DEV)
        ts, tp = torch.tensor(rows, device=DEV), torch.tensor(pos.astype(np.int32), device=DEV)
        k1, v1, q1 = k0.clone(), v0.clone(), qkv0.clone()
        ops.rope_kv_append(q1, k1, v1, tab, ts, tp, cosd, sind, Hq, Hkv, D)
        k2, v2, q2 = k0.clone(), v0.clone(), qkv0.clone()
        for a in range(0, T, 50):
            b = min(T, a + 50)
            ops.rope_kv_append(q2[a:b], k2, v2, tab, ts[a:b].contiguous(), tp[a:b].contiguous(), cosd, sind, Hq, Hkv, D)
        torch.cuda.synchronize()
        assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2), tag
        assert not torch.equal(k1, k0) and not torch.equal(v1, v0), tag


def test_lora_and_linear_kernels_on_random_shapes():
    """160 random draws over three families: the gather-matmul (1 to 2100 tokens: one-launch, vector and matrix-core
    paths; fp16 and fp32 y; row-major and fragment-ordered x; scattered ids and adapter segments) against a per-token
    float64 product; the decode linear (1 to 64 tokens, widths up to 32000, store fp16 / fp32 and accumulate)
    against the float64 product, fragment-ordered input equal to row-major input bit for bit; and the multi-rank /
    multi-projection calls against one single-rank call per (projection, rank bucket), bit for bit."""
    ops = load_pkg("ops")
    rng = np.random.default_rng(20240615)
    torch.manual_seed(20240615)
    rel, gm_ref = _rel, _gather_mm_float64
    n = 0
    for case in range(160):
        kind = rng.choice(["gm", "lin", "multi", "mproj"])
        if kind == "gm":
            T = int(rng.choice([1, 3, 16, 17, 33, 64, 65, 100, 256, 700, 1025, 1300, 2100]))
            K = int(rng.choice([64, 256, 520, 1024, 2048, 4096])); N = int(rng.choice([16, 48, 264, 1024, 4096, 4112]))
            r = int(rng.choice([8, 16, 32, 64])); n_ad = int(rng.choice([1, 2, 5, 17, 40]))
            ydt = torch.float16 if rng.random() < 0.6 else torch.float32
            x = torch.randn(T, K, device=DEV).half(); A = (torch.randn(n_ad, r, K, device=DEV) * 0.05).half(); B = (torch.randn(n_ad, N, r, device=DEV) * 0.05).half()
            ids = torch.from_numpy(rng.integers(-1, n_ad, size=T).astype(np.int32)).to(DEV)
            if T > 1024 and rng.random() < 0.7:     # adapter segments
                seg = int(rng.choice([16, 48, 64, 100])); ids = torch.from_numpy((np.arange(T) // seg % (n_ad + 1) - 1).astype(np.int32)).to(DEV)
            y0 = torch.randn(T, N, device=DEV).to(ydt); s = float(rng.choice([1.0, 0.5, 0.125]))
            tag = f"gm T={T} K={K} N={N} r={r} n_ad={n_ad} {ydt}"
            print(tag, flush=True)
            xin = ops.FragActivation.pack(x) if (T <= 64 and K % 32 == 0 and rng.random() < 0.5) else x
            got = ops.gather_mm(y0.clone(), xin, A, B, ids, s)
            e = rel(got, gm_ref(y0, x, A, B, ids.cpu().numpy(), s), 1e-2)
            tol = 2e-3 if ydt == torch.float16 else 5e-4
            assert e <= tol * 2, (tag, e)
        elif kind == "lin":
            T = int(rng.choice([1, 5, 16, 31, 32, 33, 48, 64])); K = int(rng.choice([64, 512, 1024, 2752, 4096, 11008])); N = int(rng.choice([36, 1024, 4096, 4352, 12288, 13056, 22016, 32000]))
            x = torch.randn(T, K, device=DEV).half(); W = (torch.randn(N, K, device=DEV) * 0.02).half()
            ref = x.double() @ W.double().T
            tag = f"lin T={T} K={K} N={N}"
            print(tag, flush=True)
            Wp = ops.PackedWeight(W); xf = ops.FragActivation.pack(x)
            y16 = ops.linear(xf, Wp); y32 = ops.linear(xf, Wp, out_dtype=torch.float32)
            r0 = torch.randn(T, N, device=DEV); racc = r0.clone(); ops.linear(xf, Wp, out=racc, accumulate=True)
            assert rel(y16, ref) <= 4e-3, tag
            assert rel(y32, ref, 1e-2) <= 1e-3, tag
            assert rel(racc, r0.double() + ref, 1e-2) <= 1e-3, tag
            assert torch.equal(y16, ops.linear(x, Wp)), tag
            e = 0
        else:
            T = int(rng.choice([2, 20, 40, 64, 90, 300, 1100])); K = int(rng.choice([256, 1024, 2048]))
            nb = int(rng.choice([1, 2, 3])); ranks = [int(rng.choice([8, 16, 32, 64])) for _ in range(nb)]; nads = [int(rng.choice([1, 3, 6])) for _ in range(nb)]
            x = torch.randn(T, K, device=DEV).half()
            tb = torch.from_numpy(rng.integers(-1, nb, size=T).astype(np.int32)).to(DEV)
            ta = torch.from_numpy(np.array([rng.integers(0, nads[b]) if b >= 0 else -1 for b in tb.cpu().numpy()], dtype=np.int32)).to(DEV)
            cols = [int(rng.choice([64, 128, 512])) for _ in range(3 if kind == "mproj" else 1)]
            offs = [0] + list(np.cumsum(cols)[:-1])
            ydt = torch.float16 if rng.random() < 0.6 else torch.float32
            y0 = torch.randn(T, sum(cols), device=DEV).to(ydt)
            projs = [[None if (rng.random() < 0.15 and nb > 1) else ((torch.randn(na, r, K, device=DEV) * 0.05).half(), (torch.randn(na, c, r, device=DEV) * 0.05).half(), float(rng.choice([1.0, 0.25])))
                      for r, na in zip(ranks, nads)] for c in cols]
            tag = f"{kind} T={T} K={K} cols={cols} ranks={ranks} nads={nads} {ydt}"
            print(tag, flush=True)
            xin = ops.FragActivation.pack(x) if (T <= 64 and rng.random() < 0.5) else x
            if kind == "mproj":
                got = ops.gather_mm_multi_proj(y0.clone(), xin, projs, offs, cols, tb, ta)
            else:
                got = ops.gather_mm_multi(y0.clone(), xin, projs[0], tb, ta)
            want = y0.clone()
            for p, (c0, c) in enumerate(zip(offs, cols)):
                for b, bk in enumerate(projs[p]):
                    if bk is not None:
                        ops.gather_mm(want[:, c0:c0 + c], xin, bk[0], bk[1], torch.where(tb == b, ta, torch.full_like(ta, -1)), bk[2])
            assert torch.equal(got, want), tag
            e = 0
        n += 1
