"""Pins the per-layer and model oracle (no GPU): closed forms, invariants, brute force on tiny inputs, and a
golden fixture computed with the locally installed `transformers` Llama (tests/golden/make_hf_llama_golden.py)."""
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import LlamaRef, PagedKVRef, attention_dense_ref, f16, rmsnorm_ref, rope_ref, rope_tables, silu_mul_ref
from conftest import load_pkg

HERE = os.path.dirname(os.path.abspath(__file__))


def test_rmsnorm_closed_forms():
    H = 64
    w = np.linspace(0.5, 1.5, H).astype(np.float32)
    x = np.ones((2, H), np.float32)                       # mean square 1 -> w / sqrt(1 + eps)
    np.testing.assert_allclose(rmsnorm_ref(x, w, 1e-5), np.broadcast_to(w / np.sqrt(1 + 1e-5), (2, H)), rtol=1e-6)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, H)).astype(np.float32)
    y = rmsnorm_ref(x, np.ones(H, np.float32), 0.0)
    np.testing.assert_allclose((y.astype(np.float64) ** 2).mean(-1), 1.0, rtol=1e-5)      # unit RMS out
    np.testing.assert_allclose(rmsnorm_ref(7 * x, w, 0.0), rmsnorm_ref(x, w, 0.0), rtol=1e-5)   # scale invariant


def test_silu_mul_scalar_formula():
    g = np.array([[-3.0, 0.0, 2.5]], np.float32)
    u = np.array([[2.0, 5.0, -1.0]], np.float32)
    exp = [[-3 / (1 + np.exp(3)) * 2, 0.0, 2.5 / (1 + np.exp(-2.5)) * -1]]
    np.testing.assert_allclose(silu_mul_ref(g, u), exp, rtol=1e-6)


def test_rope_invariants():
    D = 16
    cos, sin = rope_tables(D, 10000.0, 64)
    rng = np.random.default_rng(1)
    q = rng.standard_normal((1, 2, D)).astype(np.float32)
    k = rng.standard_normal((1, 2, D)).astype(np.float32)
    assert np.array_equal(rope_ref(q, [0], cos, sin), q)                                   # position 0 = identity
    for p in (1, 17, 63):
        np.testing.assert_allclose(np.linalg.norm(rope_ref(q, [p], cos, sin)), np.linalg.norm(q), rtol=1e-6)
    def dot(m, n):
        return float((rope_ref(q, [m], cos, sin) * rope_ref(k, [n], cos, sin)).sum())
    assert abs(dot(5, 2) - dot(40, 37)) < 1e-4 and abs(dot(5, 2) - dot(5, 3)) > 1e-3      # depends on m - n only
    # pairing convention: element i rotates with element i + D/2 by angle pos * theta^(-2i/D)
    e = np.zeros((1, 1, D), np.float32)
    e[0, 0, 1] = 1.0
    out = rope_ref(e, [3], cos, sin)[0, 0]
    ang = 3 * 10000.0 ** (-2 / D)
    np.testing.assert_allclose([out[1], out[1 + D // 2]], [np.cos(ang), np.sin(ang)], rtol=1e-6)
    assert np.count_nonzero(out) == 2


def _brute_attention(q, K, V, q_pos):
    n, Hq, D = q.shape
    g = Hq // K.shape[1]
    out = np.zeros((n, Hq, D))
    for i in range(n):
        for h in range(Hq):
            s = [sum(float(q[i, h, d]) * float(K[j, h // g, d]) for d in range(D)) / np.sqrt(D) for j in range(q_pos[i] + 1)]
            m = max(s)
            p = [np.exp(v - m) for v in s]
            z = sum(p)
            for d in range(D):
                out[i, h, d] = sum(p[j] * float(V[j, h // g, d]) for j in range(len(p))) / z
    return out


def test_attention_brute_force_tiny():
    rng = np.random.default_rng(2)
    ctx, Hq, Hkv, D = 40, 2, 1, 8
    K = rng.standard_normal((ctx, Hkv, D)).astype(np.float32)
    V = rng.standard_normal((ctx, Hkv, D)).astype(np.float32)
    q = rng.standard_normal((3, Hq, D)).astype(np.float32)
    pos = [0, 17, 39]
    np.testing.assert_allclose(attention_dense_ref(q, K, V, pos), _brute_attention(q, K, V, pos), rtol=1e-5, atol=1e-6)
    # several kv heads with several query heads each: query head h must read kv head h // (Hq // Hkv)
    ctx, Hq, Hkv, D = 21, 6, 3, 4
    K = rng.standard_normal((ctx, Hkv, D)).astype(np.float32)
    V = rng.standard_normal((ctx, Hkv, D)).astype(np.float32)
    q = rng.standard_normal((4, Hq, D)).astype(np.float32)
    pos = [3, 0, 20, 11]
    np.testing.assert_allclose(attention_dense_ref(q, K, V, pos), _brute_attention(q, K, V, pos), rtol=1e-5, atol=1e-6)


def _run_paged(perm, lens, chunks, seed=3, Hq=4, Hkv=2, D=8, round_fp16=False):
    """Feed each sequence's tokens in the given chunking; returns the concatenated outputs per sequence."""
    rng = np.random.default_rng(seed)
    cos, sin = rope_tables(D, 10000.0, 64)
    kv = PagedKVRef(1, len(perm), 16, Hkv, D, cos, sin, perm, round_fp16)
    data = [rng.standard_normal((n, Hq + 2 * Hkv, D)).astype(np.float32) for n in lens]
    outs = [[] for _ in lens]
    for s in range(len(lens)):
        kv.add_sequence(s)
    done = [0] * len(lens)
    for step in chunks:                      # step: list of (sid, n)
        sids, ns = [s for s, _ in step], [n for _, n in step]
        kv.begin_forward(sids, ns)
        qkv = np.concatenate([data[s][done[s]:done[s] + n] for s, n in step])
        out = kv.attention_with_fused_qkv(0, qkv, Hq)
        kv.end_forward()
        t = 0
        for s, n in step:
            outs[s].append(out[t:t + n])
            done[s] += n
            t += n
    return [np.concatenate(o) for o in outs], kv, data


def test_paged_equals_dense_and_is_permutation_invariant():
    lens = [40, 17, 33]
    one_shot = [[(0, 40), (1, 17), (2, 33)]]
    n_pages = 12
    a, kv_a, data = _run_paged(list(range(n_pages)), lens, one_shot)
    b, kv_b, _ = _run_paged(list(np.random.default_rng(5).permutation(n_pages)), lens, one_shot)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)                       # page permutation changes nothing, bit for bit
    # against dense attention on contiguous K/V
    cos, sin = rope_tables(8, 10000.0, 64)
    for s, n in enumerate(lens):
        pos = np.arange(n)
        q = rope_ref(data[s][:, :4], pos, cos, sin)
        k = rope_ref(data[s][:, 4:6], pos, cos, sin)
        v = data[s][:, 6:]
        exp = attention_dense_ref(q, k, v, pos).reshape(n, -1)
        np.testing.assert_allclose(a[s], exp, rtol=1e-6, atol=1e-6)
    # the walk itself: pages of a sequence, in order, hold its tokens
    Kc, _ = kv_b.gather(0, 2, 33)
    np.testing.assert_array_equal(Kc, rope_ref(data[2][:, 4:6], np.arange(33), cos, sin))


def test_cached_decode_equals_recompute():
    """Prefill + token-by-token decode with the cache == one causal pass over the whole sequence."""
    lens = [21, 35]
    n_pages = 8
    full, _, _ = _run_paged(list(range(n_pages)), lens, [[(0, 21), (1, 35)]])
    steps = [[(0, 16), (1, 30)]] + [[(0, 1), (1, 1)] for _ in range(5)]
    inc, _, _ = _run_paged(list(range(n_pages)), lens, steps)
    for x, y in zip(full, inc):
        np.testing.assert_allclose(x, y, rtol=1e-6, atol=1e-7)


def test_page_allocation_order_and_exhaustion():
    cos, sin = rope_tables(8, 10000.0, 64)
    kv = PagedKVRef(1, 4, 16, 1, 8, cos, sin, [2, 0, 3, 1])
    kv.add_sequence(7)
    kv.add_sequence(9)
    kv.begin_forward([7, 9], [17, 1])
    assert kv.tables == {7: [2, 0], 9: [3]}
    kv.end_forward()
    kv.begin_forward([9], [16])
    assert kv.tables[9] == [3, 1]
    kv.end_forward()
    with pytest.raises(AssertionError):
        kv.begin_forward([7], [16])


# ------------------------------------------------------------------ whole model
def _tiny(seed=123, lora=True, mode="fp32"):
    synth = load_pkg("synth")
    shape = synth.LlamaShape(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=2, head_dim=16, vocab_size=128)
    w = {k: v.numpy() for k, v in synth.base_weights(seed, shape, torch.float32, "cpu", std=0.2).items()}
    spec = synth.LoraSpec(r=8, alpha=4.0, n_adapters=3, targets=("q_proj", "v_proj", "down_proj"))
    lw = {k: v.numpy() * 5 for k, v in synth.lora_weights(seed, shape, spec, torch.float32, "cpu").items()} if lora else {}
    return shape, LlamaRef(shape, w, lw, {"a0": spec.scaling}, mode=mode), synth


def test_model_matches_transformers_golden():
    """Base decoder (no LoRA) against logits of the locally installed transformers Llama, eager attention, fp32."""
    synth = load_pkg("synth")
    g = np.load(os.path.join(HERE, "golden", "hf_llama_tiny.npz"))
    shape, ref, _ = _tiny(lora=False)
    ref.w["norm"] = (synth.normal(123, "norm", (64,), 0.3, torch.float32) + 1.0).numpy()
    for l in range(2):
        for p in ("input_layernorm", "post_attention_layernorm"):
            ref.w[f"layers.{l}.{p}"] = (synth.normal(123, f"layers.{l}.{p}", (64,), 0.3, torch.float32) + 1.0).numpy()
    ids = g["input_ids"]
    kv = ref.new_cache(4, 16, 32)
    for s in range(2):
        kv.add_sequence(s)
    kv.begin_forward([0, 1], [12, 12])
    logits = ref.forward(ids.reshape(-1), kv).reshape(2, 12, -1)
    kv.end_forward()
    np.testing.assert_allclose(logits, g["logits"], rtol=2e-4, atol=2e-4)


def test_greedy_batch_equals_single_and_recompute():
    shape, ref, synth = _tiny()
    prompts = synth.randint(1, "p", (3, 9), shape.vocab_size).numpy()
    ids = {"a0": np.array([2, -1, 0], np.int32)}
    batch = oracle.greedy_generate_ref(ref, prompts, ids, 6, 12)
    for b in range(3):
        alone = oracle.greedy_generate_ref(ref, prompts[b:b + 1], {"a0": ids["a0"][b:b + 1]}, 6, 4)
        assert alone[0] == batch[b]
    # KV-cached decode == argmax of a full re-forward over prompt + generated tokens
    b = 0
    seq = list(prompts[b]) + batch[b][:-1]
    kv = ref.new_cache(4, 16, 64)
    kv.add_sequence(0)
    kv.begin_forward([0], [len(seq)])
    logits = ref.forward(np.array(seq), kv, {"a0": np.full(len(seq), 2, np.int32)})
    kv.end_forward()
    assert list(logits.argmax(-1)[len(prompts[b]) - 1:]) == batch[b]
    assert all(len(o) == 6 for o in batch)


def test_greedy_stops_at_eos_and_respects_adapters():
    shape, ref, synth = _tiny()
    prompts = synth.randint(2, "p", (2, 7), shape.vocab_size).numpy()
    full = oracle.greedy_generate_ref(ref, prompts, {"a0": np.array([1, 1], np.int32)}, 8, 8)
    eos = full[0][2]
    cut = oracle.greedy_generate_ref(ref, prompts, {"a0": np.array([1, 1], np.int32)}, 8, 8, eos_token_id=eos)
    assert cut[0] == full[0][:full[0].index(eos) + 1] and len(cut[0]) < 8
    other = oracle.greedy_generate_ref(ref, prompts, {"a0": np.array([0, 2], np.int32)}, 8, 8)
    assert other != full                                  # the adapter index changes the output


def test_greedy_always_takes_one_decode_step_after_prefill():
    """The reference applies its finish rule only after a decode step (`llama_exec_graph.py:102-141`: the loop starts
    with every sequence), so max_gen_len = 1 still yields two tokens and an EOS that comes out of prefill does not end its sequence."""
    shape, ref, synth = _tiny()
    prompts = synth.randint(2, "p", (2, 7), shape.vocab_size).numpy()
    ids = {"a0": np.array([1, 1], np.int32)}
    full = oracle.greedy_generate_ref(ref, prompts, ids, 8, 8)
    one = oracle.greedy_generate_ref(ref, prompts, ids, 1, 8)
    assert one == [full[0][:2], full[1][:2]]
    # EOS as the prefill token is never looked at: only tokens produced by decode steps end a sequence
    eos = full[0][0]
    cut = oracle.greedy_generate_ref(ref, prompts, ids, 8, 8, eos_token_id=eos)
    for b in range(2):
        stop = next((i for i in range(1, len(full[b])) if full[b][i] == eos), len(full[b]) - 1)
        assert cut[b] == full[b][:stop + 1] and len(cut[b]) >= 2


def test_mixed_mode_rounds_storage_points_only():
    shape, ref32, synth = _tiny(mode="fp32")
    _, ref16, _ = _tiny(mode="mixed")
    for r in (ref32, ref16):
        r.w = {k: f16(v) for k, v in r.w.items()}
    ids = synth.randint(3, "p", (1, 10), shape.vocab_size).numpy().reshape(-1)
    outs = []
    for r in (ref32, ref16):
        kv = r.new_cache(2, 16, 32)
        kv.add_sequence(0)
        kv.begin_forward([0], [10])
        outs.append(r.forward(ids, kv, {"a0": np.zeros(10, np.int32)}))
        kv.end_forward()
        stored = kv.k[0][kv.tables[0][0]]
        if r.mode == "mixed":
            assert np.array_equal(stored, f16(stored))    # the cache holds fp16-representable values
    d = np.abs(outs[0] - outs[1]).max() / outs[0].std()
    assert 0 < d < 2e-2


def test_argmax_tie_rule():
    assert int(np.argmax(np.array([1.0, 3.0, 3.0, 2.0]))) == 1


def test_mixed_mode_rounds_fused_blocks_once():
    """`fuse_blocks` moves one rounding point of the mixed mode (base + delta rounded once for the tokens of an
    adapter-uniform block) and nothing else: the fp32 mode ignores it, tokens of mixed blocks keep two roundings,
    and the change stays within an fp16 step."""
    import oracle
    synth = load_pkg("synth")
    shape = synth.LlamaShape(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=4,
                             num_hidden_layers=1, head_dim=16, vocab_size=50)
    spec = synth.LoraSpec(r=8, alpha=16.0, n_adapters=3, targets=("q_proj", "gate_proj"))
    import torch
    w = {k: v.float().numpy() for k, v in synth.base_weights(5, shape, torch.float16, "cpu").items()}
    lw = {k: v.float().numpy() for k, v in synth.lora_weights(5, shape, spec, torch.float16, "cpu", tag="a0").items()}
    x = oracle.f16(np.random.default_rng(0).normal(size=(8, 64)).astype(np.float32))
    ids = np.array([1, 1, 1, 1, 2, 0, 2, 2], np.int32)            # block 0 (4 tokens) uniform, block 1 mixed
    outs = {}
    for mode in ("mixed", "fp32"):
        for fb in (None, 4):
            m = oracle.LlamaRef(shape, w, lw, {"a0": spec.scaling}, mode=mode)
            m.fuse_blocks = fb
            outs[(mode, fb)] = m._proj(x, 0, "q_proj", {"a0": ids})
    assert np.array_equal(outs[("fp32", None)], outs[("fp32", 4)])
    a, b = outs[("mixed", None)], outs[("mixed", 4)]
    assert np.array_equal(a[4:], b[4:]) and not np.array_equal(a[:4], b[:4])
    exact = outs[("fp32", None)]
    assert np.abs(b[:4] - exact[:4]).max() <= np.abs(a[:4] - exact[:4]).max() + 1e-7     # one rounding is no worse than two
    assert np.array_equal(b[:4], oracle.f16(exact[:4]))


def test_lora_wiring_equals_merged_weights():
    """Where the oracle places the LoRA delta (computed from the projection's own input - the normed residual, the
    attention output, the SiLU product - and added to that projection's output, on all 7 linears): one adapter bound to
    every token gives the logits of a model WITHOUT LoRA whose weights are W + scaling * B[a] . A[a]
    (`huggingface/custom_peft/lora_gatherbmm_linear_layer.py:21-22`, the merged branch; `tvm/llama_auto_batcher/lora.py:16-24`).
    A delta wired to the wrong input, the wrong projection or with a dropped scaling fails this; the model without
    the adapter differs visibly."""
    synth = load_pkg("synth")
    shape = synth.LlamaShape(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=2, head_dim=16, vocab_size=128)
    w = {k: v.numpy() for k, v in synth.base_weights(7, shape, torch.float32, "cpu", std=0.2).items()}
    targets = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")
    spec = synth.LoraSpec(r=8, alpha=4.0, n_adapters=3, targets=targets)
    lw = {k: v.numpy() * 5 for k, v in synth.lora_weights(7, shape, spec, torch.float32, "cpu").items()}
    a = 1
    ref = LlamaRef(shape, w, lw, {"a0": spec.scaling}, mode="fp32")
    merged = dict(w)
    for l in range(shape.num_hidden_layers):
        for p in targets:
            A, B = lw[f"layers.{l}.{p}.lora_A.a0"][a], lw[f"layers.{l}.{p}.lora_B.a0"][a]
            merged[f"layers.{l}.{p}"] = (w[f"layers.{l}.{p}"].astype(np.float64) + spec.scaling * B.astype(np.float64) @ A.astype(np.float64)).astype(np.float32)
    plain = LlamaRef(shape, merged, mode="fp32")
    bare = LlamaRef(shape, w, mode="fp32")
    ids = synth.randint(7, "p", (2, 11), shape.vocab_size).numpy()
    outs = []
    for r, tok in ((ref, {"a0": np.full(22, a, np.int32)}), (plain, None), (bare, None)):
        kv = r.new_cache(4, 16, 32)
        for s in range(2):
            kv.add_sequence(s)
        kv.begin_forward([0, 1], [11, 11])
        l0 = r.forward(ids.reshape(-1), kv, tok)
        kv.end_forward()
        kv.begin_forward([0, 1], [1, 1])                    # and one cached decode step
        l1 = r.forward(np.array([3, 5]), kv, None if tok is None else {"a0": np.full(2, a, np.int32)})
        kv.end_forward()
        outs.append(np.concatenate([l0, l1]))
    with_lora, with_merged, without = outs
    assert np.abs(with_lora - with_merged).max() <= 1e-4 * np.abs(with_merged).max()
    assert np.abs(with_lora - without).max() >= 0.1 * with_merged.std()


def test_depth_taps_equal_shallower_models():
    """`forward(..., tap_depths=)` keeps the logits of the model cut off after d layers: bit for bit what a d-layer model
    over the same weights returns for the same tokens (the GPU tests read the error at several depths off one pass)."""
    import dataclasses
    synth = load_pkg("synth")
    shape = synth.LlamaShape(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                             num_hidden_layers=5, head_dim=16, vocab_size=96)
    w = {k: v.numpy() for k, v in synth.base_weights(3, shape, torch.float32, "cpu", std=0.2).items()}
    spec = synth.LoraSpec(r=4, alpha=8.0, n_adapters=2, targets=("q_proj", "v_proj", "down_proj"))
    lw = {k: v.numpy() * 3 for k, v in synth.lora_weights(3, shape, spec, torch.float32, "cpu").items()}
    ids = synth.randint(3, "p", (13,), shape.vocab_size).numpy()
    tok = {"a0": np.array([0] * 6 + [1] * 4 + [-1] * 3, np.int32)}
    for mode in ("fp32", "mixed"):
        full = LlamaRef(shape, w, lw, {"a0": spec.scaling}, mode=mode)
        kv = full.new_cache(2, 16, 16)
        kv.add_sequence(0)
        kv.begin_forward([0], [13])
        top = full.forward(ids, kv, tok, logits_rows=[3, 12], tap_depths=(1, 3, 5))
        kv.end_forward()
        assert sorted(full.taps) == [1, 3]                  # the full depth is the return value itself
        for d in (1, 3, 5):
            cut = LlamaRef(dataclasses.replace(shape, num_hidden_layers=d), w, lw, {"a0": spec.scaling}, mode=mode)
            kvd = cut.new_cache(2, 16, 16)
            kvd.add_sequence(0)
            kvd.begin_forward([0], [13])
            exp = cut.forward(ids, kvd, tok, logits_rows=[3, 12])
            kvd.end_forward()
            assert np.array_equal(exp, top if d == 5 else full.taps[d]), (mode, d)
        assert np.abs(full.taps[1] - top).max() > 1e-3      # the depths do differ
