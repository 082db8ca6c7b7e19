"""Pins the gather-matmul oracle (no GPU): brute force, the reference's own strategy equivalences,
dense-library special cases and integer exactness.  The reference holds no golden vectors for this path;
its only checks are `np.allclose` between batching strategies on unseeded data
(`tvm/lora_only/single_rank.py:254` atol 1e-4, `tvm/lora_only/case_study/multiple_ranks.py:382-383` atol 1e-5)."""
import numpy as np

import oracle
from oracle import gather_mm_ref, max_rel_err


def _case(T=12, K=96, N=40, r=8, n_ad=5, seed=0, sorted_ids=False):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, n_ad, T)
    if sorted_ids:
        ids = np.sort(ids)
    return dict(x=rng.standard_normal((T, K)).astype(np.float32), A=(0.1 * rng.standard_normal((n_ad, r, K))).astype(np.float32),
                B=(0.1 * rng.standard_normal((n_ad, N, r))).astype(np.float32), y=rng.standard_normal((T, N)).astype(np.float32),
                ids=ids.astype(np.int32))


def test_brute_force_per_token_float64():
    c = _case()
    got = gather_mm_ref(c["y"], c["x"], c["A"], c["B"], c["ids"], 0.5, dtype=np.float64)
    for t in range(len(c["ids"])):
        a = c["ids"][t]
        exp = c["y"][t].astype(np.float64)
        for n in range(c["B"].shape[1]):
            acc = 0.0
            for j in range(c["A"].shape[1]):
                v = sum(float(c["A"][a, j, k]) * float(c["x"][t, k]) for k in range(c["x"].shape[1]))
                acc += float(c["B"][a, n, j]) * v
            exp[n] += 0.5 * acc
        np.testing.assert_allclose(got[t], exp, rtol=1e-12, atol=1e-12)


def test_equals_sequential_and_gatherbmm_strategies():
    """The reference's check: sequential == GatherBMM (single_rank.py:254), here also == the per-token oracle."""
    c = _case(T=16, sorted_ids=True)
    base = c["y"]
    seq = oracle.lora_sequential_ref(base, c["x"], c["A"], c["B"], c["ids"], 2.0)
    bmm = oracle.gather_bmm_hf_ref(base[:, None, :], c["x"][:, None, :], c["A"], c["B"], c["ids"], 2.0)[:, 0]
    tok = gather_mm_ref(base, c["x"], c["A"], c["B"], c["ids"], 2.0)
    assert np.allclose(seq, bmm, atol=1e-4) and np.allclose(seq, tok, atol=1e-4)
    assert max_rel_err(tok, seq) < 1e-4 and max_rel_err(bmm, seq) < 1e-4     # fp32 evaluation-order noise only


def test_identical_ids_reduce_to_dense_matmul():
    c = _case()
    ids = np.full_like(c["ids"], 3)
    got = gather_mm_ref(c["y"], c["x"], c["A"], c["B"], ids, 1.0, dtype=np.float64)
    exp = c["y"] + c["x"].astype(np.float64) @ c["A"][3].astype(np.float64).T @ c["B"][3].astype(np.float64).T
    np.testing.assert_allclose(got, exp, rtol=1e-12)


def test_zero_B_and_negative_ids_leave_rows_bit_identical():
    c = _case()
    assert np.array_equal(gather_mm_ref(c["y"], c["x"], c["A"], np.zeros_like(c["B"]), c["ids"], 1.0), c["y"])
    ids = c["ids"].copy()
    ids[::2] = -1
    got = gather_mm_ref(c["y"], c["x"], c["A"], c["B"], ids, 1.0)
    assert np.array_equal(got[::2], c["y"][::2]) and not np.array_equal(got[1::2], c["y"][1::2])


def test_rank_padding_and_rank_splitting():
    """Zero-padding the rank is a no-op and summing rank chunks equals the full rank
    (multiple_ranks.py:188-191 'padded', :126-137 'splitted', checked at :382-383)."""
    c = _case(r=8)
    full = gather_mm_ref(c["y"], c["x"], c["A"], c["B"], c["ids"], 1.0, dtype=np.float64)
    Ap = np.concatenate([c["A"], np.zeros_like(c["A"])], axis=1)
    Bp = np.concatenate([c["B"], np.zeros_like(c["B"])], axis=2)
    np.testing.assert_allclose(gather_mm_ref(c["y"], c["x"], Ap, Bp, c["ids"], 1.0, dtype=np.float64), full, rtol=1e-12)
    part = c["y"].astype(np.float64)
    for lo in (0, 4):
        part = gather_mm_ref(part, c["x"], c["A"][:, lo:lo + 4], c["B"][:, :, lo:lo + 4], c["ids"], 1.0, dtype=np.float64)
    np.testing.assert_allclose(part, full, rtol=1e-12)


def test_token_permutation_equivariance():
    c = _case()
    perm = np.random.default_rng(9).permutation(len(c["ids"]))
    a = gather_mm_ref(c["y"], c["x"], c["A"], c["B"], c["ids"], 1.0)
    b = gather_mm_ref(c["y"][perm], c["x"][perm], c["A"], c["B"], c["ids"][perm], 1.0)
    np.testing.assert_allclose(a[perm], b, rtol=1e-6, atol=1e-6)


def test_scale_on_B_equals_scale_after():
    """HF scales B before the bmm (lora_gatherbmm_linear_layer.py:17), TVM scales the result (lora.py:23-24)."""
    c = _case()
    a = gather_mm_ref(c["y"], c["x"], c["A"], c["B"] * np.float32(0.5), c["ids"], 1.0)
    b = gather_mm_ref(c["y"], c["x"], c["A"], c["B"], c["ids"], 0.5)
    assert max_rel_err(a, b) < 1e-5


def test_take_matmul_tvm_orientation():
    """take_matmul (fuse_take_matmul.py:85-105) on W [n_ad, K, J] equals numpy fancy indexing + matmul."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((6, 1, 32))
    W = rng.standard_normal((4, 32, 8))
    idx = np.array([3, 0, 0, 2, 1, 3])
    got = oracle.take_matmul_ref(x, W, idx, dtype=np.float64)
    for b in range(6):
        np.testing.assert_allclose(got[b], x[b] @ W[idx[b]], rtol=1e-12)
    # two chained take_matmuls with transposed tables == the PEFT-orientation oracle
    c = _case(T=6, K=32, N=8, r=4, n_ad=4)
    v = oracle.take_matmul_ref(c["x"][:, None, :], c["A"].transpose(0, 2, 1), c["ids"], np.float64)
    y = oracle.take_matmul_ref(v, c["B"].transpose(0, 2, 1), c["ids"], np.float64)[:, 0] * 0.5
    np.testing.assert_allclose(c["y"] + y, gather_mm_ref(c["y"], c["x"], c["A"], c["B"], c["ids"], 0.5, np.float64), rtol=1e-10)


def test_write_tensor_part_and_mixed_delta():
    """write_tensor_part (write_tensor_part.py:3-20) and the mixed path (compile_tvm.py:135-155):
    per-type gather -> delta -> scatter equals one per-token pass with -1 for absent types."""
    X = np.arange(24, dtype=np.float32).reshape(6, 1, 4)
    Y = -np.ones((2, 1, 4), np.float32)
    Z = oracle.write_tensor_part_ref(X, Y, [4, 1])
    assert np.array_equal(Z[[0, 2, 3, 5]], X[[0, 2, 3, 5]]) and np.all(Z[[4, 1]] == -1)
    c0, c1 = _case(T=6, r=4, seed=3), _case(T=6, r=8, seed=4)
    h = c0["x"]
    types = [dict(A=c0["A"], B=c0["B"], scaling=0.5, sids=[1, 4], wids=[2, 0]),
             dict(A=c1["A"], B=c1["B"], scaling=0.25, sids=[0, 5, 3], wids=[1, 1, 4])]
    delta = oracle.mixed_delta_ref(h, types)
    ids0 = np.array([-1, 2, -1, -1, 0, -1])
    ids1 = np.array([1, -1, -1, 4, -1, 1])
    exp = gather_mm_ref(np.zeros_like(delta), h, c0["A"], c0["B"], ids0, 0.5)
    exp = gather_mm_ref(exp, h, c1["A"], c1["B"], ids1, 0.25)
    np.testing.assert_allclose(delta, exp, rtol=1e-6, atol=1e-7)
    assert np.all(delta[2] == 0)


def test_combined_strategy_equals_sequential():
    """The reference's own check (`two_ranks_with_combine.py:1090`: combined == sequential) on its table and index
    construction (`:649-653`, `:1013-1014`): large-rank requests first, then small-rank requests, every request with
    its own adapter ("distinct"), r_mult small adapters sharing one combined slot."""
    rng = np.random.default_rng(11)
    K, N, r_large, r_small = 48, 40, 8, 2
    bl, bs = 3, 8                                             # requests of the large / small rank
    A_l, B_l = rng.standard_normal((bl, r_large, K)), rng.standard_normal((bl, N, r_large))
    A_s, B_s = rng.standard_normal((bs, r_small, K)), rng.standard_normal((bs, N, r_small))
    x = rng.standard_normal((bl + bs, K))
    A_c, B_c = oracle.combined_tables_ref(A_l, B_l, A_s, B_s)
    r_mult = r_large // r_small
    assert A_c.shape == (bl + bs // r_mult, r_large, K) and B_c.shape == (bl + bs // r_mult, N, r_large)
    xids = [i for i in range(bl) for _ in range(r_large)] + [i for i in range(bl, bl + bs) for _ in range(r_small)]
    wids = np.arange(bl + bs // r_mult)
    got = oracle.lora_combined_ref(x, A_c, B_c, xids, wids, 2.0, dtype=np.float64)
    # sequential: each request against its own adapter of its own rank
    exp = np.zeros((bl + bs, N))
    for t in range(bl):
        exp[t] = 2.0 * (B_l[t] @ (A_l[t] @ x[t]))
    for t in range(bs):
        exp[bl + t] = 2.0 * (B_s[t] @ (A_s[t] @ x[bl + t]))
    np.testing.assert_allclose(got, exp, rtol=1e-12, atol=1e-12)
    # and the per-token oracle on the two types gives the same rows
    ids_l = np.array(list(range(bl)) + [-1] * bs)
    ids_s = np.array([-1] * bl + list(range(bs)))
    two = gather_mm_ref(gather_mm_ref(np.zeros((bl + bs, N)), x, A_l, B_l, ids_l, 2.0, np.float64), x, A_s, B_s, ids_s, 2.0, np.float64)
    np.testing.assert_allclose(two, exp, rtol=1e-12, atol=1e-12)


def test_integer_payload_gather_is_exact():
    """With integer-valued operands the result is exact: the index gather itself is what is tested."""
    rng = np.random.default_rng(7)
    T, K, N, n_ad = 20, 16, 8, 6
    x = rng.integers(-3, 4, (T, K)).astype(np.float32)
    A = rng.integers(-2, 3, (n_ad, 4, K)).astype(np.float32)
    B = rng.integers(-2, 3, (n_ad, N, 4)).astype(np.float32)
    ids = rng.integers(0, n_ad, T)
    got = gather_mm_ref(np.zeros((T, N), np.float32), x, A, B, ids, 1.0)
    exp = np.einsum("tnj,tjk,tk->tn", B[ids].astype(np.int64), A[ids].astype(np.int64), x.astype(np.int64))
    assert np.array_equal(got, exp.astype(np.float32))


def test_max_rel_err_metric():
    assert max_rel_err([1.0, 0.0], [1.0, 0.0]) == 0.0
    assert abs(max_rel_err([1.001, 0.0], [1.0, 0.0]) - 1e-3) < 1e-9
    assert abs(max_rel_err([1.0, 1e-6], [1.0, 0.0]) - 1e-3) < 1e-9     # floor = 1e-3 * max|ref|
