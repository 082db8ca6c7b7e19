"""CPU oracle for the adapter-indexed LoRA delta (test infrastructure, not a product path).

Layouts are PEFT's: A [n_ad, r, K] (`lora_A.weight [r,K]` stacked), B [n_ad, N, r]
(`lora_B.weight [N,r]` stacked), as gathered in
`huggingface/custom_peft/lora_gatherbmm_linear_layer.py:16-17`.  The TVM path stores the
transposes (`tvm/llama_auto_batcher/compile_tvm.py:313`); `take_matmul_ref` follows that one.
"""
from __future__ import annotations

import numpy as np


def max_rel_err(got, ref, floor: float = 1e-3) -> float:
    """max |got-ref| / max(|ref|, floor * max|ref|): relative error with a floor that avoids 0/0."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    scale = np.maximum(np.abs(ref), floor * max(np.abs(ref).max(), 1e-30))
    return float((np.abs(got - ref) / scale).max()) if ref.size else 0.0


def gather_mm_ref(y0, x, A, B, ids, scaling=1.0, dtype=np.float32):
    """y[t] = y0[t] + scaling * B[ids[t]] @ (A[ids[t]] @ x[t]); ids[t] < 0 leaves row t untouched.

    Per-token form of `lora_gatherbmm_linear_layer.py:14-20` (result = base + bmm(bmm(x, A^T), B^T))
    and of `compile_tvm.py:106-112` (take -> matmul -> matmul -> * scaling).
    """
    x = np.asarray(x, dtype=dtype)
    A = np.asarray(A, dtype=dtype)
    B = np.asarray(B, dtype=dtype)
    y = np.array(y0, dtype=dtype, copy=True)
    ids = np.asarray(ids)
    s = dtype(scaling)
    for a in np.unique(ids):
        if a < 0:
            continue
        tok = np.nonzero(ids == a)[0]
        v = x[tok] @ A[a].T            # [n, r]
        y[tok] += s * (v @ B[a].T)     # [n, N]
    return y


def gather_bmm_hf_ref(base, x, A, B, ids, scaling):
    """Literal restatement of the hot branch of `GatherBMMLinear.forward`
    (`lora_gatherbmm_linear_layer.py:14-20`): stack A and (B * scaling) per request, two bmm, add.
    x is [B, S, K] (one adapter per request), base is [B, S, N]."""
    x = np.asarray(x, dtype=np.float32)
    A_g = np.stack([np.asarray(A[i], np.float32) for i in ids], 0).transpose(0, 2, 1)        # [B, K, r]
    B_g = np.stack([np.asarray(B[i], np.float32) * np.float32(scaling) for i in ids], 0).transpose(0, 2, 1)
    out = np.matmul(np.matmul(x, A_g), B_g)
    return np.asarray(base, np.float32) + out


def lora_sequential_ref(base, x, A, B, ids, scaling):
    """The 'sequential' strategy (`tvm/lora_only/single_rank.py:39-50`; PEFT's per-adapter loop):
    requests sorted by adapter, split at adapter boundaries, one matmul pair per adapter, concatenated."""
    x = np.asarray(x, dtype=np.float32)
    ids = np.asarray(ids)
    assert np.all(np.diff(ids) >= 0), "sequential strategy expects requests sorted by adapter"
    bounds = [0] + [i for i in range(1, len(ids)) if ids[i] != ids[i - 1]] + [len(ids)]
    outs = []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        a = ids[lo]
        outs.append((x[lo:hi] @ np.asarray(A[a], np.float32).T @ np.asarray(B[a], np.float32).T) * np.float32(scaling))
    return np.asarray(base, np.float32) + np.concatenate(outs, 0)


def take_matmul_ref(x, W, idx, dtype=np.float32):
    """out[i0,i1,j] = sum_k x[i0,i1,k] * W[idx[i0],k,j]  (`tvm/custom/fuse_take_matmul.py:85-105`).
    W is in the TVM orientation [n_ad, K, J]."""
    x = np.asarray(x, dtype=dtype)
    W = np.asarray(W, dtype=dtype)
    return np.einsum("bsk,bkj->bsj", x, W[np.asarray(idx)])


def write_tensor_part_ref(X, Y, ids):
    """Z = X; Z[ids[a]] = Y[a]  (`tvm/custom/write_tensor_part.py:3-20`)."""
    Z = np.array(X, copy=True)
    Z[np.asarray(ids)] = np.asarray(Y)
    return Z


def mixed_delta_ref(h, types, dtype=np.float32):
    """Mixed-adapter-type delta of `compile_tvm.py:135-155`: for each adapter type, gather the rows
    `sids`, apply that type's LoRA with `wids`, scatter into a zero tensor; returns the summed delta.
    `types` is a list of dicts(A [n,r,K], B [n,N,r], scaling, sids, wids)."""
    h = np.asarray(h, dtype=dtype)
    N = types[0]["B"].shape[1]
    delta = np.zeros((h.shape[0], N), dtype=dtype)
    for t in types:
        sids = np.asarray(t["sids"])
        h_lcl = h[sids]
        d = gather_mm_ref(np.zeros((len(sids), N), dtype), h_lcl, t["A"], t["B"], t["wids"], t["scaling"], dtype)
        delta = write_tensor_part_ref(delta, d, sids)
    return delta


def combined_tables_ref(A_large, B_large, A_small, B_small):
    """The 'combined' tables of `tvm/lora_only/case_study/two_ranks_with_combine.py:649-653`, in PEFT orientation:
    r_mult = r_large / r_small small-rank adapters share one slot of rank r_large, adapter i * r_mult + j of the small
    type taking rank entries j * r_small .. of slot i; the large-rank adapters come first.
    A_* [n, r, K], B_* [n, N, r]  ->  A [n_large + n_small / r_mult, r_large, K], B [.., N, r_large]."""
    A_large, B_large = np.asarray(A_large), np.asarray(B_large)
    A_small, B_small = np.asarray(A_small), np.asarray(B_small)
    r_mult = A_large.shape[1] // A_small.shape[1]
    assert A_large.shape[1] == r_mult * A_small.shape[1] and A_small.shape[0] % r_mult == 0
    groups = A_small.shape[0] // r_mult
    A_sc = np.stack([np.concatenate([A_small[i * r_mult + j] for j in range(r_mult)], axis=0) for i in range(groups)])
    B_sc = np.stack([np.concatenate([B_small[i * r_mult + j] for j in range(r_mult)], axis=1) for i in range(groups)])
    return np.concatenate([A_large, A_sc], 0), np.concatenate([B_large, B_sc], 0)


def lora_combined_ref(x, A, B, xids, wids, scaling, n_rows=None, dtype=np.float32):
    """The 'combined' strategy's two kernels (`two_ranks_with_combine.py:343-398` take_matmul_combined and `:400-468`
    fused_take_matmul_multiply_combined): combined row c uses slot wids[c]; rank entry j of that row belongs to token
    xids[c * R + j]:
        v[c, j]   = sum_k x[xids[c R + j], k] * A[wids[c], j, k]
        out[t, n] = scaling * sum over (c, j) with xids[c R + j] == t of v[c, j] * B[wids[c], n, j]
    The reference indexes the expand's operands `lv` and `lora_B` by wids[c] (`:437-446`), which is row c for the
    only table it builds (wids = arange, `:1014`); this follows the row.  Returns out [n_rows, N] (no base added)."""
    x = np.asarray(x, dtype=dtype)
    A = np.asarray(A, dtype=dtype)
    B = np.asarray(B, dtype=dtype)
    xids = np.asarray(xids).reshape(len(wids), -1)
    R = A.shape[1]
    assert xids.shape[1] == R
    out = np.zeros((x.shape[0] if n_rows is None else n_rows, B.shape[1]), dtype=dtype)
    for c, w in enumerate(np.asarray(wids)):
        v = np.einsum("jk,jk->j", x[xids[c]], A[w])          # [R]: entry j from its own token
        for j in range(R):
            out[xids[c, j]] += v[j] * B[w][:, j]
    return out * dtype(scaling)
