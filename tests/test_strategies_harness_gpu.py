"""GPU checks of three corners of the path: the shrink half alone against the reference's fused take-matmul, the
case study's 'combined' two-rank strategy against the multi-rank call, and the measure.txt harness of the front end."""
import numpy as np
import pytest
import torch

import oracle
from oracle import max_rel_err
from conftest import load_pkg
from helpers import hip_model, n_pages_for

pytestmark = pytest.mark.gpu
TOL = 2e-3
DEV = "cuda:0"


def _np(t):
    return t.detach().float().cpu().numpy()


@pytest.mark.parametrize("T,K,r,n_ad,frag", [(64, 4096, 16, 32, False), (32, 4096, 16, 16, True), (9, 1536, 64, 3, False),
                                             (130, 11008, 8, 5, False)])
def test_lora_shrink_alone_equals_take_matmul(ops, synth, T, K, r, n_ad, frag):
    """mlora_lora_shrink by itself: its K-slice partials, summed in slice order, are the reference's fused
    take-matmul `out[b, 0, j] = sum_k x[b, 0, k] * W[idx[b], k, j]` (`tvm/custom/fuse_take_matmul.py:85-105`) on the
    transposed tables; tokens without adapter are left alone (their rows of the partials are never written)."""
    print(f"case lora_shrink T={T} K={K} r={r} n_ad={n_ad} frag={frag}", flush=True)
    x = synth.normal(51, f"shr.x{T}", (T, K), 1.0, torch.float16, DEV)
    A = synth.normal(51, f"shr.A{T}", (n_ad, r, K), 0.02, torch.float16, DEV)
    ids = synth.randint(51, f"shr.ids{T}", (T,), n_ad + 1, DEV) - 1            # -1 = no adapter
    ids = ids.to(torch.int32)
    kc = ops.lib().mlora_gather_mm_workspace_bytes(T, K, r) // (4 * T * r)
    part = torch.full((kc, T, r), 777.0, dtype=torch.float32, device=DEV)
    ops.lora_shrink(part, ops.FragActivation.pack(x) if frag else x, A, ids)
    torch.cuda.synchronize()
    got = _np(part)
    idh = ids.cpu().numpy()
    has = idh >= 0
    ref = oracle.take_matmul_ref(_np(x)[has][:, None, :], _np(A).transpose(0, 2, 1), idh[has], np.float64)[:, 0]
    assert max_rel_err(got[:, has].sum(0), ref) <= TOL
    assert np.all(got[:, ~has] == 777.0)


@pytest.mark.parametrize("frag", [False, True])
def test_combined_strategy_tables_equal_the_multi_rank_call(ops, synth, frag):
    """The case study's 'combined' strategy (`tvm/lora_only/case_study/two_ranks_with_combine.py:343-511`): r_mult
    small-rank adapters packed into one slot of the large rank, a token index per (combined row, rank entry).  The
    tables and index arrays are built as the reference builds them (`:649-653`, `:1013-1014`: large-rank requests
    first, every request with its own adapter) and evaluated by the oracle's restatement of the two combined kernels;
    the multi-rank call, which reads every table at its own rank and needs no combined tables, gives the same rows
    (the reference's own assert, `:1090`: combined == sequential)."""
    K, N, r_large, r_small = 2048, 1024, 32, 8
    bl, bs = 5, 12                                            # requests of the large / small rank
    r_mult = r_large // r_small
    A_l = synth.normal(61, "cmb.Al", (bl, r_large, K), 0.05, torch.float16, DEV)
    B_l = synth.normal(61, "cmb.Bl", (bl, N, r_large), 0.05, torch.float16, DEV)
    A_s = synth.normal(61, "cmb.As", (bs, r_small, K), 0.05, torch.float16, DEV)
    B_s = synth.normal(61, "cmb.Bs", (bs, N, r_small), 0.05, torch.float16, DEV)
    T = bl + bs
    x = synth.normal(61, "cmb.x", (T, K), 1.0, torch.float16, DEV)
    A_c, B_c = oracle.combined_tables_ref(_np(A_l), _np(B_l), _np(A_s), _np(B_s))
    xids = [i for i in range(bl) for _ in range(r_large)] + [i for i in range(bl, T) for _ in range(r_small)]
    wids = np.arange(bl + bs // r_mult)
    want = oracle.lora_combined_ref(_np(x), A_c, B_c, xids, wids, 2.0, dtype=np.float64)
    tok_bucket = torch.tensor([0] * bl + [1] * bs, dtype=torch.int32, device=DEV)
    tok_adapter = torch.tensor(list(range(bl)) + list(range(bs)), dtype=torch.int32, device=DEV)
    y = torch.zeros((T, N), dtype=torch.float32, device=DEV)
    ops.gather_mm_multi(y, ops.FragActivation.pack(x) if frag else x, [(A_l, B_l, 2.0), (A_s, B_s, 2.0)], tok_bucket, tok_adapter)
    torch.cuda.synchronize()
    assert max_rel_err(_np(y), want) <= TOL
    # the combined tables themselves, used as rank-32 adapters on the large-rank requests only, agree as well: the
    # first bl slots are the large adapters unchanged
    y2 = torch.zeros((T, N), dtype=torch.float32, device=DEV)
    only_large = torch.tensor(list(range(bl)) + [-1] * bs, dtype=torch.int32, device=DEV)
    ops.gather_mm(y2, x, torch.from_numpy(A_c).to(DEV, torch.float16), torch.from_numpy(B_c).to(DEV, torch.float16), only_large, 2.0)
    assert torch.equal(y2[:bl], y[:bl]) and not y2[bl:].any()


def test_measure_file_one_line_per_prefill_and_decode_step(tmp_path):
    """`set_measurement_vars(trials, dest)` (`tvm/llama_auto_batcher/llama_auto_batcher.py:122-136`): warm-up passes
    write nothing; every measured pass writes one millisecond value per line, one line per prefill call and one per
    decode step (`llama_exec_graph.py:48-50,70-74,86-90,116-132`), each pass from an empty cache; the tokens are those
    of a run without measuring."""
    synth, ab, lora, xg = (load_pkg(m) for m in ("synth", "auto_batcher", "lora", "llama_exec_graph"))
    wl = synth.config1()
    model = hip_model(wl)
    prompts = synth.prompts(wl)[:3, :40]
    max_gen_len, trials, warmup = 5, 2, 2
    n_pages = n_pages_for(wl, max_gen_len)
    perm = synth.permutation(7, "measure.pages", n_pages)

    def run(dest):
        b = ab.LlamaAutoBatcherClass()
        b.set_model(model)
        b.set_exec_config(xg.LlamaExecConfig(max_prompt_len=40, max_gen_len=max_gen_len, page_size=wl.page_size))
        b.set_free_pages(perm)
        if dest is not None:
            b.set_measurement_vars(trials, dest, warmup_trials=warmup)
        outs = []
        for i in range(3):
            v = b.create_var(np.asarray(prompts[i], dtype=np.int32))
            b.set_adapter(lora.LoraConfig(r=wl.lora.r, alpha=wl.lora.scaling * wl.lora.r), wid=i)
            outs.append(b.generate(v, max_gen_len=max_gen_len - (i == 2)))      # the last request stops one token early
            b.print(outs[-1])
        b.compile()
        b.execute()
        return [list(map(int, o.var)) for o in outs], b

    plain, _ = run(None)
    dest = str(tmp_path / "measure.txt")
    timed, b = run(dest)
    assert timed == plain and [len(t) for t in timed] == [5, 5, 4]
    b.graph.measure_file.flush()
    lines = open(dest).read().split("\n")
    assert lines[-1] == ""                                     # every value ends its line
    vals = [float(v) for v in lines[:-1]]
    per_pass = 3 + (max_gen_len - 1)                           # three prefill calls + four decode steps
    assert len(vals) == trials * per_pass and all(0.0 < v < 1e4 for v in vals)
    assert len(b.graph.step_ms) == trials * per_pass           # the warm-up passes were not recorded
