"""The gather-matmul entry point that allocates nothing (`mlora_gather_mm_static`: kernel scratch in a buffer built into
the library) against `mlora_gather_mm` with a caller workspace: same result bits, on calls in a row that share the
built-in buffer, the later ones with smaller inputs."""
import pytest
import torch

from conftest import load_pkg

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

CASES = [
    # T, K, N, r, n_ad, y dtype - in this order, so that each call finds the previous call's contents in the buffer
    (300, 4096, 4096, 64, 6, torch.float16),      # matrix-core shrink / expand pair: v [T, r] per K range in the scratch
    (130, 11008, 4096, 8, 5, torch.float32),      # a smaller input right after
    (70, 1000, 264, 16, 3, torch.float16),        # odd K: the vector shrink / expand pair with K-slice partials
    (32, 4096, 4096, 16, 16, torch.float16),      # decode-sized: one launch, partials in LDS (the scratch is not touched)
]


def test_gather_mm_static_equals_gather_mm_on_consecutive_calls(ops, synth):
    lm = load_pkg("_lib")
    assert lm.lib().mlora_gather_mm_static_max_bytes() == 8 << 20
    inputs = []
    for T, K, N, r, n_ad, ydt in CASES:
        c = synth.gather_mm_case(seed=9, T=T, K=K, N=N, r=r, n_ad=n_ad, device=DEV, tag=f"static.{T}")
        ids = c["ids"].clone()
        ids[::7] = -1                                           # some rows without adapter
        inputs.append((c, ids, ydt))
    torch.cuda.synchronize()
    for rep in range(2):                                        # the whole sequence twice: big after small as well
        for (T, K, N, r, n_ad, _), (c, ids, ydt) in zip(CASES, inputs):
            print(f"case gather_mm_static T={T} K={K} N={N} r={r} n_ad={n_ad} {ydt} rep={rep}", flush=True)
            want = ops.gather_mm(c["y"].to(ydt).clone(), c["x"], c["A"], c["B"], ids, 0.5)
            got = ops.gather_mm_static(c["y"].to(ydt).clone(), c["x"], c["A"], c["B"], ids, 0.5)
            torch.cuda.synchronize()
            assert torch.equal(got, want)
            assert not torch.equal(got, c["y"].to(ydt))


def test_gather_mm_static_rejects_what_the_buffer_cannot_hold(ops, synth):
    lm = load_pkg("_lib")
    T, K, N, r, n_ad = 4097, 4096, 64, 64, 2                    # 8 slices x 4097 x 64 x 4 bytes: just above 8 MiB
    assert lm.lib().mlora_gather_mm_workspace_bytes(T, K, r) > lm.lib().mlora_gather_mm_static_max_bytes()
    x = torch.zeros((T, K), dtype=torch.float16, device=DEV)
    A = torch.zeros((n_ad, r, K), dtype=torch.float16, device=DEV)
    B = torch.zeros((n_ad, N, r), dtype=torch.float16, device=DEV)
    y = torch.ones((T, N), dtype=torch.float16, device=DEV)
    ids = torch.zeros(T, dtype=torch.int32, device=DEV)
    with pytest.raises(lm.MloraError) as e:
        ops.gather_mm_static(y, x, A, B, ids, 1.0)
    assert e.value.code == -3 and "scratch" in str(e.value)
    assert bool((y == 1).all())                                 # nothing was launched
