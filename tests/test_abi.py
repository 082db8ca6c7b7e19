"""The C-ABI library builds, loads and exports exactly what include/mlora.h declares (no compute calls)."""
import ctypes
import os
import re

import pytest

from conftest import ROOT, load_pkg


def _declared():
    text = open(os.path.join(ROOT, "include", "mlora.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlora_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib_mod = load_pkg("_lib")
    if not os.path.exists(lib_mod.LIB_PATH):
        load_pkg("build").build()
    lib = ctypes.CDLL(lib_mod.LIB_PATH)
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in mlora.h but not exported"
    assert sorted(lib_mod.SIGNATURES) == names, "ctypes signature table and header disagree"
    assert lib.mlora_version() == 1


def test_argument_validation_without_gpu():
    """Shape checks happen on the host before any launch, so they can be exercised without a GPU."""
    lib = load_pkg("_lib").lib()
    assert lib.mlora_gather_mm(1, 0, 64, 1, 0, 1, 1, 1, 1.0, 4, 64, 64, 12, 2, 1, 1 << 20, None) == -2
    assert b"rank" in lib.mlora_last_error()
    assert lib.mlora_gather_mm_workspace_bytes(64, 4096, 16) == 8 * 64 * 16 * 4
    assert lib.mlora_gather_mm_workspace_bytes(32, 11008, 64) == 8 * 32 * 64 * 4
    assert lib.mlora_packed_weight_elems(40, 64) == 48 * 64
    assert lib.mlora_gemv(1, 0, 0, 1, 64, 1, 65, 64, 64, None) == -2
    assert lib.mlora_gemv(1, 0, 1, 1, 64, 1, 4, 64, 64, None) == -2          # accumulate into fp16
    assert lib.mlora_gemv(1, 1, 0, 1, 60, 1, 4, 64, 64, None) == -1          # ldx < K
    assert lib.mlora_rmsnorm(1, 0, 1, 0, 1, 1e-5, 4, 12, None) == -2
    assert lib.mlora_rmsnorm(1, 1, 1, 0, 1, 1e-5, 65, 72, None) == -2        # fragment order needs H % 32 == 0
    assert lib.mlora_frag_activation_elems(17, 64) == 32 * 64 and lib.mlora_frag_activation_elems(33, 64) == 64 * 64
    assert lib.mlora_frag_activation_elems(65, 64) == 80 * 64 and lib.mlora_frag_activation_elems(4096, 64) == 4096 * 64
    assert lib.mlora_linear_frag(1, 0, 0, 16, 16, 100, 48, 64, None) == -2   # fragment order: K % 32
    assert lib.mlora_linear_frag(1, 0, 0, 24, 16, 100, 64, 64, None) == -1   # xf not 16-byte aligned
    assert lib.mlora_gemv_ksplit(256, 4096, 4096) == 4 and lib.mlora_gemv_ksplit(256, 4096, 12288) == 2 and lib.mlora_gemv_ksplit(256, 4096, 32000) == 1
    assert lib.mlora_gemv_frag_acc_ksplit(16, None, None, 2, 16, 16, 100, 64, 64, 0, None, None, 0, None, 0, 0, None) == -1   # slices without partials
    assert lib.mlora_gemm_frag_preferred(4096, 4096, 4096) == 1 and lib.mlora_gemm_frag_preferred(4096, 4096, 4095 - 255) == 0
    assert lib.mlora_gemm_frag_preferred(64, 4096, 1 << 20) == 0 and lib.mlora_gemm_frag_preferred(4096, 4128, 4096) == 0
    assert lib.mlora_paged_attn_prefill(1, 7, 1, 1, 1, 1, 4, 1, 1, 5, 8, 8, 128, 4, 2, None) == -1    # unknown output layout
    assert lib.mlora_paged_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 2, 8, 8, 96, 4, 2, None) == -2   # head_dim 96
    assert lib.mlora_paged_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 2, 8, 3, 128, 4, 2, None) == -1  # Hq % Hkv


def test_argument_validation_of_fused_and_batched_entry_points():
    """Every error below is detected on the host before a launch (pointers are dummies)."""
    import ctypes as C
    lm = load_pkg("_lib")
    lib = lm.lib()
    # multi-rank: bad rank in the second bucket is reported before the first bucket runs; workspace sized by the largest rank
    bk = (lm.LoraBucket * 2)()
    bk[0].A, bk[0].B, bk[0].r, bk[0].n_ad, bk[0].scaling = 1, 1, 16, 4, 0.5
    bk[1].A, bk[1].B, bk[1].r, bk[1].n_ad, bk[1].scaling = 1, 1, 12, 4, 0.5
    args = (1, 0, 64, 1, 0, C.cast(bk, C.c_void_p), 2, 1, 1, 8, 64, 64, 1, 1 << 20, None)
    assert lib.mlora_gather_mm_multi(*args) == -2 and b"rank" in lib.mlora_last_error()
    bk[1].r = 64
    small = lib.mlora_gather_mm_workspace_bytes(8, 64, 16)
    assert lib.mlora_gather_mm_multi(1, 0, 64, 1, 0, C.cast(bk, C.c_void_p), 2, 1, 1, 8, 64, 64, 1, small, None) == -3
    bk[1].A = None
    assert lib.mlora_gather_mm_multi(1, 0, 64, 1, 0, C.cast(bk, C.c_void_p), 2, 1, 1, 8, 64, 64, 1, 1 << 20, None) == -1   # one null table
    assert lib.mlora_gather_mm_multi(1, 0, 64, 1, 0, None, 2, 1, 1, 8, 64, 64, 1, 1 << 20, None) == -1
    # several projections in one call: column ranges and every bucket are checked before anything is launched
    bk4 = (lm.LoraBucket * 4)()
    for e in bk4:
        e.A, e.B, e.r, e.n_ad, e.scaling = 1, 1, 16, 4, 0.5
    co, nc = (C.c_int32 * 2)(0, 64), (C.c_int32 * 2)(64, 64)
    mp = lambda ldy=128, r3=16, co=co: lib.mlora_gather_mm_multi_proj(1, 0, ldy, 1, 0, C.cast(bk4, C.c_void_p), 2, 2, C.cast(co, C.c_void_p),
                                                                      C.cast(nc, C.c_void_p), 1, 1, 8, 64, 1, 1 << 20, None)
    assert mp(ldy=120) == -1 and b"columns" in lib.mlora_last_error()               # second projection ends past the row
    assert mp(co=(C.c_int32 * 2)(0, 60)) == -1                                         # offset not a multiple of 8
    bk4[3].r = 12
    assert mp() == -2 and b"rank" in lib.mlora_last_error()
    bk4[3].r = 16
    assert lib.mlora_gather_mm_multi_proj(1, 0, 128, 1, 0, C.cast(bk4, C.c_void_p), 2, 9, C.cast(co, C.c_void_p), C.cast(nc, C.c_void_p),
                                          1, 1, 8, 64, 1, 1 << 20, None) == -1         # more than 8 projections
    # batched gather-matmul: decode shapes only
    assert lib.mlora_gather_mm_batch(1, 4, 0, 64, 0, 1, 1.0, 65, 64, 64, 16, 2, None, 0, None) == -2
    assert lib.mlora_gather_mm_batch(None, 4, 0, 64, 0, 1, 1.0, 8, 64, 64, 16, 2, None, 0, None) == -1
    assert lib.mlora_gather_mm_batch(1, 0, 0, 64, 0, 1, 1.0, 8, 64, 64, 16, 2, None, 0, None) == 0           # nothing to do
    assert lib.mlora_gather_mm_batch(1, 16, 0, 64, 0, 1, 1.0, 8, 64, 64, 16, 2, 1, 64, None) == -3          # workspace too small for 16 sets
    # the entry point without workspace: shapes beyond its built-in scratch are refused before anything else happens
    assert lib.mlora_gather_mm_static_max_bytes() == 8 << 20
    assert lib.mlora_gather_mm_static(1, 0, 64, 1, 0, 1, 1, 1, 1.0, 4097, 4096, 64, 64, 2, None) == -3 and b"scratch" in lib.mlora_last_error()
    assert lib.mlora_gather_mm_static(1, 0, 64, 1, 0, 1, 1, 1, 1.0, 8, 64, 64, 12, 2, None) == -2
    assert lib.mlora_gather_mm_static(1, 0, 64, 1, 0, 1, 1, 1, 1.0, 0, 64, 64, 16, 2, None) == 0
    # fused decode attention
    ra = lambda Hq, Hkv, D, B, lay: lib.mlora_rope_attn_decode(1, lay, 1, 1, 1, 1, 4, 1, 1, 1, 1, 1, 64, B, Hq, Hkv, D, 4, 2,
                                                               None, 0, None, None, 0.0, 0, 0, 0, None)
    assert ra(8, 8, 96, 2, 0) == -2                    # head_dim
    assert ra(34, 2, 128, 2, 0) == -2                  # 17 query heads per kv head
    assert ra(8, 8, 128, 65, 7) == -1                  # unknown output layout
    assert ra(8, 8, 128, 0, 0) == 0
    assert lib.mlora_rope_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 1, 1, 1, 64, 2, 8, 8, 128, 4, 2,
                                      1, 1, None, None, 0.5, 64, 16, 2, None) == -1     # LoRA without B / ids
    # dense shrink results come in at most four K-range blocks: a larger count would overrun the kernel's LDS array
    b3 = C.cast((C.c_void_p * 3)(1, 1, 1), C.c_void_p)       # host array of three (dummy) B table pointers
    assert lib.mlora_rope_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 1, 1, 1, 64, 2, 8, 8, 128, 4, 2,
                                      1, 5, b3, 1, 0.5, 64, 16, 2, None) == -2 and b"v_dense" in lib.mlora_last_error()
    assert lib.mlora_rope_attn_decode(1, 0, 1, 1, 1, 1, 4, 1, 1, 1, 1, 1, 64, 2, 8, 8, 128, 4, 2,
                                      1, -1, b3, 1, 0.5, 64, 16, 2, None) == -2
    assert lib.mlora_rope_kv_append_lora(1, 1, 1, 1, 4, 1, 1, 1, 1, 64, 2, 8, 8, 128, 4, 2,
                                         1, 5, b3, 1, 0.5, 64, 16, 2, None) == -2 and b"v_dense" in lib.mlora_last_error()
    # SiLU epilogue GEMV and split GEMV
    assert lib.mlora_gemv_frag_silu(1, 1, 1, 65, 64, 64, None) == -2
    assert lib.mlora_gemv_frag_silu(1, 1, 1, 8, 64, 48, None) == -2
    assert lib.mlora_gemv_frag_silu(None, 1, 1, 8, 64, 64, None) == -1
    # K-split GEMV: slice counts, partials buffer, argument checks
    assert lib.mlora_gemv_ksplit(32, 11008, 4096) == 4 and lib.mlora_gemv_ksplit(32, 4096, 4352) == 3
    assert lib.mlora_gemv_ksplit(33, 11008, 4096) == 4 and lib.mlora_gemv_ksplit(32, 4096, 12288) == 1
    assert lib.mlora_gemv_ksplit(65, 11008, 4096) == 4 and lib.mlora_gemv_ksplit(64, 4096, 4352) == 3
    assert lib.mlora_gemv_ksplit_bytes(32, 4096, 4) == 3 * 32 * 4096 * 4 and lib.mlora_gemv_ksplit_bytes(32, 4096, 1) == 0
    # shrink units riding in the launch weigh a constant number of rows in that rule (the slice count must not follow the batch)
    assert lib.mlora_gemv_shrink_rows(4096, 1, 16) == lib.mlora_gemv_shrink_rows(11008, 1, 200) == 256 and lib.mlora_gemv_shrink_rows(4096, 0, 16) == 0
    assert lib.mlora_gemv_ksplit(32, 4096, 4096 + lib.mlora_gemv_shrink_rows(4096, 1, 16)) == 3
    # K-range blocks of the appended rows in the per-unit split GEMV: 1 where the form does not apply (and without a device)
    assert lib.mlora_gemv_split_kq(32, 4096, 12288, 768) in (1, 4)
    assert lib.mlora_gemv_split_kq(33, 4096, 12288, 768) == 1 and lib.mlora_gemv_split_kq(32, 4096, 1024, 768) == 1
    assert lib.mlora_gemv_split_kq(32, 4096, 12288, 772) == 1
    assert lib.mlora_gemv_frag_split_kq(1, 1, 3, 1, 1, 32, 4096, 12288, 768, None) == -1 and b"kq" in lib.mlora_last_error()
    assert lib.mlora_gemv_frag_split_kq(1, None, 1, 1, 1, 32, 4096, 12288, 768, None) == -1
    ksg = lambda ks, part, T=32, n_ext=0, y2=None, A=None: lib.mlora_gemv_frag_acc_ksplit(1, y2, part, ks, 1, 1, T, 4096, 4096, n_ext,
                                                                                         None, A, 1 if A else 0, None, 16, 4, None)
    assert ksg(2, None) == -1                        # split without a partials buffer
    assert ksg(5, 1) == -1                           # more than four slices
    assert ksg(2, 1, T=70) == -2                     # beyond 64 tokens: the matrix-core kernel, whose xf must be 16-byte aligned
    assert ksg(1, None, n_ext=64) == -1              # appended rows without y2
    assert ksg(2, 1, T=0) == 0
    nk = lambda ks, part, ld: lib.mlora_rmsnorm_ksplit(1, 0, 1, part, ks, ld, 1, 1e-5, 4, 4096, None, 0, None, None, 0.0, 0, 0, 0, None)
    assert nk(2, None, 4096) == -1 and nk(2, 1, 1024) == -1 and nk(5, 1, 4096) == -1
    assert lib.mlora_rmsnorm_ksplit(1, 0, 1, 1, 2, 4096, 1, 1e-5, 4, 4096, 1, 1, 1, 1, 0.5, 4096, 16, 4, None) == -1   # dense partials need wider ld
    assert lib.mlora_rmsnorm_ksplit(1, 0, 1, 1, 2, 16384, 1, 1e-5, 4, 16384, None, 0, None, None, 0.0, 0, 0, 0, None) == -2   # H > 8192
    # prefill linear that carries the LoRA deltas of adapter-uniform 256-token blocks as extra k-steps
    assert lib.mlora_lora_block_adapters(None, 1, 1, 512, 4, None) == -1
    assert lib.mlora_lora_block_adapters(1, 1, 1, 0, 4, None) == 0 and lib.mlora_lora_block_adapters(1, 1, 1, 512, 0, None) == -1
    p3 = C.cast((C.c_void_p * 3)(16, 16, 16), C.c_void_p)
    ss = lambda r=64, T=4096, K=4096, wsb=1 << 30, n_proj=3: lib.mlora_lora_shrink_split(p3, p3, 16, 1, p3, n_proj, 1, 0.5, T, K, r, 64, 16, wsb, None)
    assert ss(r=16) == -2 and b"rank" in lib.mlora_last_error()      # ranks 32 and 64 only
    assert ss(T=64) == -2 and ss(K=4100) == -2 and ss(n_proj=4) == -1
    assert ss(wsb=1024) == -3 and b"workspace" in lib.mlora_last_error()
    fl = (lm.FusedLora * 2)()
    for i, e in enumerate(fl):
        e.B, e.v_hi, e.v_lo, e.n_begin, e.n_rows = 16, 16, 16, 4096 * i, 4096
    lf = lambda r=64, T=4096, N=8192, n_proj=2, blk=16: lib.mlora_linear_frag_lora(16, 0, 0, 16, 16, T, 4096, N, C.cast(fl, C.c_void_p), n_proj,
                                                                                    blk, r, None)
    assert lf(r=16) == -2 and lf(n_proj=4) == -2 and lf(blk=None) == -2
    assert lf(T=256, N=4096) == -2 and b"persistent" in lib.mlora_last_error()      # too few 256 x 256 blocks for that kernel
    fl[1].n_begin = 4096 + 128
    assert lf() == -2 and b"256-row" in lib.mlora_last_error()
    fl[1].n_begin, fl[1].n_rows = 4096, 8192
    assert lf() == -2                                                              # rows past N
    fl[1].n_rows, fl[1].v_lo = 4096, None
    assert lf() == -1
    # gate/up projection with the SiLU product in the epilogue of the persistent GEMM
    fs = (lm.FusedLora * 2)()
    for i, e in enumerate(fs):
        e.B, e.v_hi, e.v_lo, e.n_begin, e.n_rows = 16, 16, 16, 4096 * i, 4096
    sl = lambda act=16, T=4096, I=4096, n_proj=2, blk=16, r=64: lib.mlora_linear_frag_silu(act, 16, 16, T, 4096, I, C.cast(fs, C.c_void_p), n_proj,
                                                                                            blk, r, None)
    assert sl(act=None) == -1 and sl(I=4100) == -2 and sl(n_proj=3) == -2 and sl(r=16) == -2 and sl(blk=None) == -2
    assert sl(T=256, I=2048) == -2 and b"persistent" in lib.mlora_last_error()
    fs[1].n_begin = 2048
    assert sl() == -2 and b"gate rows" in lib.mlora_last_error()                   # neither rows 0..I nor rows I..2I
    fs[1].n_begin = 0
    assert sl() == -1 and b"same rows" in lib.mlora_last_error()
    fs[1].n_begin, fs[1].B = 4096, None
    assert sl() == -1
    # decode step: a plan without layers / with a token count beyond the decode tile
    plan = lm.DecodePlan()
    assert lib.mlora_decode_step(C.byref(plan), None) < 0
    assert lib.mlora_decode_step(None, None) == -1


def test_ops_refuse_cpu_tensors():
    import torch
    ops = load_pkg("ops")
    x = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(ValueError):
        ops.rmsnorm(x, torch.ones(64, dtype=torch.float16), 1e-5)
    with pytest.raises(ValueError):
        ops.linear(x, torch.zeros(8, 64, dtype=torch.float16))
