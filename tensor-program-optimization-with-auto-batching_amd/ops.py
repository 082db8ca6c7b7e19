"""Operator surface over the C ABI: torch tensors supply device memory and the stream, nothing else.

Each function validates dtypes/contiguity on the host, hands raw pointers to libmlora_hip.so and
enqueues on torch's current stream.  None of them has a CPU path.
"""
from __future__ import annotations

import torch

from ._lib import F16, F32, ROWMAJOR, FRAG, STORE, ACCUMULATE, check, lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, dtype=None, name="tensor") -> int:
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.float32:
        return F32
    raise TypeError(f"expected float16 or float32, got {t.dtype}")


class FragActivation:
    """A [T, K] fp16 activation block stored in matrix-core fragment order (MLORA_FRAG)."""

    def __init__(self, T: int, K: int, device, data: torch.Tensor = None):
        self.T, self.K = T, K
        n = lib().mlora_frag_activation_elems(T, K)
        self.data = torch.empty(n, dtype=torch.float16, device=device) if data is None else data
        if self.data.numel() < n:
            raise ValueError("FragActivation: buffer too small")

    @property
    def shape(self):
        return (self.T, self.K)

    @property
    def device(self):
        return self.data.device

    @classmethod
    def pack(cls, x: torch.Tensor, out: "FragActivation" = None):
        """Row-major [T, K] fp16 (unit inner stride) -> fragment order."""
        T, K = x.shape
        out = cls(T, K, x.device) if out is None else out
        ld = x.stride(0) if T > 1 else max(K, x.stride(0))
        check(lib().mlora_pack_activation(out.data.data_ptr(), x.data_ptr(), ld, T, K, _stream()))
        return out

    def unpack(self) -> torch.Tensor:
        """Back to row-major [T, K] (host-side index arithmetic on the device tensor; for tests)."""
        TT = 1 if self.T <= 16 else (2 if self.T <= 32 else (4 if self.T <= 64 else -(-self.T // 16)))
        v = self.data[: TT * 16 * self.K].view(self.K // 32, TT, 4, 16, 8)
        return v.permute(1, 3, 0, 2, 4).reshape(TT * 16, self.K)[: self.T].contiguous()


def _x_arg(x, name="x"):
    """(pointer, layout, T, K) of a row-major tensor or a FragActivation."""
    if isinstance(x, FragActivation):
        return x.data.data_ptr(), FRAG, x.T, x.K
    return _dev(x, torch.float16, name), ROWMAJOR, x.shape[0], x.shape[1]


def gather_mm_workspace(T: int, K: int, r: int, device) -> torch.Tensor:
    n = lib().mlora_gather_mm_workspace_bytes(T, K, r)
    return torch.empty(max(n, 16) // 4, dtype=torch.float32, device=device)


def gather_mm(y, x, A, B, tok_adapter, scaling: float, workspace=None):
    """y[t] += scaling * B[id_t] @ (A[id_t] @ x[t]) in place.  y [T,N] f16|f32 (rows may be strided: a
    column slice of a wider buffer), x [T,K] f16, A [n_ad,r,K] f16, B [n_ad,N,r] f16,
    tok_adapter [T] int32 (-1 = no adapter)."""
    xptr, xlay, T, K = _x_arg(x)
    n_ad, r, K2 = A.shape
    N = B.shape[1]
    if K2 != K or B.shape != (n_ad, N, r) or y.shape != (T, N) or tok_adapter.shape != (T,):
        raise ValueError(f"gather_mm: inconsistent shapes y{tuple(y.shape)} x{tuple(x.shape)} A{tuple(A.shape)} "
                         f"B{tuple(B.shape)} ids{tuple(tok_adapter.shape)}")
    if T == 0:
        return y                                   # an empty batch: nothing to add (an empty tensor has no device pointer)
    if workspace is None:
        workspace = gather_mm_workspace(T, K, r, x.device)
    if not y.is_cuda or y.stride(1) != 1:
        raise ValueError("gather_mm: y must be a GPU tensor with unit inner stride")
    ldy = y.stride(0) if T > 1 else max(N, y.stride(0))
    check(lib().mlora_gather_mm(y.data_ptr(), _dt(y), ldy, xptr, xlay, _dev(A, torch.float16, "A"),
                                _dev(B, torch.float16, "B"), _dev(tok_adapter, torch.int32, "tok_adapter"),
                                float(scaling), T, K, N, r, n_ad, _dev(workspace, torch.float32, "workspace"),
                                workspace.numel() * 4, _stream()))
    return y


def gather_mm_static(y, x, A, B, tok_adapter, scaling: float):
    """gather_mm through the entry point that allocates nothing: the kernels' scratch is a buffer built into the
    library (raises for shapes whose scratch exceeds it).  Calls that overlap on one GPU share that buffer and race."""
    xptr, xlay, T, K = _x_arg(x)
    n_ad, r, K2 = A.shape
    N = B.shape[1]
    if K2 != K or B.shape != (n_ad, N, r) or y.shape != (T, N) or tok_adapter.shape != (T,):
        raise ValueError("gather_mm_static: inconsistent shapes")
    if T == 0:
        return y
    if not y.is_cuda or y.stride(1) != 1:
        raise ValueError("gather_mm_static: y must be a GPU tensor with unit inner stride")
    ldy = y.stride(0) if T > 1 else max(N, y.stride(0))
    check(lib().mlora_gather_mm_static(y.data_ptr(), _dt(y), ldy, xptr, xlay, _dev(A, torch.float16, "A"),
                                       _dev(B, torch.float16, "B"), _dev(tok_adapter, torch.int32, "tok_adapter"),
                                       float(scaling), T, K, N, r, n_ad, _stream()))
    return y


def gather_mm_multi(y, x, buckets, tok_bucket, tok_adapter, workspace=None):
    """Adapters of several ranks in one batch: buckets = [(A [n_ad,r,K], B [n_ad,N,r], scaling) | None, ...]; token t uses
    adapter tok_adapter[t] of bucket tok_bucket[t] (-1 = none).  y is updated in place."""
    import ctypes
    from ._lib import LoraBucket
    xptr, xlay, T, K = _x_arg(x)
    N = y.shape[1]
    if y.shape[0] != T or tok_bucket.shape != (T,) or tok_adapter.shape != (T,):
        raise ValueError("gather_mm_multi: inconsistent shapes")
    arr = (LoraBucket * len(buckets))()
    rmax = 8
    for i, bk in enumerate(buckets):
        if bk is None:                      # the bucket's adapters do not target this projection
            arr[i].A = arr[i].B = None
            continue
        A, B, scaling = bk
        n_ad, r, K2 = A.shape
        if K2 != K or B.shape != (n_ad, N, r):
            raise ValueError(f"gather_mm_multi: bucket {i} has A{tuple(A.shape)} B{tuple(B.shape)} for K={K} N={N}")
        arr[i].A, arr[i].B = _dev(A, torch.float16, "A"), _dev(B, torch.float16, "B")
        arr[i].r, arr[i].n_ad, arr[i].scaling = r, n_ad, float(scaling)
        rmax = max(rmax, r)
    if workspace is None:
        workspace = gather_mm_workspace(T, K, rmax, x.device)
    if not y.is_cuda or y.stride(1) != 1:
        raise ValueError("gather_mm_multi: y must be a GPU tensor with unit inner stride")
    ldy = y.stride(0) if T > 1 else max(N, y.stride(0))
    check(lib().mlora_gather_mm_multi(y.data_ptr(), _dt(y), ldy, xptr, xlay, ctypes.cast(arr, ctypes.c_void_p), len(buckets),
                                      _dev(tok_bucket, torch.int32, "tok_bucket"), _dev(tok_adapter, torch.int32, "tok_adapter"),
                                      T, K, N, _dev(workspace, torch.float32, "workspace"), workspace.numel() * 4, _stream()))
    return y


def gather_mm_multi_proj(y, x, proj_buckets, col_offsets, n_cols, tok_bucket, tok_adapter, workspace=None):
    """gather_mm_multi for several projections that read the same x and own disjoint column ranges of y (q, k, v in the
    fused qkv row; gate and up): proj_buckets[p] is the bucket list of projection p (as for gather_mm_multi, all of the
    same length), whose delta goes to y[:, col_offsets[p] : col_offsets[p] + n_cols[p]].  One launch at decode sizes."""
    import ctypes
    from ._lib import LoraBucket
    xptr, xlay, T, K = _x_arg(x)
    n_proj = len(proj_buckets)
    n_buckets = len(proj_buckets[0])
    if y.shape[0] != T or tok_bucket.shape != (T,) or tok_adapter.shape != (T,) or len(col_offsets) != n_proj or len(n_cols) != n_proj \
            or any(len(b) != n_buckets for b in proj_buckets):
        raise ValueError("gather_mm_multi_proj: inconsistent shapes")
    if T == 0:
        return y
    arr = (LoraBucket * (n_proj * n_buckets))()
    rmax = 8
    for p, buckets in enumerate(proj_buckets):
        for i, bk in enumerate(buckets):
            e = arr[p * n_buckets + i]
            if bk is None:                      # the bucket's adapters do not target this projection
                e.A = e.B = None
                continue
            A, B, scaling = bk
            n_ad, r, K2 = A.shape
            if K2 != K or B.shape != (n_ad, n_cols[p], r):
                raise ValueError(f"gather_mm_multi_proj: projection {p} bucket {i} has A{tuple(A.shape)} B{tuple(B.shape)} "
                                 f"for K={K} N={n_cols[p]}")
            e.A, e.B = _dev(A, torch.float16, "A"), _dev(B, torch.float16, "B")
            e.r, e.n_ad, e.scaling = r, n_ad, float(scaling)
            rmax = max(rmax, r)
    if workspace is None:
        one = gather_mm_workspace(T, K, rmax, x.device).numel()
        workspace = torch.empty(3 * one, dtype=torch.float32, device=x.device)     # a slice per projection sharing a launch
    if not y.is_cuda or y.stride(1) != 1:
        raise ValueError("gather_mm_multi_proj: y must be a GPU tensor with unit inner stride")
    ldy = y.stride(0) if T > 1 else max(y.shape[1], y.stride(0))
    co = (ctypes.c_int32 * n_proj)(*[int(c) for c in col_offsets])
    nc = (ctypes.c_int32 * n_proj)(*[int(c) for c in n_cols])
    check(lib().mlora_gather_mm_multi_proj(y.data_ptr(), _dt(y), ldy, xptr, xlay, ctypes.cast(arr, ctypes.c_void_p), n_buckets, n_proj,
                                           ctypes.cast(co, ctypes.c_void_p), ctypes.cast(nc, ctypes.c_void_p),
                                           _dev(tok_bucket, torch.int32, "tok_bucket"), _dev(tok_adapter, torch.int32, "tok_adapter"),
                                           T, K, _dev(workspace, torch.float32, "workspace"), workspace.numel() * 4, _stream()))
    return y


class GatherMMBatch:
    """Several gather-matmul problems of one shape and one token->adapter table, issued as one launch.
    sets: list of (y, x, A, B) as for gather_mm (x row-major); the tensors are kept alive by this object."""

    def __init__(self, sets, tok_adapter, scaling: float, stream_passes: bool = True):
        """stream_passes: give the call a workspace, which lets it run eight or more sets as a shrink pass and an
        expand pass over all of them (same result bits as the single launch it uses otherwise)."""
        y0, x0, A0, B0 = sets[0]
        self.T, self.K = x0.shape
        self.n_ad, self.r, _ = A0.shape
        self.N = B0.shape[1]
        self.ldy = y0.stride(0) if self.T > 1 else max(self.N, y0.stride(0))
        self.ydt = _dt(y0)
        ptrs = []
        for y, x, A, B in sets:
            if (x.shape != (self.T, self.K) or A.shape != (self.n_ad, self.r, self.K) or B.shape != (self.n_ad, self.N, self.r)
                    or y.shape != (self.T, self.N) or _dt(y) != self.ydt or y.stride(1) != 1
                    or (self.T > 1 and y.stride(0) != self.ldy)):
                raise ValueError("GatherMMBatch: all sets must share shape, dtype and row stride")
            ptrs += [y.data_ptr(), _dev(x, torch.float16, "x"), _dev(A, torch.float16, "A"), _dev(B, torch.float16, "B")]
        self.sets = list(sets)
        self.ids = tok_adapter
        _dev(tok_adapter, torch.int32, "tok_adapter")
        self.scaling = float(scaling)
        self.table = torch.tensor(ptrs, dtype=torch.int64, device=x0.device)
        self.ws = None
        if stream_passes:
            n = len(sets) * lib().mlora_gather_mm_workspace_bytes(self.T, self.K, self.r)
            self.ws = torch.empty(max(n, 16) // 4, dtype=torch.float32, device=x0.device)

    def run(self):
        ws, nb = (self.ws.data_ptr(), self.ws.numel() * 4) if self.ws is not None else (None, 0)
        check(lib().mlora_gather_mm_batch(self.table.data_ptr(), len(self.sets), self.ydt, self.ldy, ROWMAJOR,
                                          self.ids.data_ptr(), self.scaling, self.T, self.K, self.N, self.r, self.n_ad,
                                          ws, nb, _stream()))


def lora_shrink(v_part, x, A, tok_adapter):
    xptr, xlay, T, K = _x_arg(x)
    n_ad, r, _ = A.shape
    check(lib().mlora_lora_shrink(_dev(v_part, torch.float32), xptr, xlay, _dev(A, torch.float16),
                                  _dev(tok_adapter, torch.int32), T, K, r, n_ad, _stream()))
    return v_part


def lora_expand(y, v_part, B, tok_adapter, scaling: float, K: int):
    T, N = y.shape
    n_ad, _, r = B.shape
    check(lib().mlora_lora_expand(_dev(y), _dt(y), N, _dev(v_part, torch.float32), _dev(B, torch.float16),
                                  _dev(tok_adapter, torch.int32), float(scaling), T, K, N, r, n_ad, _stream()))
    return y


def write_tensor_part(X, Y, ids, out=None):
    """Z = X; Z[ids[a]] = Y[a] over the leading dimension."""
    Z = torch.empty_like(X) if out is None else out
    B, A = X.shape[0], Y.shape[0]
    PH = X[0].numel() if B else (Y[0].numel() if A else 8)
    check(lib().mlora_write_tensor_part(_dev(Z, torch.float16), _dev(X, torch.float16), _dev(Y, torch.float16),
                                        _dev(ids, torch.int32), B, A, PH, _stream()))
    return Z


class PackedWeight:
    """A [N, K] fp16 weight stored in matrix-core fragment order (see mlora_pack_weight)."""

    def __init__(self, W: torch.Tensor):
        N, K = W.shape
        self.N, self.K = N, K
        n = lib().mlora_packed_weight_elems(N, K)
        self.data = torch.empty(n, dtype=torch.float16, device=W.device)
        check(lib().mlora_pack_weight(_dev(self.data), _dev(W, torch.float16, "W"), N, K, _stream()))

    @property
    def shape(self):
        return (self.N, self.K)

    def unpack(self) -> torch.Tensor:
        """Back to row-major [N, K] (index arithmetic on the device tensor)."""
        nt = (self.N + 15) // 16
        v = self.data[: nt * 16 * self.K].view(nt, self.K // 32, 4, 16, 8)
        return v.permute(0, 3, 1, 2, 4).reshape(nt * 16, self.K)[: self.N].contiguous()


def linear(x, W, out=None, out_dtype=torch.float16, accumulate=False, kernel="auto"):
    """y (=|+=) x @ W.T.  x [T,K] f16 (row stride may exceed K) or a FragActivation, W [N,K] f16 or a
    PackedWeight.  accumulate=True adds into the fp32 tensor `out`.  kernel: "auto" | "gemv" | "gemm"."""
    if isinstance(x, FragActivation):
        return _linear_frag(x, W, out, out_dtype, accumulate)
    T, K = x.shape
    packed = isinstance(W, PackedWeight)
    N, K2 = W.shape
    if K2 != K:
        raise ValueError(f"linear: x{tuple(x.shape)} vs W{tuple(W.shape)}")
    if T == 0:                                     # an empty batch
        if out is None:
            out = torch.empty((0, N), dtype=torch.float32 if accumulate else out_dtype, device=x.device)
        return out
    if not x.is_cuda or x.dtype != torch.float16 or x.stride(1) != 1:
        raise ValueError("linear: x must be a GPU fp16 tensor with unit inner stride")
    ldx = x.stride(0) if T > 1 else max(K, x.stride(0))
    if out is None:
        if accumulate:
            raise ValueError("linear: accumulate needs out")
        out = torch.empty((T, N), dtype=out_dtype, device=x.device)
    if out.shape != (T, N):
        raise ValueError(f"linear: out{tuple(out.shape)} expected {(T, N)}")
    if packed:
        fn = {"auto": lib().mlora_linear_packed, "gemv": lib().mlora_gemv_packed, "gemm": lib().mlora_gemm_packed}[kernel]
        wptr = W.data.data_ptr()
    else:
        fn = {"auto": lib().mlora_linear, "gemv": lib().mlora_gemv, "gemm": lib().mlora_gemm}[kernel]
        wptr = _dev(W, torch.float16, "W")
    check(fn(_dev(out), _dt(out), ACCUMULATE if accumulate else STORE, x.data_ptr(), ldx, wptr, T, K, N, _stream()))
    return out


def _linear_frag(x, W, out, out_dtype, accumulate):
    if not isinstance(W, PackedWeight):
        raise TypeError("a fragment-ordered activation needs a PackedWeight")
    T, K = x.shape
    N, K2 = W.shape
    if K2 != K:
        raise ValueError(f"linear: x{x.shape} vs W{W.shape}")
    if out is None:
        if accumulate:
            raise ValueError("linear: accumulate needs out")
        out = torch.empty((T, N), dtype=out_dtype, device=x.device)
    if out.shape != (T, N):
        raise ValueError(f"linear: out{tuple(out.shape)} expected {(T, N)}")
    check(lib().mlora_linear_frag(_dev(out), _dt(out), ACCUMULATE if accumulate else STORE, x.data.data_ptr(),
                                  W.data.data_ptr(), T, K, N, _stream()))
    return out


def gemm_frag_preferred(T: int, K: int, N: int) -> bool:
    """Whether a [T, K] x [N, K]^T product of this size runs best with its activations in fragment order."""
    return bool(lib().mlora_gemm_frag_preferred(T, K, N))


def lora_block_adapters(tok_adapter: torch.Tensor, n_ad: int):
    """ids [T] int32 -> (blk_adapter [ceil(T / 256)]: the adapter a 256-token block agrees on or -1,
    tok_rest [T]: -1 where the block's delta can ride in the GEMM, else the token's id)."""
    T = tok_adapter.shape[0]
    blk = torch.empty((max(-(-T // 256), 1),), dtype=torch.int32, device=tok_adapter.device)
    rest = torch.empty((max(T, 1),), dtype=torch.int32, device=tok_adapter.device)[:T]
    check(lib().mlora_lora_block_adapters(blk.data_ptr(), rest.data_ptr(), _dev(tok_adapter, torch.int32), T, n_ad, _stream()))
    return blk, rest


def lora_shrink_split(x, A_list, tok_adapter, scaling: float, workspace, out=None):
    """The matrix-core shrink of up to three projections that read x (A [n_ad, r, K] each), as fp16 hi + lo halves:
    -> [(v_hi [T, r], v_lo [T, r]), ...]."""
    import ctypes as C
    xp, lay, T, K = _x_arg(x)
    n_ad, r, _ = A_list[0].shape
    dev = tok_adapter.device
    if out is None:
        out = [(torch.empty((T, r), dtype=torch.float16, device=dev), torch.empty((T, r), dtype=torch.float16, device=dev)) for _ in A_list]
    n = len(A_list)
    hi = (C.c_void_p * n)(*[o[0].data_ptr() for o in out])
    lo = (C.c_void_p * n)(*[o[1].data_ptr() for o in out])
    Ap = (C.c_void_p * n)(*[_dev(a, torch.float16, "A") for a in A_list])
    check(lib().mlora_lora_shrink_split(C.cast(hi, C.c_void_p), C.cast(lo, C.c_void_p), xp, lay, C.cast(Ap, C.c_void_p), n,
                                        _dev(tok_adapter, torch.int32), float(scaling), T, K, r, n_ad, _dev(workspace, torch.float32),
                                        workspace.numel() * 4, _stream()))
    return out


def linear_frag_lora(x: FragActivation, W: PackedWeight, projs, blk_adapter, r: int, out=None, out_dtype=torch.float16, accumulate=False):
    """`linear(x, W)` with the LoRA deltas of `projs` = [(B [n_ad, rows, r], v_hi, v_lo, first row, rows), ...] carried as
    extra k-steps of the GEMM for the token blocks that `blk_adapter` gives an adapter (shapes of the persistent GEMM)."""
    import ctypes as C
    from ._lib import FusedLora
    T, K = x.shape
    N, K2 = W.shape
    if K2 != K:
        raise ValueError(f"linear_frag_lora: x{x.shape} vs W{W.shape}")
    if out is None:
        if accumulate:
            raise ValueError("linear_frag_lora: accumulate needs out")
        out = torch.empty((T, N), dtype=out_dtype, device=x.device)
    if out.shape != (T, N):
        raise ValueError(f"linear_frag_lora: out{tuple(out.shape)} expected {(T, N)}")
    arr = (FusedLora * len(projs))()
    for e, (B, vh, vl, n0, rows) in zip(arr, projs):
        if B.shape[1] != rows or B.shape[2] != r or vh.shape != (T, r) or vl.shape != (T, r):
            raise ValueError("linear_frag_lora: table or v shape")
        e.B, e.v_hi, e.v_lo, e.n_begin, e.n_rows = _dev(B, torch.float16, "B"), _dev(vh, torch.float16, "v_hi"), _dev(vl, torch.float16, "v_lo"), n0, rows
    check(lib().mlora_linear_frag_lora(_dev(out), _dt(out), ACCUMULATE if accumulate else STORE, x.data.data_ptr(), W.data.data_ptr(),
                                       T, K, N, C.cast(arr, C.c_void_p), len(projs), _dev(blk_adapter, torch.int32), r, _stream()))
    return out


def linear_frag_silu(x: FragActivation, W: PackedWeight, projs=(), blk_adapter=None, r: int = 0, out: FragActivation = None) -> FragActivation:
    """silu(gate) * up of the fused gate/up projection `W` [2I, K] in the epilogue of the persistent GEMM, in fragment
    order.  `projs` as for linear_frag_lora, over the gate rows (first row 0) and / or the up rows (first row I); every
    256-token block must agree on one adapter (lora_block_adapters leaves no rest)."""
    import ctypes as C
    from ._lib import FusedLora
    T, K = x.shape
    N, K2 = W.shape
    I = N // 2
    if K2 != K or N % 2:
        raise ValueError(f"linear_frag_silu: x{x.shape} vs W{W.shape}")
    if out is None:
        out = FragActivation(T, I, x.device)
    if out.shape != (T, I):
        raise ValueError(f"linear_frag_silu: out{tuple(out.shape)} expected {(T, I)}")
    arr = (FusedLora * max(len(projs), 1))()
    for e, (B, vh, vl, n0, rows) in zip(arr, projs):
        if B.shape[1] != rows or B.shape[2] != r or vh.shape != (T, r) or vl.shape != (T, r):
            raise ValueError("linear_frag_silu: table or v shape")
        e.B, e.v_hi, e.v_lo, e.n_begin, e.n_rows = _dev(B, torch.float16, "B"), _dev(vh, torch.float16, "v_hi"), _dev(vl, torch.float16, "v_lo"), n0, rows
    check(lib().mlora_linear_frag_silu(out.data.data_ptr(), x.data.data_ptr(), W.data.data_ptr(), T, K, I,
                                       C.cast(arr, C.c_void_p) if projs else None, len(projs),
                                       _dev(blk_adapter, torch.int32) if projs else None, r, _stream()))
    return out


def interleave_gate_up(gate_up: torch.Tensor) -> PackedWeight:
    """[2I, K] (gate rows, then up rows) -> PackedWeight whose 16-row tiles alternate gate and up."""
    I2, K = gate_up.shape
    I = I2 // 2
    if I % 16:
        raise ValueError("interleave_gate_up: intermediate size must be a multiple of 16")
    return PackedWeight(gate_up.view(2, I // 16, 16, K).permute(1, 0, 2, 3).reshape(I2, K).contiguous())


def gate_up_silu(x: FragActivation, W_il: PackedWeight, out: FragActivation = None) -> FragActivation:
    """silu(x @ Wgate.T) * (x @ Wup.T) in one launch; W_il from interleave_gate_up.  T <= 64."""
    T, K = x.shape
    I2, K2 = W_il.shape
    if K2 != K:
        raise ValueError(f"gate_up_silu: x{x.shape} vs W{W_il.shape}")
    out = FragActivation(T, I2 // 2, x.device) if out is None else out
    check(lib().mlora_gemv_frag_silu(out.data.data_ptr(), x.data.data_ptr(), W_il.data.data_ptr(), T, K, I2 // 2, _stream()))
    return out


def _out_arg(out, T, H, frag, device):
    """Output buffer of a producer: row-major tensor or FragActivation."""
    if frag:
        out = FragActivation(T, H, device) if out is None else out
        return out, out.data.data_ptr(), FRAG
    if out is None:
        out = torch.empty((T, H), dtype=torch.float16, device=device)
    return out, _dev(out, torch.float16, "out"), ROWMAJOR


class KSplitParts:
    """Partial results of a K-split accumulating GEMV (slices 1..ks-1), to be added by the next RMSNorm of the row."""

    def __init__(self, part: torch.Tensor, ks: int, ld: int):
        self.part, self.ks, self.ld = part, ks, ld


def linear_acc_ksplit(x: FragActivation, W: PackedWeight, resid: torch.Tensor, ws: torch.Tensor = None, riding_rows: int = 0):
    """resid [T, N] fp32 += x @ W.T as `linear(..., accumulate=True)`, with K split over several workgroups when the
    library recommends it for this shape and `ws` (fp32 scratch) is large enough: slice 0 lands in resid, the other
    slices in the returned KSplitParts, which the caller hands to the next `rmsnorm(resid, ..., parts=...)`.
    Returns None when the GEMV ran unsplit.  riding_rows: what the native decode step's launch of this linear carries
    besides the weight rows (`mlora_gemv_shrink_rows` for the shrink units of an adapted projection) - the slice count
    follows the same rule here, so that both paths add the same partial sums."""
    T, K = x.shape
    N, K2 = W.shape
    if K2 != K or resid.shape != (T, N) or resid.dtype != torch.float32:
        raise ValueError(f"linear_acc_ksplit: x{x.shape} W{W.shape} resid{tuple(resid.shape)}")
    ks = lib().mlora_gemv_ksplit(T, K, N + riding_rows) if ws is not None else 1
    if ks > 1 and ws.numel() * 4 < lib().mlora_gemv_ksplit_bytes(T, N, ks):
        ks = 1
    check(lib().mlora_gemv_frag_acc_ksplit(_dev(resid, torch.float32), None, _dev(ws, torch.float32) if ks > 1 else None, ks,
                                           x.data.data_ptr(), W.data.data_ptr(), T, K, N, 0, None, None, 0, None, 0, 0, _stream()))
    return KSplitParts(ws, ks, N) if ks > 1 else None


def linear_acc_ksplit_delta(x: FragActivation, W: PackedWeight, resid: torch.Tensor, ws: torch.Tensor, vpart, B, tok_adapter, scaling: float):
    """resid [T, N] fp32 += x @ W.T over K slices, with the LoRA expand scaling * B[id] @ sum_h vpart[h, t] of every token
    done by workgroups riding in the same launch (vpart [n_shares, T, r] fp32: the shrink results as shares that are
    added in order): returns the KSplitParts (slice partials, then the delta rows) that the next
    `rmsnorm(resid, ..., parts=...)` adds - or None when the library does not serve the shape this way (nothing is
    launched then)."""
    T, K = x.shape
    N, K2 = W.shape
    n_ad, N2, r = B.shape
    if K2 != K or N2 != N or vpart.dim() != 3 or tuple(vpart.shape[1:]) != (T, r) or resid.shape != (T, N) or resid.dtype != torch.float32:
        raise ValueError(f"linear_acc_ksplit_delta: x{x.shape} W{W.shape} vpart{tuple(vpart.shape)} B{tuple(B.shape)} resid{tuple(resid.shape)}")
    ks = lib().mlora_gemv_delta_ride_ksplit(T, K, N, r)
    if ks <= 0:
        return None
    if ws.numel() * 4 < lib().mlora_gemv_ksplit_bytes(T, N, ks + 1):
        raise ValueError("linear_acc_ksplit_delta: workspace too small")
    check(lib().mlora_gemv_frag_acc_ksplit_delta(_dev(resid, torch.float32), _dev(ws, torch.float32), ks, x.data.data_ptr(), W.data.data_ptr(),
                                                 T, K, N, _dev(vpart, torch.float32), vpart.shape[0], _dev(B, torch.float16, "B"),
                                                 _dev(tok_adapter, torch.int32), float(scaling), r, n_ad, _stream()))
    return KSplitParts(ws, ks + 1, N)


def rmsnorm(x, w, eps: float, out=None, frag=False, parts: KSplitParts = None):
    """Row-wise RMSNorm of x [T, H] (f16 | f32); frag=True writes a FragActivation.  With `parts` (x fp32) the K-split
    partials are first added to x in place."""
    T, H = x.shape
    if T == 0 and not frag:
        return torch.empty((0, H), dtype=torch.float16, device=x.device) if out is None else out
    out, optr, lay = _out_arg(out, T, H, frag, x.device)
    if parts is not None:
        check(lib().mlora_rmsnorm_ksplit(optr, lay, _dev(x, torch.float32), _dev(parts.part, torch.float32), parts.ks, parts.ld,
                                         _dev(w, torch.float16), float(eps), T, H, None, 0, None, None, 0.0, 0, 0, 0, _stream()))
        return out
    check(lib().mlora_rmsnorm(optr, lay, _dev(x), _dt(x), _dev(w, torch.float16), float(eps), T, H, _stream()))
    return out


def silu_mul(gate_up, out=None, frag=False):
    """gate_up [T, 2I] (gate columns first) -> silu(gate) * up [T, I]."""
    T, I2 = gate_up.shape
    I = I2 // 2
    if T == 0 and not frag:
        return torch.empty((0, I), dtype=torch.float16, device=gate_up.device) if out is None else out
    out, optr, lay = _out_arg(out, T, I, frag, gate_up.device)
    p = _dev(gate_up, torch.float16)
    check(lib().mlora_silu_mul(optr, lay, p, p + I * 2, I2, T, I, _stream()))
    return out


def silu_mul_split(gate, up, out=None):
    T, I = gate.shape
    if out is None:
        out = torch.empty((T, I), dtype=torch.float16, device=gate.device)
    check(lib().mlora_silu_mul(_dev(out, torch.float16), ROWMAJOR, _dev(gate, torch.float16), _dev(up, torch.float16), I, T, I, _stream()))
    return out


def embed(table, ids, out_dtype=torch.float32, out=None):
    T = ids.numel()
    V, H = table.shape
    if out is None:
        out = torch.empty((T, H), dtype=out_dtype, device=table.device)
    if T == 0:
        return out
    check(lib().mlora_embed(_dev(out), _dt(out), _dev(table, torch.float16), _dev(ids, torch.int32), T, H, V, _stream()))
    return out


def argmax(logits, out=None):
    B, V = logits.shape
    if out is None:
        out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if B == 0:
        return out
    check(lib().mlora_argmax(_dev(out, torch.int32), _dev(logits, torch.float32), B, V, _stream()))
    return out


def rope_kv_append(qkv, k_cache, v_cache, block_table, tok_seq, tok_pos, rope_cos, rope_sin, Hq, Hkv, D):
    """qkv [T, Hq+2Hkv, D] f16 (q rotated in place); k_cache [n_pages,Hkv,D/32,4,16,8] (fragment order),
    v_cache [n_pages,Hkv,D,16]."""
    T = qkv.shape[0]
    n_pages = k_cache.shape[0]
    n_seq, max_blocks = block_table.shape
    max_pos = rope_cos.shape[0]
    check(lib().mlora_rope_kv_append(_dev(qkv, torch.float16), _dev(k_cache, torch.float16), _dev(v_cache, torch.float16),
                                     _dev(block_table, torch.int32), max_blocks, _dev(tok_seq, torch.int32),
                                     _dev(tok_pos, torch.int32), _dev(rope_cos, torch.float32), _dev(rope_sin, torch.float32),
                                     max_pos, T, Hq, Hkv, D, n_pages, n_seq, _stream()))


def o_shrink_served(B: int, Hq: int, Hkv: int, D: int, N: int, r: int) -> bool:
    """Whether a decode step of B sequences can take the o projection's adapter delta as head shares off the attention
    launch plus a launch of expand workgroups (the rule the native step applies for more than 64 sequences)."""
    return bool(lib().mlora_rope_attn_oshrink_ok(B, Hq, Hkv, D, r)) and bool(lib().mlora_lora_expand_shares_ok(N, r))


def lora_expand_shares(y, vpart, B, tok_adapter, scaling: float):
    """y [T, N] fp32 += scaling * B[id] @ sum_h vpart[h, t] for the tokens that name an adapter (vpart [shares, T, r] fp32)."""
    T, N = y.shape
    n_ad, N2, r = B.shape
    if N2 != N or y.dtype != torch.float32 or vpart.dim() != 3 or tuple(vpart.shape[1:]) != (T, r):
        raise ValueError(f"lora_expand_shares: y{tuple(y.shape)} vpart{tuple(vpart.shape)} B{tuple(B.shape)}")
    check(lib().mlora_lora_expand_shares(_dev(y, torch.float32), _dev(vpart, torch.float32), vpart.shape[0], _dev(B, torch.float16, "B"),
                                         _dev(tok_adapter, torch.int32), float(scaling), T, N, r, n_ad, _stream()))
    return y


def paged_attn_decode(qkv, k_cache, v_cache, block_table, seq_ids, ctx_len, Hq, Hkv, D, out=None, frag=False, o_shrink=None):
    """o_shrink = (A [n_ad, r, Hq * D] f16, tok_adapter [B] int32): the launch also writes the o projection's shrink as one
    share per query head and the call returns (out, vpart [Hq, B, r] fp32; rows of tokens without adapter are not written)."""
    B = qkv.shape[0]
    n_seq, max_blocks = block_table.shape
    out, optr, lay = _out_arg(out, B, Hq * D, frag, qkv.device)
    if o_shrink is not None:
        A, ids = o_shrink
        n_ad, r, Kq = A.shape
        if Kq != Hq * D or not lib().mlora_rope_attn_oshrink_ok(B, Hq, Hkv, D, r):
            raise ValueError(f"paged_attn_decode: o shrink A{tuple(A.shape)} not served for B={B} Hq={Hq} Hkv={Hkv} D={D}")
        vpart = torch.empty((Hq, B, r), dtype=torch.float32, device=qkv.device)
        check(lib().mlora_paged_attn_decode_oshrink(optr, lay, _dev(qkv, torch.float16), _dev(k_cache, torch.float16),
                                                    _dev(v_cache, torch.float16), _dev(block_table, torch.int32), max_blocks,
                                                    _dev(seq_ids, torch.int32), _dev(ctx_len, torch.int32), B, Hq, Hkv, D,
                                                    k_cache.shape[0], n_seq, _dev(ids, torch.int32), r, n_ad,
                                                    _dev(A, torch.float16, "A"), vpart.data_ptr(), _stream()))
        return out, vpart
    check(lib().mlora_paged_attn_decode(optr, lay, _dev(qkv, torch.float16), _dev(k_cache, torch.float16),
                                        _dev(v_cache, torch.float16), _dev(block_table, torch.int32), max_blocks,
                                        _dev(seq_ids, torch.int32), _dev(ctx_len, torch.int32), B, Hq, Hkv, D,
                                        k_cache.shape[0], n_seq, _stream()))
    return out


def rope_attn_decode(qkv, k_cache, v_cache, block_table, seq_ids, tok_pos, ctx_len, rope_cos, rope_sin, Hq, Hkv, D,
                     out=None, frag=False, o_shrink=None):
    """rope_kv_append + paged_attn_decode of one decode step in one launch (no LoRA on q, k, v); qkv is left unrotated.
    o_shrink = (A [n_ad, r, Hq * D] f16, tok_adapter [B] int32): the launch also writes the o projection's shrink as
    one share per query head and the call returns (out, vpart [Hq, B, r] fp32; rows of tokens without adapter are NaN)."""
    B = qkv.shape[0]
    n_seq, max_blocks = block_table.shape
    out, optr, lay = _out_arg(out, B, Hq * D, frag, qkv.device)
    if o_shrink is not None:
        A, ids = o_shrink
        n_ad, r, Kq = A.shape
        if Kq != Hq * D or not lib().mlora_rope_attn_oshrink_ok(B, Hq, Hkv, D, r):
            raise ValueError(f"rope_attn_decode: o shrink A{tuple(A.shape)} not served for B={B} Hq={Hq} Hkv={Hkv} D={D}")
        vpart = torch.full((Hq, B, r), float("nan"), dtype=torch.float32, device=qkv.device)
        check(lib().mlora_rope_attn_decode_oshrink(optr, lay, _dev(qkv, torch.float16), _dev(k_cache, torch.float16),
                                                   _dev(v_cache, torch.float16), _dev(block_table, torch.int32), max_blocks,
                                                   _dev(seq_ids, torch.int32), _dev(tok_pos, torch.int32), _dev(ctx_len, torch.int32),
                                                   _dev(rope_cos, torch.float32), _dev(rope_sin, torch.float32), rope_cos.shape[0],
                                                   B, Hq, Hkv, D, k_cache.shape[0], n_seq, None, 0, None, _dev(ids, torch.int32), 0.0,
                                                   0, r, n_ad, _dev(A, torch.float16, "A"), vpart.data_ptr(), _stream()))
        return out, vpart
    check(lib().mlora_rope_attn_decode(optr, lay, _dev(qkv, torch.float16), _dev(k_cache, torch.float16),
                                       _dev(v_cache, torch.float16), _dev(block_table, torch.int32), max_blocks,
                                       _dev(seq_ids, torch.int32), _dev(tok_pos, torch.int32), _dev(ctx_len, torch.int32),
                                       _dev(rope_cos, torch.float32), _dev(rope_sin, torch.float32), rope_cos.shape[0],
                                       B, Hq, Hkv, D, k_cache.shape[0], n_seq, None, 0, None, None, 0.0, 0, 0, 0, _stream()))
    return out


def paged_attn_prefill(qkv, k_cache, v_cache, block_table, tok_seq, tok_pos, Hq, Hkv, D, out=None, frag=False):
    T = qkv.shape[0]
    n_seq, max_blocks = block_table.shape
    out, optr, lay = _out_arg(out, T, Hq * D, frag, qkv.device)
    check(lib().mlora_paged_attn_prefill(optr, lay, _dev(qkv, torch.float16), _dev(k_cache, torch.float16),
                                         _dev(v_cache, torch.float16), _dev(block_table, torch.int32), max_blocks,
                                         _dev(tok_seq, torch.int32), _dev(tok_pos, torch.int32), T, Hq, Hkv, D,
                                         k_cache.shape[0], n_seq, _stream()))
    return out
