"""LoRA adapter description and the adapter-indexed linear layer.

`LoraConfig` is the reference's dataclass (`tvm/llama_auto_batcher/lora.py:5-8`); `scaling = alpha / r`
(`lora.py:13`); `Lora` its adapter definition with the four protocol methods (`lora.py:10-24`).  `GatherMMLinear` is the drop-in for the PEFT custom module
`GatherBMMLinear` (`huggingface/custom_peft/lora_gatherbmm_linear_layer.py:5-54`): same forward contract
(`forward(x, adapter_names=[...])`, one adapter per request), but the per-request stack of A / B and the
two bmm launches are replaced by one gather-matmul call that indexes the stacked adapter table inside
the kernel.
"""
from __future__ import annotations

import dataclasses

import torch

from . import ops


@dataclasses.dataclass(frozen=True)
class LoraConfig:
    r: int
    alpha: float

    @property
    def scaling(self) -> float:
        return self.alpha / self.r


class Lora:
    """The reference's adapter definition (`tvm/llama_auto_batcher/lora.py:10-24`) on this package's operators: the
    four protocol methods its compiler checks for (`compile_tvm.py:29-93`) with the same names, argument order and
    meaning.  Parameters come in the reference's orientation, `lora_A [in_features, r]` and `lora_B [r, out_features]`
    (the transposes of PEFT's `lora_A.weight` / `lora_B.weight`).  For ONE adapter
    `post_computation(weight_application(x, lora_A, lora_B))` is the delta that the model adds to the base linear's
    output; the serving path computes the same per token from the stacked tables of all adapters
    (`ops.gather_mm`, see `stack`)."""

    def __init__(self, in_features: int, out_features: int, config: LoraConfig):
        self.in_features, self.out_features, self.config = in_features, out_features, config
        self.scaling = config.alpha / config.r

    def define_parameters(self, in_features: int, out_features: int, config: LoraConfig) -> tuple:
        """Shapes and dtype of the adapter's parameters, in the order `weight_application` takes them."""
        return ((in_features, config.r), "float16"), ((config.r, out_features), "float16")

    def weight_application(self, x: torch.Tensor, lora_A: torch.Tensor, lora_B: torch.Tensor) -> torch.Tensor:
        """(x . lora_A) . lora_B on the base-linear kernels: x [T, in] fp16 -> [T, out] fp16 (fp32 accumulation)."""
        r = lora_A.shape[1]
        rp = -(-r // 32) * 32                 # the base-linear kernels take K in multiples of 32: exact zeros up to there
        At = torch.zeros((rp, lora_A.shape[0]), dtype=torch.float16, device=x.device)
        At[:r] = lora_A.t()
        Bt = torch.zeros((lora_B.shape[1], rp), dtype=torch.float16, device=x.device)
        Bt[:, :r] = lora_B.t()
        return ops.linear(ops.linear(x, At), Bt)

    def post_computation(self, y: torch.Tensor) -> torch.Tensor:
        return y * self.scaling

    @staticmethod
    def stack(params):
        """[(lora_A [in, r], lora_B [r, out]), ...] of equal rank -> the stacked tables of the gather-matmul,
        A [n_ad, r, in] and B [n_ad, out, r]."""
        A = torch.stack([a.t() for a, _ in params]).contiguous()
        B = torch.stack([b.t() for _, b in params]).contiguous()
        return A, B


class GatherMMLinear:
    """Base linear + per-request LoRA delta.

    weight [N, K] fp16 (bias-free).  Adapters are registered by name and kept stacked:
    lora_A [n_ad, r, K], lora_B [n_ad, N, r] (PEFT's `lora_A[name].weight`, `lora_B[name].weight`).
    The branches of the reference forward (`lora_gatherbmm_linear_layer.py:6-54`) in its order: adapters disabled ->
    base only (`:10-13`); `adapter_names` given -> base + the gathered per-request delta (`:14-20`); merged -> base
    only, the active adapters live in the weight (`:21-22`); otherwise every active adapter is applied to every row
    (`:23-52`; DoRA, which the reference inherits from PEFT there, is not offered).
    """

    def __init__(self, weight: torch.Tensor, pack: bool = True):
        self.out_features, self.in_features = weight.shape
        self._pack = pack
        self.weight = ops.PackedWeight(weight) if pack else weight
        self.names = []
        self.scaling = {}
        self.lora_A = None
        self.lora_B = None
        self.disable_adapters = False
        self.active_adapters = []
        self.merged_adapters = []

    @property
    def merged(self) -> bool:
        return bool(self.merged_adapters)

    def add_adapter(self, name: str, A: torch.Tensor, B: torch.Tensor, scaling: float):
        """A [r, K], B [N, r] - the PEFT parameter shapes."""
        if name in self.names:
            raise ValueError(f"adapter {name} already present")
        if self.lora_A is not None and A.shape[0] != self.lora_A.shape[1]:
            raise ValueError("all adapters of one layer must share the rank; use one layer per adapter type")
        A = A.to(torch.float16)[None]
        B = B.to(torch.float16)[None]
        self.lora_A = A.contiguous() if self.lora_A is None else torch.cat([self.lora_A, A])
        self.lora_B = B.contiguous() if self.lora_B is None else torch.cat([self.lora_B, B])
        self.names.append(name)
        self.scaling[name] = float(scaling)

    def set_adapter(self, names):
        """The adapters applied to every row when a call names none (PEFT's active adapters)."""
        names = [names] if isinstance(names, str) else list(names)
        for n in names:
            if n not in self.names:
                raise ValueError(f"unknown adapter {n}")
        self.active_adapters = names

    def _rowmajor(self) -> torch.Tensor:
        return self.weight.unpack() if isinstance(self.weight, ops.PackedWeight) else self.weight

    def _add_to_weight(self, names, sign: float):
        W = self._rowmajor().float()
        for n in names:
            i = self.names.index(n)
            W += sign * self.scaling[n] * (self.lora_B[i].float() @ self.lora_A[i].float())
        W = W.to(torch.float16)
        self.weight = ops.PackedWeight(W) if self._pack else W

    def merge(self, names=None):
        """Fold adapters (default: the active ones) into the base weight: W += scaling * B . A, rounded to fp16."""
        names = self.active_adapters if names is None else ([names] if isinstance(names, str) else list(names))
        names = [n for n in names if n not in self.merged_adapters]
        self._add_to_weight(names, 1.0)
        self.merged_adapters += names

    def unmerge(self):
        """Subtract the merged adapters again (exact up to the fp16 rounding of the merged weight)."""
        self._add_to_weight(self.merged_adapters, -1.0)
        self.merged_adapters = []

    def _delta(self, y, x2, ids_per_row, names):
        """One gather-matmul call per distinct scaling among `names` (the reference folds scaling[name] into B per
        request; the kernel takes one scaling per call, so rows of other scalings are masked)."""
        by_scale = {}
        for n in names:
            by_scale.setdefault(self.scaling[n], set()).add(self.names.index(n))
        for sc, rows in by_scale.items():
            ids = ids_per_row if len(by_scale) == 1 else \
                torch.where(torch.isin(ids_per_row, torch.tensor(sorted(rows), dtype=torch.int32, device=ids_per_row.device)),
                            ids_per_row, torch.full_like(ids_per_row, -1))
            ops.gather_mm(y, x2, self.lora_A, self.lora_B, ids, sc)

    def forward(self, x: torch.Tensor, adapter_names=None) -> torch.Tensor:
        """x [B, S, K] or [B, K]; adapter_names: one name per request (len == x.shape[0]; None or an unknown name =
        no adapter for that request) or None."""
        shp = x.shape
        x2 = x.reshape(-1, shp[-1]).contiguous()
        if self.disable_adapters and self.merged:
            self.unmerge()                              # `lora_gatherbmm_linear_layer.py:10-13`: adapters off = base weight only
        y = ops.linear(x2, self.weight)
        if self.disable_adapters or self.lora_A is None:
            return y.view(*shp[:-1], self.out_features)
        if adapter_names is not None:
            if len(adapter_names) != shp[0]:
                raise ValueError("Length of `adapter_names` should be the same as the number of inputs")
            per_req = [self.names.index(n) if n is not None and n in self.names else -1 for n in adapter_names]
            rows_per_req = x2.shape[0] // shp[0]
            ids = torch.tensor(per_req, dtype=torch.int32).repeat_interleave(rows_per_req).to(x.device)
            used = sorted({n for n in adapter_names if n in self.scaling})
            if used:
                self._delta(y, x2, ids, used)
        elif not self.merged:
            for n in self.active_adapters:             # every active adapter on every row, one after the other
                ids = torch.full((x2.shape[0],), self.names.index(n), dtype=torch.int32, device=x.device)
                ops.gather_mm(y, x2, self.lora_A, self.lora_B, ids, self.scaling[n])
        return y.view(*shp[:-1], self.out_features)

    __call__ = forward


# ---------------------------------------------------------------------------------------------------------------
# Multi-rank table transforms of the reference's case study (`tvm/lora_only/case_study/multiple_ranks.py`): the
# same delta can be computed from tables padded to the largest rank (`:165-178`, PaddedLora `:66-95`) or split into
# chunks of the smallest rank whose partial deltas are summed (`:180-194`, SplittedLora `:98-151`).  The kernels do
# not need either (mlora_gather_mm_multi reads every table at its own rank); these are kept for the equivalence
# checks and for callers that hold padded or splitted tables already.
# ---------------------------------------------------------------------------------------------------------------
def pad_rank(A: torch.Tensor, B: torch.Tensor, r_to: int):
    """A [n, r, K], B [n, N, r] -> zero-padded to rank r_to.  The padded rows contribute exact zeros."""
    n, r, K = A.shape
    if r_to < r:
        raise ValueError(f"cannot pad rank {r} down to {r_to}")
    Ap = torch.zeros((n, r_to, K), dtype=A.dtype, device=A.device)
    Bp = torch.zeros((n, B.shape[1], r_to), dtype=B.dtype, device=B.device)
    Ap[:, :r] = A
    Bp[:, :, :r] = B
    return Ap, Bp


def split_rank(A: torch.Tensor, B: torch.Tensor, r_chunk: int):
    """A [n, r, K], B [n, N, r] -> [n * r/r_chunk, r_chunk, K], [n * r/r_chunk, N, r_chunk]; adapter i becomes rows
    i*m .. i*m+m-1 (m = r / r_chunk), and its delta is the sum of the m chunk deltas."""
    n, r, K = A.shape
    if r % r_chunk:
        raise ValueError(f"rank {r} is not a multiple of {r_chunk}")
    m = r // r_chunk
    As = A.reshape(n, m, r_chunk, K).reshape(n * m, r_chunk, K).contiguous()
    Bs = B.reshape(n, B.shape[1], m, r_chunk).permute(0, 2, 1, 3).reshape(n * m, B.shape[1], r_chunk).contiguous()
    return As, Bs
