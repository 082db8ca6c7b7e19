"""LoRA adapter description and the adapter-indexed linear layer.

`LoraConfig` is the reference's dataclass (`tvm/llama_auto_batcher/lora.py:5-8`); `scaling = alpha / r`
(`lora.py:13`).  `GatherMMLinear` is the drop-in for the PEFT custom module
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


class GatherMMLinear:
    """Base linear + per-request LoRA delta.

    weight [N, K] fp16 (bias-free).  Adapters are registered by name and kept stacked:
    lora_A [n_ad, r, K], lora_B [n_ad, N, r] (PEFT's `lora_A[name].weight`, `lora_B[name].weight`).
    """

    def __init__(self, weight: torch.Tensor, pack: bool = True):
        self.out_features, self.in_features = weight.shape
        self.weight = ops.PackedWeight(weight) if pack else weight
        self.names = []
        self.scaling = {}
        self.lora_A = None
        self.lora_B = None
        self.disable_adapters = False

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

    def forward(self, x: torch.Tensor, adapter_names=None) -> torch.Tensor:
        """x [B, S, K] or [B, K]; adapter_names: one name per request (len == x.shape[0]) or None.
        Mirrors the branch structure of the reference forward: adapters disabled / no names -> base only;
        names given -> base + gathered delta."""
        shp = x.shape
        x2 = x.reshape(-1, shp[-1]).contiguous()
        y = ops.linear(x2, self.weight)
        if self.disable_adapters or adapter_names is None or self.lora_A is None:
            return y.view(*shp[:-1], self.out_features)
        if len(adapter_names) != shp[0]:
            raise ValueError("Length of `adapter_names` should be the same as the number of inputs")
        per_req = [self.names.index(n) if n is not None and n in self.names else -1 for n in adapter_names]
        scal = {self.scaling[n] for n in adapter_names if n in self.scaling}
        if len(scal) > 1:
            raise ValueError("adapters of one call must share alpha / r")
        rows_per_req = x2.shape[0] // shp[0]
        ids = torch.tensor(per_req, dtype=torch.int32).repeat_interleave(rows_per_req).to(x.device)
        if scal:
            ops.gather_mm(y, x2, self.lora_A, self.lora_B, ids, scal.pop())
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
