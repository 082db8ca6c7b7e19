"""Adapters on disk: one safetensors file per adapter, named by rank and weight id.

File format of the reference (`init_peft_weights/lora_weights.py:14-25`): `r{rank}_a{wid}.safetensors` holding fp32
tensors `layers.{L}.self_attn.{q,v}_proj.lora_A.weight` [r, K] and `...lora_B.weight` [N, r] (PEFT orientation).
Here any of the seven decoder linears may appear; q/k/v/o live under `self_attn`, gate/up/down under `mlp`.

Loading (`tvm/llama_auto_batcher/compile_tvm.py:296-314`) stacks the adapters of one type along a leading
dimension.  The reference stacks in the order the weight ids were first seen and then indexes the stack with the
raw weight id, which is only right when the ids happen to be 0..n-1 in order; here the loader records which stack
row holds which weight id (`LoraType.row_of`) and the model translates ids before they reach a kernel.
"""
from __future__ import annotations

import os

import torch
from safetensors.torch import load_file, save_file

from .llama import LoraType
from .synth import LINEARS, LlamaShape, linear_dims, normal

_BLOCK = {"q_proj": "self_attn", "k_proj": "self_attn", "v_proj": "self_attn", "o_proj": "self_attn",
          "gate_proj": "mlp", "up_proj": "mlp", "down_proj": "mlp"}


def adapter_path(directory: str, r: int, wid: int) -> str:
    return os.path.join(directory, f"r{r}_a{wid}.safetensors")


def tensor_key(layer: int, proj: str, which: str) -> str:
    """which: 'A' or 'B'."""
    return f"layers.{layer}.{_BLOCK[proj]}.{proj}.lora_{which}.weight"


def write_synthetic_adapters(directory: str, shape: LlamaShape, ranks, n_adapters: int, targets=("q_proj", "v_proj"),
                             seed: int = 0, std: float = 0.01):
    """Random adapters in the reference's file layout (fp32, N(0, std) for both A and B as in
    `init_peft_weights/lora_weights.py:9,16-23`), from the package's seeded generator."""
    os.makedirs(directory, exist_ok=True)
    for r in ranks:
        for wid in range(n_adapters):
            w = {}
            for l in range(shape.num_hidden_layers):
                for proj in targets:
                    N, K = linear_dims(shape, proj)
                    w[tensor_key(l, proj, "A")] = normal(seed, f"file.r{r}.a{wid}.{l}.{proj}.A", (r, K), std, torch.float32)
                    w[tensor_key(l, proj, "B")] = normal(seed, f"file.r{r}.a{wid}.{l}.{proj}.B", (N, r), std, torch.float32)
            save_file(w, adapter_path(directory, r, wid))


def load_lora_type(directory: str, r: int, alpha: float, wids, shape: LlamaShape, device="cuda:0") -> LoraType:
    """Stack the adapters `wids` (weight ids, any order, no duplicates) of rank r into one LoraType.
    Every file must target the same projections with the shapes the model expects."""
    wids = [int(w) for w in wids]
    if len(set(wids)) != len(wids) or not wids:
        raise ValueError(f"weight ids must be distinct and non-empty: {wids}")
    files = []
    for wid in wids:
        path = adapter_path(directory, r, wid)
        if not os.path.isfile(path):
            raise FileNotFoundError(f"adapter file {path} not found")
        files.append(load_file(path))
    keys = sorted(files[0].keys())
    for wid, f in zip(wids, files):
        if sorted(f.keys()) != keys:
            raise ValueError(f"adapter r{r}_a{wid} targets different tensors than r{r}_a{wids[0]}")
    lt = LoraType(r, alpha / r, len(wids))
    lt.row_of = {wid: row for row, wid in enumerate(wids)}
    for l in range(shape.num_hidden_layers):
        for proj in LINEARS:
            ka, kb = tensor_key(l, proj, "A"), tensor_key(l, proj, "B")
            if ka not in files[0]:
                continue
            N, K = linear_dims(shape, proj)
            for wid, f in zip(wids, files):
                if tuple(f[ka].shape) != (r, K) or tuple(f[kb].shape) != (N, r):
                    raise ValueError(f"adapter r{r}_a{wid} layer {l} {proj}: A{tuple(f[ka].shape)} B{tuple(f[kb].shape)}, "
                                     f"expected A{(r, K)} B{(N, r)}")
            A = torch.stack([f[ka] for f in files]).to(device, torch.float16)
            B = torch.stack([f[kb] for f in files]).to(device, torch.float16)
            lt.add(l, proj, A, B)
    if not lt.tables:
        raise ValueError(f"adapter files of rank {r} hold no tensor for {shape.num_hidden_layers} layers")
    return lt


def load_adapters_for(seq_info, model, cache_dir: str):
    """Load every adapter type the registered requests use, in type order (type id = position), from
    `{cache_dir}/lora_adapters/` - the directory layout of `compile_tvm.py:301`."""
    directory = os.path.join(cache_dir, "lora_adapters")
    configs, wids = seq_info.get_adapter_configs(), seq_info.get_wids_per_type()
    if model.lora_types:
        raise RuntimeError("the model already holds adapter types")
    for cfg, w in zip(configs, wids):
        model.add_lora_type(load_lora_type(directory, cfg.r, cfg.alpha, w, model.shape, model.device))
