"""Seeded synthetic inputs that are bit-identical on CPU and on the GPU.

Every tensor is a pure function of (seed, stream name, element index): a 32-bit
integer hash evaluated with int64 arithmetic that never overflows, so the same
torch code gives the same bits on any device.  No floating-point transcendental
is involved: the "normal" draw is a 4-term Irwin-Hall sum of 16-bit uniforms
(mean 0, unit variance, support +-3.46 sigma), scaled by one fp32 multiply and
rounded to the storage dtype.  This is what lets the CPU oracle and the HIP path
consume identical weights without shipping them.

The reference draws its inputs unseeded (`tvm/lora_only/single_rank.py:142-155,182`:
0.01*randn adapters, U(-1e-2,1e-2) activations; `init_peft_weights/lora_weights.py:14-22`);
shapes and distributions here follow the benchmark configurations instead.
"""
from __future__ import annotations

import zlib
from dataclasses import dataclass, field

import numpy as np
import torch

_M32 = 0xFFFFFFFF


def _mul32(x: torch.Tensor, c: int) -> torch.Tensor:
    """(x * c) mod 2^32 for 0 <= x < 2^32 held in int64, without int64 overflow."""
    xl = x & 0xFFFF
    xh = x >> 16
    return (xl * c + (((xh * c) & 0xFFFF) << 16)) & _M32


def _mix32(x: torch.Tensor) -> torch.Tensor:
    x = x ^ (x >> 16)
    x = _mul32(x, 0x7FEB352D)
    x = x ^ (x >> 15)
    x = _mul32(x, 0x846CA68B)
    x = x ^ (x >> 16)
    return x


def _stream_key(seed: int, name: str) -> int:
    return (zlib.crc32(name.encode()) ^ (seed * 0x9E3779B1)) & _M32


def hash32(seed: int, name: str, n: int, device="cpu", offset: int = 0, lane: int = 0) -> torch.Tensor:
    """n hashes (int64 tensor holding 32-bit values) for indices offset..offset+n-1."""
    key = _stream_key(seed, name)
    idx = torch.arange(offset, offset + n, dtype=torch.int64, device=device)
    x = (idx * 4 + lane) & _M32
    x = _mix32(x ^ key)
    x = _mix32((x + 0x9E3779B9 + key) & _M32)
    return x


_CHUNK = 1 << 24


def normal(seed: int, name: str, shape, std: float = 1.0, dtype=torch.float16, device="cpu") -> torch.Tensor:
    """Approximately N(0, std^2): Irwin-Hall(4) on 16-bit uniforms, exact integer sum."""
    n = int(np.prod(shape))
    out = torch.empty(n, dtype=dtype, device=device)
    # std of the sum of four discrete uniforms on 0..65535
    sum_std = float(np.sqrt(4.0 * (65536.0 ** 2 - 1.0) / 12.0))
    scale = np.float32(std / sum_std)
    for off in range(0, n, _CHUNK):
        m = min(_CHUNK, n - off)
        h0 = hash32(seed, name, m, device, off, 0)
        h1 = hash32(seed, name, m, device, off, 1)
        s = (h0 & 0xFFFF) + (h0 >> 16) + (h1 & 0xFFFF) + (h1 >> 16) - 131070
        out[off:off + m] = (s.to(torch.float32) * float(scale)).to(dtype)
    return out.view(*shape)


def uniform(seed: int, name: str, shape, bound: float, dtype=torch.float16, device="cpu") -> torch.Tensor:
    """U(-bound, bound) from a 24-bit field (exactly representable in fp32)."""
    n = int(np.prod(shape))
    out = torch.empty(n, dtype=dtype, device=device)
    for off in range(0, n, _CHUNK):
        m = min(_CHUNK, n - off)
        h = hash32(seed, name, m, device, off, 0) >> 8
        u = h.to(torch.float32) * float(2.0 ** -23) - 1.0
        out[off:off + m] = (u * float(np.float32(bound))).to(dtype)
    return out.view(*shape)


def randint(seed: int, name: str, shape, high: int, device="cpu") -> torch.Tensor:
    """Integers in [0, high) as int32 (multiply-shift, no modulo bias beyond 2^-32)."""
    n = int(np.prod(shape))
    h = hash32(seed, name, n, device, 0, 0)
    return ((h * high) >> 32).to(torch.int32).view(*shape)


def permutation(seed: int, name: str, n: int) -> np.ndarray:
    """A permutation of 0..n-1 (stable argsort of hashes, CPU only)."""
    h = hash32(seed, name, n, "cpu").numpy()
    return np.argsort(h, kind="stable").astype(np.int32)


def zipf_ids(seed: int, name: str, n: int, n_items: int, s: float = 1.1) -> np.ndarray:
    """n draws from p_k ~ (k+1)^-s over n_items items (inverse CDF on a 32-bit uniform)."""
    p = 1.0 / np.arange(1, n_items + 1, dtype=np.float64) ** s
    cdf = np.cumsum(p / p.sum())
    u = (hash32(seed, name, n, "cpu").numpy().astype(np.float64) + 0.5) / 2.0 ** 32
    return np.minimum(np.searchsorted(cdf, u), n_items - 1).astype(np.int32)


# --------------------------------------------------------------------------------------
# model / workload descriptions
# --------------------------------------------------------------------------------------

@dataclass
class LlamaShape:
    """Llama-style decoder shape (field names follow `tvm/llama_auto_batcher/llama_for_causal_lm.py:10-21`)."""
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    num_hidden_layers: int = 32
    head_dim: int = 128
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0

    @property
    def q_size(self):
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self):
        return self.num_key_value_heads * self.head_dim


LINEARS = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")


def linear_dims(shape: LlamaShape, name: str):
    """(out_features N, in_features K) of a decoder-layer linear."""
    H, I = shape.hidden_size, shape.intermediate_size
    return {
        "q_proj": (shape.q_size, H), "k_proj": (shape.kv_size, H), "v_proj": (shape.kv_size, H),
        "o_proj": (H, shape.q_size), "gate_proj": (I, H), "up_proj": (I, H), "down_proj": (H, I),
    }[name]


@dataclass
class LoraSpec:
    """One adapter type: rank, alpha (scaling = alpha / r, `tvm/llama_auto_batcher/lora.py:13`), targets."""
    r: int = 16
    alpha: float = 8.0
    n_adapters: int = 16
    targets: tuple = ("q_proj", "k_proj", "v_proj", "o_proj")
    a_init: str = "normal"  # "normal" (std 0.02) or "kaiming" (U(-1/sqrt(K), 1/sqrt(K)))

    @property
    def scaling(self):
        return self.alpha / self.r


def base_weights(seed: int, shape: LlamaShape, dtype=torch.float16, device="cpu", layers=None, std=0.02) -> dict:
    """Random-init base model: linears ~N(0, std), norm weights 1.  Keys are HF-style short names."""
    w = {}
    w["embed_tokens"] = normal(seed, "embed_tokens", (shape.vocab_size, shape.hidden_size), std, dtype, device)
    w["lm_head"] = normal(seed, "lm_head", (shape.vocab_size, shape.hidden_size), std, dtype, device)
    w["norm"] = torch.ones(shape.hidden_size, dtype=dtype, device=device)
    for l in (range(shape.num_hidden_layers) if layers is None else layers):
        w.update(layer_weights(seed, shape, l, dtype, device, std))
    return w


def layer_weights(seed: int, shape: LlamaShape, l: int, dtype=torch.float16, device="cpu", std=0.02) -> dict:
    w = {}
    for name in LINEARS:
        N, K = linear_dims(shape, name)
        w[f"layers.{l}.{name}"] = normal(seed, f"layers.{l}.{name}", (N, K), std, dtype, device)
    w[f"layers.{l}.input_layernorm"] = torch.ones(shape.hidden_size, dtype=dtype, device=device)
    w[f"layers.{l}.post_attention_layernorm"] = torch.ones(shape.hidden_size, dtype=dtype, device=device)
    return w


def lora_weights(seed: int, shape: LlamaShape, spec: LoraSpec, dtype=torch.float16, device="cpu",
                 layers=None, tag="a0") -> dict:
    """Stacked adapters in PEFT orientation: A [n_ad, r, K], B [n_ad, N, r]
    (`huggingface/custom_peft/lora_gatherbmm_linear_layer.py:16-17` stacks `lora_A.weight [r,K]`,
    `lora_B.weight [N,r]`)."""
    w = {}
    for l in (range(shape.num_hidden_layers) if layers is None else layers):
        for name in spec.targets:
            N, K = linear_dims(shape, name)
            ka = f"layers.{l}.{name}.lora_A.{tag}"
            kb = f"layers.{l}.{name}.lora_B.{tag}"
            if spec.a_init == "kaiming":
                w[ka] = uniform(seed, ka, (spec.n_adapters, spec.r, K), 1.0 / np.sqrt(K), dtype, device)
            else:
                w[ka] = normal(seed, ka, (spec.n_adapters, spec.r, K), 0.02, dtype, device)
            w[kb] = normal(seed, kb, (spec.n_adapters, N, spec.r), 0.02, dtype, device)
    return w


@dataclass
class Workload:
    name: str
    seed: int
    shape: LlamaShape
    lora: LoraSpec
    batch: int
    prompt_len: int
    gen_len: int
    page_size: int = 16
    dtype: str = "float16"
    adapter_ids: np.ndarray = field(default=None, repr=False)
    ctx_lens: np.ndarray = field(default=None, repr=False)


def config1() -> Workload:
    """2-layer plumbing model, 4 requests x 4 rank-8 adapters on q/v, 128-token prompts, 32 greedy steps."""
    shape = LlamaShape(hidden_size=1024, intermediate_size=2752, num_attention_heads=16, num_key_value_heads=16,
                       num_hidden_layers=2, head_dim=64, vocab_size=32000)
    lora = LoraSpec(r=8, alpha=4.0, n_adapters=4, targets=("q_proj", "v_proj"), a_init="kaiming")
    return Workload("c1_plumbing", 0, shape, lora, batch=4, prompt_len=128, gen_len=32,
                    adapter_ids=np.arange(4, dtype=np.int32))


def llama31_8b_shape(num_layers: int = 32) -> LlamaShape:
    """The reference's default model shape (`tvm/llama_auto_batcher/llama_for_causal_lm.py:12-21`): grouped-query
    attention with 8 kv heads, intermediate size 14336, vocabulary 128256, rope theta 5e5."""
    return LlamaShape(intermediate_size=14336, num_key_value_heads=8, num_hidden_layers=num_layers, vocab_size=128256,
                      rope_theta=500000.0)


def config3(num_layers: int = 32, batch: int = 32, prompt_len: int = 512, gen_len: int = 128, shape: str = "llama2_7b") -> Workload:
    """Llama-2-7B-shape decode: rank-16 adapters on q/k/v/o, 16 adapters round-robin over 32 requests
    (shape="llama31_8b": the same workload on the reference's default model shape)."""
    if shape == "llama31_8b":
        sh, name = llama31_8b_shape(num_layers), "c3_llama31_8b_decode"
    else:
        sh, name = LlamaShape(num_hidden_layers=num_layers), "c3_llama7b_decode"
    lora = LoraSpec(r=16, alpha=8.0, n_adapters=16, targets=("q_proj", "k_proj", "v_proj", "o_proj"))
    return Workload(name, 2, sh, lora, batch=batch, prompt_len=prompt_len, gen_len=gen_len,
                    adapter_ids=(np.arange(batch) % 16).astype(np.int32))


def config4(num_layers: int = 32) -> Workload:
    """Llama-2-7B-shape prefill: 8 x 512 tokens, 64 rank-64 adapters on all 7 linears."""
    shape = LlamaShape(num_hidden_layers=num_layers)
    lora = LoraSpec(r=64, alpha=32.0, n_adapters=64, targets=LINEARS)
    ids = randint(3, "c4.adapter_ids", (8,), 64).numpy()
    return Workload("c4_llama7b_prefill", 3, shape, lora, batch=8, prompt_len=512, gen_len=0, adapter_ids=ids)


def config5(num_layers: int = 32, batch: int = 256) -> Workload:
    """Auto-batching stress: 256 requests, Zipf(1.1) over 256 rank-16 adapters, context 128..2048."""
    shape = LlamaShape(num_hidden_layers=num_layers)
    lora = LoraSpec(r=16, alpha=8.0, n_adapters=256, targets=("q_proj", "k_proj", "v_proj", "o_proj"))
    ids = zipf_ids(4, "c5.adapter_ids", batch, 256, 1.1)
    ctx = 128 + randint(4, "c5.ctx", (batch,), 2048 - 128 + 1).numpy()
    return Workload("c5_autobatch_stress", 4, shape, lora, batch=batch, prompt_len=0, gen_len=64,
                    adapter_ids=ids, ctx_lens=ctx.astype(np.int32))


def prompts(wl: Workload) -> np.ndarray:
    return randint(wl.seed, f"{wl.name}.prompts", (wl.batch, wl.prompt_len), wl.shape.vocab_size).numpy()


def gather_mm_case(seed: int = 1, T: int = 64, K: int = 4096, N: int = 4096, r: int = 16, n_ad: int = 32,
                   device="cpu", tag: str = "") -> dict:
    """Isolated gather-matmul inputs (decode shape): x ~N(0,1), A/B ~N(0,0.02), y_base ~N(0,1), ids uniform."""
    p = f"gmm{tag}"
    return {
        "x": normal(seed, p + ".x", (T, K), 1.0, torch.float16, device),
        "A": normal(seed, p + ".A", (n_ad, r, K), 0.02, torch.float16, device),
        "B": normal(seed, p + ".B", (n_ad, N, r), 0.02, torch.float16, device),
        "y": normal(seed, p + ".y", (T, N), 1.0, torch.float16, device),
        "ids": randint(seed, p + ".ids", (T,), n_ad, device),
        "scaling": 1.0,
    }
