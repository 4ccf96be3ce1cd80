"""Workload definitions and seeded input generators for the MoE dispatch / expert path.

The seeding convention follows the reference's generators: token shard ``s`` is seeded
``seed + s`` (reference utils.py:128,153), the router ``seed + 777`` (utils.py:165-166),
expert weights of rank ``r`` ``seed + 12345 + r`` (utils.py:258).  The distributions are the
ones the workload descriptions state (x ~ N(0,1), router ~ N(0,1/H), weights ~ N(0,1/fan_in)).
Everything is generated on the CPU with ``torch.Generator`` so that the CPU checker and the
GPU path see identical bits.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class MoEConfig:
    name: str
    seed: int
    tokens: int          # T: tokens per source shard (batch * seq)
    hidden: int          # H
    dtype: str           # "f32" | "bf16"  (activation / weight storage type)
    experts: int         # E (global)
    topk: int            # k
    world: int           # W (simulated ranks)
    ffn: int             # F (expert intermediate size)
    act: str             # "gelu" | "silu" | "swiglu"
    bias: str = "none"   # "none" | "normal" | "zipf"  (additive router-logit bias)
    zipf_s: float = 1.2
    quant: str = "none"  # "none" | "fp8"

    @property
    def e_local(self) -> int:
        return self.experts // self.world

    @property
    def torch_dtype(self) -> torch.dtype:
        return {"f32": torch.float32, "bf16": torch.bfloat16}[self.dtype]

    @property
    def n_mat(self) -> int:
        return 3 if self.act == "swiglu" else 2

    def scaled(self, tokens: int) -> "MoEConfig":
        return replace(self, tokens=tokens, name=f"{self.name}@T{tokens}")


CONFIGS: Dict[str, MoEConfig] = {
    # CPU-runnable plumbing case
    "plumbing": MoEConfig("plumbing", 0, 2 * 128, 256, "f32", 8, 2, 4, 512, "gelu"),
    # small-message, dispatch-bound
    "small": MoEConfig("small", 1, 512, 2048, "bf16", 16, 1, 8, 4096, "silu"),
    # Mixtral-style
    "mixtral": MoEConfig("mixtral", 2, 4 * 4096, 4096, "bf16", 8, 2, 8, 14336, "swiglu"),
    # fine-grained DeepSeek-style, per-expert N(0,1) logit bias
    "finegrained": MoEConfig("finegrained", 3, 4096, 7168, "bf16", 256, 8, 8, 2048, "swiglu", bias="normal"),
    # quantised skew sweep (top-k in {1,2,4,8})
    "zipf_k1": MoEConfig("zipf_k1", 4, 8 * 1024, 2048, "bf16", 60, 1, 4, 1408, "swiglu", bias="zipf", quant="fp8"),
    "zipf_k2": MoEConfig("zipf_k2", 4, 8 * 1024, 2048, "bf16", 60, 2, 4, 1408, "swiglu", bias="zipf", quant="fp8"),
    "zipf_k4": MoEConfig("zipf_k4", 4, 8 * 1024, 2048, "bf16", 60, 4, 4, 1408, "swiglu", bias="zipf", quant="fp8"),
    "zipf_k8": MoEConfig("zipf_k8", 4, 8 * 1024, 2048, "bf16", 60, 8, 4, 1408, "swiglu", bias="zipf", quant="fp8"),
}


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    return g


def gen_shard_tokens(cfg: MoEConfig, shard: int) -> torch.Tensor:
    """x_s [T,H] ~ N(0,1) in the config dtype; generator seeded seed + shard."""
    x = torch.randn(cfg.tokens, cfg.hidden, generator=_gen(cfg.seed + shard), dtype=torch.float32)
    return x.to(cfg.torch_dtype)


def gen_router(cfg: MoEConfig) -> torch.Tensor:
    """W_r [H,E] ~ N(0, 1/H), shared by all ranks; generator seeded seed + 777."""
    w = torch.randn(cfg.hidden, cfg.experts, generator=_gen(cfg.seed + 777), dtype=torch.float32)
    return (w / math.sqrt(cfg.hidden)).to(cfg.torch_dtype)


def gen_router_bias(cfg: MoEConfig) -> Optional[torch.Tensor]:
    """fp32 [E] additive logit bias: N(0,1) per expert, or log Zipf(s) popularity (expert 0 hottest)."""
    if cfg.bias == "none":
        return None
    if cfg.bias == "normal":
        return torch.randn(cfg.experts, generator=_gen(cfg.seed + 999), dtype=torch.float32)
    if cfg.bias == "zipf":
        p = torch.arange(1, cfg.experts + 1, dtype=torch.float64) ** (-cfg.zipf_s)
        p = p / p.sum()
        return torch.log(p).to(torch.float32)
    raise ValueError(cfg.bias)


def gen_expert_weights(cfg: MoEConfig, rank: int) -> Tuple[torch.Tensor, ...]:
    """Expert weights of ``rank``, layout [E_l, in, out] (reference utils.py:259), ~N(0,1/fan_in).

    gelu/silu: (w1 [E_l,H,F], w2 [E_l,F,H]);  swiglu: (w_gate [E_l,H,F], w_up [E_l,H,F], w_down [E_l,F,H]).
    """
    g = _gen(cfg.seed + 12345 + rank)
    E_l, H, F = cfg.e_local, cfg.hidden, cfg.ffn

    def mat(i, o):
        w = torch.randn(E_l, i, o, generator=g, dtype=torch.float32)
        return (w / math.sqrt(i)).to(cfg.torch_dtype)

    if cfg.act == "swiglu":
        return mat(H, F), mat(H, F), mat(F, H)
    return mat(H, F), mat(F, H)
