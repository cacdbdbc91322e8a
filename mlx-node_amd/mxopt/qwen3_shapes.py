"""Qwen3 parameter lists (name, shape), in the order and with the names the reference expects
(crates/mlx-core/src/param_manager.rs:125-152).  Used to size benchmark and test workloads;
no weights are involved."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Tuple


@dataclass(frozen=True)
class Qwen3Dims:
    vocab: int
    hidden: int
    layers: int
    q_heads: int
    kv_heads: int
    head_dim: int
    intermediate: int
    tied: bool


QWEN3 = {
    "0.6B": Qwen3Dims(151936, 1024, 28, 16, 8, 128, 3072, True),
    "1.7B": Qwen3Dims(151936, 2048, 28, 16, 8, 128, 6144, True),
    "4B": Qwen3Dims(151936, 2560, 36, 32, 8, 128, 9728, True),
    "8B": Qwen3Dims(151936, 4096, 36, 32, 8, 128, 12288, False),
}


def param_list(d: Qwen3Dims) -> List[Tuple[str, Tuple[int, ...]]]:
    out: List[Tuple[str, Tuple[int, ...]]] = [("embedding.weight", (d.vocab, d.hidden))]
    for i in range(d.layers):
        pre = f"layers.{i}"
        out += [
            (f"{pre}.self_attn.q_proj.weight", (d.q_heads * d.head_dim, d.hidden)),
            (f"{pre}.self_attn.k_proj.weight", (d.kv_heads * d.head_dim, d.hidden)),
            (f"{pre}.self_attn.v_proj.weight", (d.kv_heads * d.head_dim, d.hidden)),
            (f"{pre}.self_attn.o_proj.weight", (d.hidden, d.q_heads * d.head_dim)),
            (f"{pre}.self_attn.q_norm.weight", (d.head_dim,)),
            (f"{pre}.self_attn.k_norm.weight", (d.head_dim,)),
            (f"{pre}.mlp.gate_proj.weight", (d.intermediate, d.hidden)),
            (f"{pre}.mlp.up_proj.weight", (d.intermediate, d.hidden)),
            (f"{pre}.mlp.down_proj.weight", (d.hidden, d.intermediate)),
            (f"{pre}.input_layernorm.weight", (d.hidden,)),
            (f"{pre}.post_attention_layernorm.weight", (d.hidden,)),
        ]
    out.append(("final_norm.weight", (d.hidden,)))
    if not d.tied:
        out.append(("lm_head.weight", (d.vocab, d.hidden)))
    return out


def numel(shape: Tuple[int, ...]) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


def total_elems(name: str) -> int:
    return sum(numel(s) for _, s in param_list(QWEN3[name]))
