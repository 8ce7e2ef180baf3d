"""Shapes of the synthetic workloads the primitives are measured and tested on.

Pure shape arithmetic (no tensors): the Llama-3-8B decoder layer and full model, the uneven
flat-parameter set, and the shard sizes each implies. Shared by bench.py and the tests.
"""

from __future__ import annotations

import math
from typing import List, Tuple

HIDDEN, FFN, Q_HEADS, KV_HEADS, HEAD_DIM, VOCAB, LAYERS = 4096, 14336, 32, 8, 128, 128256, 32


def llama3_8b_layer_shapes() -> List[Tuple[str, Tuple[int, ...]]]:
    """The 9 parameters of one decoder layer, 218 112 000 elements in all."""
    return [
        ("input_layernorm", (HIDDEN,)),
        ("q_proj", (Q_HEADS * HEAD_DIM, HIDDEN)),
        ("k_proj", (KV_HEADS * HEAD_DIM, HIDDEN)),
        ("v_proj", (KV_HEADS * HEAD_DIM, HIDDEN)),
        ("o_proj", (HIDDEN, Q_HEADS * HEAD_DIM)),
        ("post_attention_layernorm", (HIDDEN,)),
        ("gate_proj", (FFN, HIDDEN)),
        ("up_proj", (FFN, HIDDEN)),
        ("down_proj", (HIDDEN, FFN)),
    ]


def llama3_8b_units() -> List[Tuple[str, List[Tuple[str, Tuple[int, ...]]]]]:
    """FSDP units of the full model in forward order: embedding, 32 layers, final norm + untied
    lm_head; 8 030 261 248 elements."""
    units = [("embed_tokens", [("embed_tokens", (VOCAB, HIDDEN))])]
    for i in range(LAYERS):
        units.append((f"layers.{i}", llama3_8b_layer_shapes()))
    units.append(("head", [("norm", (HIDDEN,)), ("lm_head", (VOCAB, HIDDEN))]))
    return units


def numel(shape) -> int:
    return math.prod(shape)


def shard_numel(n: int, world_size: int) -> int:
    """Flat-parameter rule: every rank holds ceil(n / W) elements, the tail zero padded."""
    return -(-n // world_size)


def uneven_flat_numels(count: int = 40, world_size: int = 12, lo: int = 4096,
                       hi: int = 58_720_256, seed: int = 0) -> List[int]:
    """``count`` sizes drawn log-uniformly in [lo, hi] from a seeded torch generator, each
    bumped until it is not divisible by ``world_size``."""
    import torch

    g = torch.Generator().manual_seed(seed)
    u = torch.rand(count, generator=g, dtype=torch.float64)
    out = []
    for x in u.tolist():
        n = int(math.floor(math.exp(math.log(lo) + x * (math.log(hi) - math.log(lo)))))
        while n % world_size == 0:
            n += 1
        out.append(n)
    return out
