"""Closed-form parameter-shape lists of the benchmark workloads (no model files, no downloads).

BERT and GPT-2 parameter tensors written out layer by layer in the order a state dict lists them;
only the list of element counts matters to the optimizer step.
"""
from __future__ import annotations

import math
from typing import List, Tuple

import numpy as np

Shape = Tuple[int, ...]


def bert_shapes(hidden: int, ffn: int, layers: int, vocab: int = 30522, positions: int = 512,
                types: int = 2) -> List[Shape]:
    """Embeddings (word, position, type, LayerNorm), `layers` encoder blocks of 16 tensors, pooler."""
    H, F = hidden, ffn
    shapes: List[Shape] = [(vocab, H), (positions, H), (types, H), (H,), (H,)]
    for _ in range(layers):
        shapes += [(H, H), (H,)] * 4          # query, key, value, attention output
        shapes += [(H,), (H,)]                # attention LayerNorm
        shapes += [(F, H), (F,), (H, F), (H,)]  # intermediate, output
        shapes += [(H,), (H,)]                # output LayerNorm
    shapes += [(H, H), (H,)]                  # pooler
    return shapes


def bert_base_shapes() -> List[Shape]:
    return bert_shapes(768, 3072, 12)


def bert_large_shapes() -> List[Shape]:
    return bert_shapes(1024, 4096, 24)


def gpt2_shapes(hidden: int = 1600, ffn: int = 6400, layers: int = 48, vocab: int = 50257,
                positions: int = 1024) -> List[Shape]:
    """wte, wpe, `layers` blocks of 12 tensors, final LayerNorm (GPT-2 1.5B by default)."""
    H, F = hidden, ffn
    shapes: List[Shape] = [(vocab, H), (positions, H)]
    for _ in range(layers):
        shapes += [(H,), (H,)]                # ln_1
        shapes += [(H, 3 * H), (3 * H,)]      # attn.c_attn
        shapes += [(H, H), (H,)]              # attn.c_proj
        shapes += [(H,), (H,)]                # ln_2
        shapes += [(H, F), (F,)]              # mlp.c_fc
        shapes += [(F, H), (H,)]              # mlp.c_proj
    shapes += [(H,), (H,)]                    # ln_f
    return shapes


def log_uniform_numels(count: int = 2000, lo: int = 1, hi: int = 65536, seed: int = 2024) -> List[int]:
    """`count` sizes with log-uniform distribution in [lo, hi] (the many-tiny-tensors workload)."""
    rng = np.random.default_rng([seed, 4])
    u = rng.uniform(math.log(lo), math.log(hi), size=count)
    return [int(min(hi, max(lo, math.floor(math.exp(x))))) for x in u]


def numels(shapes) -> List[int]:
    return [int(np.prod(s, dtype=np.int64)) for s in shapes]
