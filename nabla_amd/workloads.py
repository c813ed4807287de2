"""Tensor-shape lists of the benchmark configurations (synthetic parameter sets).

Each function returns a list of (rows, cols); only rows*cols matters to the
optimizer.  The shapes are those of the model families the configurations name;
no model is built.
"""
from __future__ import annotations

import numpy as np

# README MLP 784 -> 256 -> 128 -> 10 with biases: 6 tensors, 235,146 params
MLP_SHAPES = [(784, 256), (1, 256), (256, 128), (1, 128), (128, 10), (1, 10)]


def gpt2_small_shapes():
    """148 tensors, 124,439,808 params."""
    s = []
    for _ in range(12):
        s += [(768, 2304), (1, 2304), (768, 768), (1, 768), (768, 3072), (1, 3072),
              (3072, 768), (1, 768), (1, 768), (1, 768), (1, 768), (1, 768)]
    s += [(50257, 768), (1024, 768), (1, 768), (1, 768)]
    return s


def llama_shapes(layers, hidden, kv, ffn, vocab):
    """Per layer: q, k, v, o, gate, up, down, 2 RMSNorm; plus embed and lm_head."""
    s = []
    for _ in range(layers):
        s += [(hidden, hidden), (hidden, kv), (hidden, kv), (hidden, hidden),
              (hidden, ffn), (hidden, ffn), (ffn, hidden), (1, hidden), (1, hidden)]
    s += [(vocab, hidden), (vocab, hidden)]
    return s


def llama_1b_shapes():
    """200 tensors, 1,100,046,336 params."""
    return llama_shapes(22, 2048, 256, 5632, 32000)


def llama_8b_shapes():
    """290 tensors, 8,030,257,152 params."""
    return llama_shapes(32, 4096, 1024, 14336, 128256)


def ragged_sizes(n_tensors=4096, lo=1, hi=65536, seed=1234):
    """Sizes log-uniform in [lo, hi] from a seeded stream."""
    rng = np.random.default_rng(seed)
    u = rng.random(n_tensors)
    sizes = np.floor(np.exp(u * np.log(hi / lo)) * lo).astype(np.int64)
    return [int(min(max(x, lo), hi)) for x in sizes]


def n_params(shapes):
    return sum(r * c for r, c in shapes)
