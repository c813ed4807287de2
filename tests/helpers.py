"""Shared helpers for the parity tests: seeded inputs, oracle <-> device plumbing,
ulp comparisons.  The oracle is the checker only; the device path under test is
always libnabla_optim.so through nabla_amd.optim."""
from __future__ import annotations

import numpy as np

import oracle as O

# ---- configuration shapes of the benchmark contract --------------------------------

MLP_SHAPES = [(784, 256), (1, 256), (256, 128), (1, 128), (128, 10), (1, 10)]  # 235,146 params


def gpt2_small_shapes():
    """148 tensors, 124,439,808 params."""
    s = []
    for _ in range(12):
        s += [(768, 2304), (1, 2304), (768, 768), (1, 768), (768, 3072), (1, 3072),
              (3072, 768), (1, 768), (1, 768), (1, 768), (1, 768), (1, 768)]
    s += [(50257, 768), (1024, 768), (1, 768), (1, 768)]
    return s


def llama_shapes(layers, hidden, kv, ffn, vocab):
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


# ---- seeded tensors (the reference's xorshift64 + Box-Muller stream) ----------------

def randn_list(shapes, seed0, sigma, dtype=np.float32):
    out = []
    for i, (r, c) in enumerate(shapes):
        n = r * c
        a = O.randn_f64(n, seed0 + i) * sigma
        out.append(a.astype(dtype))
    return out


def zeros_like_list(arrs):
    return [np.zeros_like(a) for a in arrs]


def copy_list(arrs):
    return [a.copy() for a in arrs]


# ---- numpy <-> torch (device) -----------------------------------------------------------

def to_dev(arr, shape=None):
    import torch

    if arr.dtype == np.uint16:  # bf16 bit patterns
        t = torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16)
    else:
        t = torch.from_numpy(arr.copy())
    t = t.to("cuda:0")
    if shape is not None:
        t = t.reshape(shape)
    return t


def to_host(t):
    import torch

    t = t.detach().reshape(-1).cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def dev_list(arrs, shapes):
    return [to_dev(a, s) for a, s in zip(arrs, shapes)]


def host_list(tensors):
    return [to_host(t) for t in tensors]


# ---- comparisons ---------------------------------------------------------------------------

def max_ulp_f32(a_list, b_list):
    worst = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            worst = max(worst, int(O.ulp_distance_f32(a, b).max()))
    return worst


def max_ulp_bf16(a_list, b_list):
    worst = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            worst = max(worst, int(O.ulp_distance_bf16(a, b).max()))
    return worst


def assert_bits_equal(a_list, b_list, what):
    for i, (a, b) in enumerate(zip(a_list, b_list)):
        av = a.view(np.uint32) if a.dtype == np.float32 else (
            a.view(np.uint64) if a.dtype == np.float64 else a)
        bv = b.view(np.uint32) if b.dtype == np.float32 else (
            b.view(np.uint64) if b.dtype == np.float64 else b)
        if not np.array_equal(av, bv):
            bad = np.nonzero(av != bv)[0]
            raise AssertionError(
                f"{what}: tensor {i} differs in {bad.size}/{a.size} elements, first at {bad[0]}: "
                f"{a[bad[0]]!r} vs {b[bad[0]]!r}")


def count_beyond_ulp_f32(a_list, b_list, tol):
    """(#elements beyond tol ulp, total) over a list."""
    n_bad = 0
    total = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            n_bad += int((O.ulp_distance_f32(a, b) > tol).sum())
            total += a.size
    return n_bad, total
