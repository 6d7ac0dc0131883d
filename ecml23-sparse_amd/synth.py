"""Seeded synthetic inputs for the fixed-fan-in layer at the benchmark configurations.

The reference ships no datasets; its native tests and benchmarks draw random tensors
(testing/test_case_templates.h:52-69, testing/quick-bench.cpp:12-35).  This module draws tensors of
the shapes and laws the benchmark configurations name, with torch generators, on any device.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class FfiConfig:
    name: str
    batch: int
    num_features: int
    num_units: int
    fan_in: int
    x_law: str = "relu_normal"      # "relu_normal" | "l2_abs_normal" | "uniform"
    distinct: bool = True           # distinct column ids inside a lookup row
    sorted_rows: bool = False


CONFIGS = {
    # the reference's CPU-runnable case
    "c1": FfiConfig("c1", 32, 768, 131_072, 32),
    # headline: Amazon-670k-sized output layer on 768-d encoder features
    "c2": FfiConfig("c2", 128, 768, 670_091, 32),
    # Wiki-500k-sized layer, unit-norm non-negative inputs
    "c3": FfiConfig("c3", 256, 512, 501_070, 64, x_law="l2_abs_normal"),
    # wide intermediate layer, fan-in not a power of two
    "c4": FfiConfig("c4", 128, 65_536, 670_091, 72),
    # inference variant: sorted rows (bf16 storage is applied by the caller)
    "c5": FfiConfig("c5", 512, 100_000, 670_091, 64, sorted_rows=True),
}


def make_lookup(num_units, fan_in, num_features, *, distinct=True, sorted_rows=False, generator=None,
                device="cpu"):
    """int32 [num_units, fan_in] column ids, uniform in [0, num_features).

    With ``distinct`` every row holds ``fan_in`` different ids (the benchmark law); without it ids
    are drawn with replacement, which is what the reference layer itself does
    (sparse/custom_layer.py:12-15) and what its tests exercise (test_case_templates.h:59-64).
    """
    if distinct and fan_in > num_features:
        raise ValueError("cannot draw more distinct ids than there are features")
    if not distinct:
        idx = torch.randint(0, num_features, (num_units, fan_in), generator=generator, device=device, dtype=torch.int64)
    elif num_features <= 8192:
        # random keys per row, take the positions of the fan_in smallest: a uniform K-subset in random order
        rows_per_chunk = max(1, (1 << 26) // num_features)
        parts = []
        for r0 in range(0, num_units, rows_per_chunk):
            r = min(rows_per_chunk, num_units - r0)
            keys = torch.rand((r, num_features), generator=generator, device=device)
            parts.append(torch.topk(keys, fan_in, dim=1, largest=False, sorted=True).indices)
        idx = torch.cat(parts, dim=0)
    else:
        # wide inputs: draw with replacement, redraw the rows that hold a duplicate until none is left
        idx = torch.randint(0, num_features, (num_units, fan_in), generator=generator, device=device, dtype=torch.int64)
        for _ in range(1000):
            srt = torch.sort(idx, dim=1).values
            bad = (srt[:, 1:] == srt[:, :-1]).any(dim=1).nonzero().squeeze(1)
            if bad.numel() == 0:
                break
            idx[bad] = torch.randint(0, num_features, (bad.numel(), fan_in), generator=generator, device=device, dtype=torch.int64)
        else:
            raise RuntimeError("could not draw distinct lookup rows")
    if sorted_rows:
        idx = torch.sort(idx, dim=1).values
    return idx.to(torch.int32).contiguous()


def make_features(batch, num_features, law="relu_normal", *, generator=None, device="cpu"):
    """float32 [batch, num_features] inputs."""
    if law == "uniform":
        return torch.rand((batch, num_features), generator=generator, device=device) * 2 - 1
    x = torch.randn((batch, num_features), generator=generator, device=device)
    if law == "relu_normal":
        return torch.relu(x)
    if law == "l2_abs_normal":
        x = x.abs()
        return x / x.norm(dim=1, keepdim=True)
    raise ValueError(f"unknown feature law {law!r}")


def make_inputs(cfg: FfiConfig, seed: int = 42, device="cpu", transposed: bool = False, num_units=None):
    """Returns dict(features, lookup, weights, out_grad) for ``cfg``.

    ``features`` is [B,N], or [N,B] (contiguous) when ``transposed``.  weights ~ N(0, 1/K)
    (variance), out_grad ~ N(0, 1e-2) (variance).  ``num_units`` overrides cfg.num_units to draw a
    bounded sample of the same workload.
    """
    L = int(num_units or cfg.num_units)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    features = make_features(cfg.batch, cfg.num_features, cfg.x_law, generator=gen, device=device)
    if transposed:
        features = features.t().contiguous()
    lookup = make_lookup(L, cfg.fan_in, cfg.num_features, distinct=cfg.distinct, sorted_rows=cfg.sorted_rows,
                         generator=gen, device=device)
    weights = torch.randn((L, cfg.fan_in), generator=gen, device=device) * (cfg.fan_in ** -0.5)
    out_grad = torch.randn((cfg.batch, L), generator=gen, device=device) * 0.1
    return {"features": features, "lookup": lookup, "weights": weights, "out_grad": out_grad}


def _splitmix64(seed: int, first: int, count: int):
    """Draws first .. first+count-1 of the counter-based generator the C++ caller uses (tests/cpp/cabi_harness.cpp):
    draw i of seed s is mix(s + (i + 1) * 0x9e3779b97f4a7c15) with splitmix64's finaliser."""
    import numpy as np

    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (np.arange(first + 1, first + count + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def counter_case(batch, num_features, num_units, fan_in, transposed=False, seed=42):
    """One case of the reference's test law (testing/test_case_templates.h:52-69,113-114: uniform [-1,1) features and
    weights, column ids uniform with replacement, out_grad clipped at zero), drawn from the seeded counter-based
    generator that the C++ caller of the C ABI draws from too: both produce the same bits for the same seed, so a
    case can be run on one side and checked on the other.  numpy arrays (features, lookup, weights, out_grad)."""
    import numpy as np

    def uniform(first, count):
        return ((_splitmix64(seed, first, count) >> np.uint64(11)).astype(np.float64) * (2.0 / 9007199254740992.0) - 1.0).astype(np.float32)

    B, N, L, K = batch, num_features, num_units, fan_in
    at = 0
    x = uniform(at, B * N).reshape(B, N); at += B * N
    lookup = (_splitmix64(seed, at, L * K) % np.uint64(N)).astype(np.int32).reshape(L, K); at += L * K
    w = uniform(at, L * K).reshape(L, K); at += L * K
    g = np.maximum(uniform(at, B * L), 0).astype(np.float32).reshape(B, L)
    features = np.ascontiguousarray(x.T) if transposed else x
    return features, lookup, w, g


def algorithmic_bytes(cfg: FfiConfig, num_units=None):
    """Compulsory HBM traffic per pass (every input read once, every output written once), bytes."""
    B, N, K = cfg.batch, cfg.num_features, cfg.fan_in
    L = int(num_units or cfg.num_units)
    fwd = 4 * L * K + 4 * L * K + 4 * B * N + 4 * B * L          # W, idx, x, out
    gx = 4 * L * K + 4 * L * K + 4 * B * L + 4 * B * N           # W, idx, g, gx
    gw = 4 * L * K + 4 * B * L + 4 * B * N + 4 * L * K           # idx, g, x, gW
    return {"forward": fwd, "input_grad": gx, "weight_grad": gw, "total": fwd + gx + gw}
