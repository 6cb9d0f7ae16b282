"""Shared test plumbing: import paths, the `gpu` marker and seeded input builders."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "fp-quant_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# The library's documented opt-out switches; the suite runs under each of them as well as under the defaults.
PACKED_WEIGHTS = os.environ.get("FPQ_PACKED_WEIGHTS", "1") != "0"
SINGLE_WEIGHT_COPY = os.environ.get("FPQ_SINGLE_WEIGHT_COPY", "0") == "1"
needs_packed = pytest.mark.skipif(
    not PACKED_WEIGHTS, reason="FPQ_PACKED_WEIGHTS=0 switches the packed operand path off, which this test is about")
needs_row_major_parameters = pytest.mark.skipif(
    SINGLE_WEIGHT_COPY, reason="FPQ_SINGLE_WEIGHT_COPY=1 releases the row-major parameters this test reads or hands on")


def row_major_weights(lin):
    """(qweight [N, K/2], scales [N, K/group]) of an FPQuantLinear as the reference holds them, on the CPU --
    through state_dict(), which re-tiles a layer that keeps its weight in the packed layout only (whose
    `qweight` / `scales` parameters are 1-D buffers and must not be indexed by output feature)."""
    sd = lin.state_dict()
    return sd["qweight"].detach().cpu(), sd["scales"].detach().cpu()


def packed_copy(lin):
    """(codes, scales) of the layer's weight in the packed operand layout, or None if it has none (yet)."""
    q = lin.qweight
    if q.dim() == 1:
        return q, lin.scales
    hit = getattr(q, "_fpq_packed", None)
    return None if hit is None else (hit[1], hit[2])


def make_outlier_normal(rows, cols, seed, frac=0.005, mult=25.0):
    """N(0,1) with a seeded Bernoulli(frac) mask scaling entries by `mult`, cast to bf16."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=gen)
    mask = torch.rand(rows, cols, generator=gen) < frac
    return torch.where(mask, x * mult, x).to(torch.bfloat16)


def make_student_t(rows, cols, seed, df=3):
    """Student-t(df) as randn / sqrt(chi2(df)/df) from one seeded generator, cast to bf16."""
    gen = torch.Generator().manual_seed(seed)
    z = torch.randn(rows, cols, generator=gen)
    chi = torch.randn(df, rows, cols, generator=gen).pow(2).sum(0)
    return (z / torch.sqrt(chi / df)).to(torch.bfloat16)
