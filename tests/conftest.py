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
