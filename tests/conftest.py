"""Shared fixtures. GPU tests carry the ``gpu`` marker; everything else runs on the CPU."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(Path(__file__).resolve().parent)):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config: pytest.Config) -> None:
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config: pytest.Config, items: list) -> None:
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory: pytest.TempPathFactory) -> dict[str, Path]:
    """Model folders of the tiny configurations, written once per session by the
    random-weights mode into a temporary folder."""
    from configs import INIT_STD, TINY
    from prefixserve_amd.weights import write_random_model

    out = {}
    for name, cfg in TINY.items():
        d = tmp_path_factory.mktemp(f"tiny-{name}")
        write_random_model(d, cfg, seed=11 + len(out), std=INIT_STD)
        out[name] = d
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs: dict[str, Path]) -> dict:
    from plain.llama_plain import PlainLlama

    return {name: PlainLlama(d) for name, d in model_dirs.items()}


@pytest.fixture(scope="session")
def plain_bf16_error(model_dirs: dict[str, Path], plain_models: dict) -> dict[str, float]:
    """The yardstick for bfloat16: the mean error (per row, relative to the row's largest
    logit) of the plain model when every operation's result is rounded to bfloat16, against
    the plain model in float64. The reference accepts its bfloat16 engine when it is no worse
    than 1.5x a plain bfloat16 run (tests/gpu/test_engine_flashinfer.py:104-108)."""
    import numpy as np

    from configs import TINY
    from plain.llama_plain import PlainLlama

    out = {}
    for name, d in model_dirs.items():
        toks = np.random.default_rng(77).integers(0, TINY[name]["vocab_size"], 130).tolist()
        truth = plain_models[name].logits(toks)
        rough = PlainLlama(d, bf16=True).logits(toks)
        out[name] = float(np.mean(np.abs(rough - truth).max(-1) / np.abs(truth).max(-1)))
    return out
