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

    return {name: rows[0] for name, rows in _plain_bf16_rows(model_dirs, plain_models).items()}


_BF16_ROWS: dict = {}


def _plain_bf16_rows(model_dirs, plain_models) -> dict[str, tuple[float, float]]:
    """name -> (mean over the rows of the first 130 tokens, worst row over four such sequences) of
    a plain bfloat16 run against the plain model in float64."""
    import numpy as np

    from configs import TINY
    from plain.llama_plain import PlainLlama

    if not _BF16_ROWS:
        for name, d in model_dirs.items():
            rng = np.random.default_rng(77)
            rough = PlainLlama(d, bf16=True)
            rows = []
            for _ in range(4):
                toks = rng.integers(0, TINY[name]["vocab_size"], 130).tolist()
                truth = plain_models[name].logits(toks)
                rows.append(np.abs(rough.logits(toks) - truth).max(-1) / np.abs(truth).max(-1))
            _BF16_ROWS[name] = (float(np.mean(rows[0])), float(np.max(rows)))
    return _BF16_ROWS


@pytest.fixture(scope="session")
def bf16_row_bar(model_dirs: dict[str, Path], plain_models: dict) -> dict[str, float]:
    """The bar for a single row of bfloat16 logits: 1.5 x the worst row of a plain bfloat16 run
    of the same model (520 rows). How far rounding to 8 bits moves a row depends on the model
    (its depth, its widths, how large its logits are), not on the engine: a fixed number is too
    tight for some configurations and too loose for others."""
    from configs import BF16_ROW_FACTOR

    return {name: BF16_ROW_FACTOR * rows[1] for name, rows in _plain_bf16_rows(model_dirs, plain_models).items()}
