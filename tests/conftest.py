"""Test configuration: the ``gpu`` marker and paths."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config: pytest.Config) -> None:
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config: pytest.Config, items: list[pytest.Item]) -> None:
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter, exitstatus, config) -> None:
    mod = sys.modules.get("test_model_gpu")
    worst = getattr(mod, "WORST", None)
    if worst:
        terminalreporter.write_line("largest logit error as a fraction of its bound, and the test that saw it:")
        for key, (ratio, test) in sorted(worst.items()):
            terminalreporter.write_line(f"  {key} {ratio:.3f}  {test}")
