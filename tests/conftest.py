"""
Test configuration: registers the `gpu` marker and makes the repository root importable.
"""

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config: pytest.Config) -> None:
    config.addinivalue_line('markers', 'gpu: test needs a HIP device (MI355X)')
