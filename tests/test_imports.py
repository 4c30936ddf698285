"""Every subpackage can be the first thing a program imports: none needs another one
to have been imported before it (a cycle between two of them shows only then)."""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
SUBPACKAGES = ("config", "weights", "parts", "cache", "engine", "sampling", "ops", "entrypoint", "cli")


@pytest.mark.parametrize("name", SUBPACKAGES)
def test_a_subpackage_imports_first(name):
    code = f"import miniserve_amd.{name} as module; print(module.__name__)"
    done = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.strip() == f"miniserve_amd.{name}"
