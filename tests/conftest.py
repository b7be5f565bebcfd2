"""Shared fixtures.  `-m "not gpu"` covers the oracle (against the reference's own compiled code and against closed
forms), the host logic and the ABI surface; `-m gpu` runs the HIP kernels through the C ABI and the ggml plugin through
the unmodified whisper.cpp host, against the oracle and the reference's CPU backend."""
from __future__ import annotations

import importlib.util
import json
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    mod = entry.oracle()
    mod.lib()          # builds oracle/liboracle_ops.so on first use
    return mod


@pytest.fixture(scope="session")
def ref():
    """the reference's compiled libraries (oracle/_ref); built here when the whisper.cpp tree is mounted"""
    import ggml_ref
    if not ggml_ref.available():
        b = entry.builder()
        if not b.have_reference():
            pytest.skip("oracle/_ref is not built and the whisper.cpp tree is not mounted")
        b.build_reference()
    ggml_ref.libs()
    return ggml_ref


@pytest.fixture(scope="session")
def pkg():
    return entry.package()


@pytest.fixture(scope="session")
def harness():
    """path of the harness binary; built here when missing and the whisper.cpp tree is mounted"""
    pkg = entry.package()
    if not pkg.HARNESS_BIN.exists():
        b = entry.builder()
        if not b.have_reference():
            pytest.skip("harness is not built and the whisper.cpp tree is not mounted")
        b.build_all()
    return pkg.HARNESS_BIN


def run_harness(binary, args, timeout=600, env=None, check=True):
    """run the harness, return (returncode, list of parsed JSON lines)"""
    res = subprocess.run([str(binary), *args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout,
                         env={**os.environ, **(env or {})})
    rows = []
    for line in res.stdout.splitlines():
        if line.startswith("{"):
            rows.append(json.loads(line))
    if check and res.returncode not in (0, 1):
        raise AssertionError(f"harness {args} exited with {res.returncode}:\n{res.stderr[-3000:]}")
    return res.returncode, rows
