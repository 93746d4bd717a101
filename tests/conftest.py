"""Shared pytest set-up: the ``gpu`` marker, import paths, built artefacts."""

from __future__ import annotations

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # The oracle is small C; build it once if the shared object is missing.
    from oracle import nf4_oracle

    nf4_oracle.build(force=False)
    # The HIP library is built ahead of time (hipcc cross-compiles).  Where the toolchain
    # is at hand, rebuild when a source is newer than the library, so that an edited
    # kernel is never tested through a stale build; without hipcc use what is there.
    from deepfold_amd import build_ext

    if not os.path.exists(build_ext.LIB):
        build_ext.build(force=True)
    elif build_ext.stale() and build_ext.have_hipcc():
        build_ext.build(force=True)


def pytest_collection_modifyitems(config, items):
    try:
        import torch

        have_gpu = torch.cuda.is_available()
    except Exception:  # pragma: no cover
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
