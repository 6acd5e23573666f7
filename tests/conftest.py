"""Shared pytest configuration: the `gpu` marker, repo root on sys.path, golden loader."""
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_golden(stem):
    """Returns (cases, arrays): the JSON index (or None) and the npz arrays of one fixture."""
    arrays = np.load(os.path.join(GOLDEN_DIR, stem + ".npz"), allow_pickle=False)
    index_path = os.path.join(GOLDEN_DIR, stem + ".json")
    cases = None
    if os.path.exists(index_path):
        with open(index_path) as f:
            cases = json.load(f)
    return cases, arrays


@pytest.fixture(scope="session")
def golden():
    return load_golden
