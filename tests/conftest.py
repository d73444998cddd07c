import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (ROOT, os.path.join(ROOT, "tests")):
  if _p not in sys.path:
    sys.path.insert(0, _p)


def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X")


def _has_gpu() -> bool:
  try:
    import torch

    return torch.cuda.is_available()
  except Exception:
    return False


def pytest_collection_modifyitems(config, items):
  if _has_gpu():
    return
  skip = pytest.mark.skip(reason="no GPU visible")
  for item in items:
    if "gpu" in item.keywords:
      item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def _current_library():
  """Before the first test of a session touches the library: make sure that what is built comes from the sources in the
  tree (a test that loaded a stale library first would keep it mapped for the whole session)."""
  from maxdiffusion_amd import build

  try:
    build.ensure_built()
  except RuntimeError as e:
    if "hipcc not found" not in str(e):
      raise
    # no compiler on this machine: tests of the oracle and of the host logic still run; the `lib` fixture below
    # fails the ones that need the library


@pytest.fixture(scope="session")
def lib():
  """The built C-ABI library; built here only if nothing is built yet or what is built comes from other sources."""
  from maxdiffusion_amd import _lib, build

  build.ensure_built()
  return _lib.load()


@pytest.fixture(scope="session")
def dev(lib):
  import torch

  return torch.device("cuda:0")
