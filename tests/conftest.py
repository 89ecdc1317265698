import json
import os
import sys

import numpy as np
import pytest

# torch (used by GPU tests only to hold device buffers) ships its own copy of the HIP
# runtime: it has to be loaded before libcuhnsw_amd.so pulls in the system one, or the
# process ends up with two runtimes and torch finds no GPU.
try:
  import torch  # noqa: F401  pylint: disable=unused-import
except ImportError:
  torch = None

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)


def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def write_options(tmp_path, **over):
  """Option file as the Python wrapper writes it (all fields, defaults filled)."""
  from cuhnsw_amd import aux
  opt = aux.proto_to_dict(aux.get_opt_as_proto(over))
  if not opt["level_mult"]:
    opt["level_mult"] = 1.0 / np.log(opt["max_m"])
  path = os.path.join(str(tmp_path), "opt.json")
  with open(path, "w") as f:
    json.dump(opt, f)
  return path, opt


@pytest.fixture(scope="session")
def oracle():
  from oracle import oracle as orc
  orc.lib()
  return orc
