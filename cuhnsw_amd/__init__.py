"""MI355X-native HNSW engine with the cuhnsw Python API.

`from cuhnsw_amd import CuHNSW` loads the native extension (and fails if it is
not built).  `cuhnsw_amd.datasets` and `cuhnsw_amd.build` import without it.
"""


def __getattr__(name):
  if name == "CuHNSW":
    from cuhnsw_amd.pyhnsw import CuHNSW
    return CuHNSW
  raise AttributeError(name)
