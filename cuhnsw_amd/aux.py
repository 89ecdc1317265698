"""Option table and logging helpers of the Python wrapper.

Field names, types and defaults are those of the reference's ConfigProto
(cuhnsw/proto/config.proto:10-26 in js1010/cuhnsw); unknown keys and wrongly typed
values are rejected as the reference's protobuf json_format.Parse does
(cuhnsw/aux.py:60-67).  A plain table replaces protobuf, which is not needed for a
flat option set.
"""
import logging

# name -> (type, default); None default = unset (reads as 0 / False like proto2)
OPTION_TABLE = {
    "seed": (int, 777),
    "c_log_level": (int, 2),
    "py_log_level": (int, 2),
    "max_m": (int, 12),
    "max_m0": (int, 24),
    "ef_construction": (int, 150),
    "level_mult": (float, None),
    "save_remains": (bool, None),
    "hyper_threads": (float, 10.0),
    "block_dim": (int, 32),
    "dist_type": (str, "dot"),
    "visited_table_size": (int, None),
    "visited_list_size": (int, 8192),
    "nrz": (bool, None),
    "reverse_cand": (bool, None),
    "heuristic_coef": (float, 0.25),
}
_ZERO = {int: 0, float: 0.0, bool: False, str: ""}


class Options:
  """Attribute access to a validated option set (stands in for the protobuf message)."""

  def __init__(self, values):
    self.__dict__.update(values)

  def as_dict(self):
    return dict(self.__dict__)


def _coerce(name, typ, value):
  if typ is bool:
    if isinstance(value, (bool,)) or (hasattr(value, "dtype") and value.dtype == bool):
      return bool(value)
    raise ValueError("option %s expects a bool, got %r" % (name, value))
  if typ is int:
    if isinstance(value, bool):
      raise ValueError("option %s expects an int, got %r" % (name, value))
    if isinstance(value, float) and value != int(value):
      raise ValueError("option %s expects an int, got %r" % (name, value))
    try:
      import numbers
      if isinstance(value, numbers.Real) or hasattr(value, "__int__"):
        return int(value)
    except (TypeError, ValueError):
      pass
    raise ValueError("option %s expects an int, got %r" % (name, value))
  if typ is float:
    if isinstance(value, bool) or isinstance(value, str):
      raise ValueError("option %s expects a number, got %r" % (name, value))
    return float(value)
  if not isinstance(value, str):
    raise ValueError("option %s expects a string, got %r" % (name, value))
  return value


def get_opt_as_proto(raw):
  """Validates a dict of options: fills defaults, rejects unknown keys / bad types."""
  raw = dict(raw or {})
  values = {}
  for name, (typ, default) in OPTION_TABLE.items():
    if name in raw:
      values[name] = _coerce(name, typ, raw.pop(name))
    else:
      values[name] = _ZERO[typ] if default is None else default
  if raw:
    raise ValueError("unknown option(s): %s" % ", ".join(sorted(raw)))
  return Options(values)


def proto_to_dict(opt):
  return opt.as_dict()


def get_logger(name, level=2):
  logging.basicConfig(
      format="[%(levelname)-8s] %(asctime)s [%(filename)s] [%(funcName)s:%(lineno)d] %(message)s",
      datefmt="%Y-%m-%d %H:%M:%S")
  logger = logging.getLogger(name)
  if level <= 1:
    logger.setLevel(logging.WARNING)
  elif level == 2:
    logger.setLevel(logging.INFO)
  else:
    logger.setLevel(logging.DEBUG)
  return logger
