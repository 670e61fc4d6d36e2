"""The module-text builders for windowed ops live in the package (reactant.jl_amd/nn_programs.py);
tests use them under this name."""
import importlib

from _loader import load_pkg

load_pkg()
_m = importlib.import_module("reactant_jl_amd.nn_programs")
globals().update({k: getattr(_m, k) for k in dir(_m) if not k.startswith("__")})
