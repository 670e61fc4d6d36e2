"""Import the package directory `reactant.jl_amd` (its name is not a valid
Python identifier) under the module name `reactant_jl_amd`."""
import importlib.util
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "reactant.jl_amd")


def load_pkg():
    if "reactant_jl_amd" in sys.modules:
        return sys.modules["reactant_jl_amd"]
    spec = importlib.util.spec_from_file_location(
        "reactant_jl_amd", os.path.join(PKG_DIR, "__init__.py"), submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["reactant_jl_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def load_programs():
    load_pkg()
    import importlib
    return importlib.import_module("reactant_jl_amd.programs")
