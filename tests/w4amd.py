"""Imports the shipped package (its directory name is not a Python identifier)
and offers torch-side helpers for the GPU tests."""
import importlib.util
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "w4a16-dequant-gemm_amd")


def package():
    name = "w4a16_dequant_gemm_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(
        name, os.path.join(PKG_DIR, "__init__.py"), submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def capi():
    return package().capi


def load():
    return capi().load()
