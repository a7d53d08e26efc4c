"""Importable alias of the package directory ``layered-prefill_amd/`` (a hyphen
cannot appear in an ``import`` statement): ``import layered_prefill_amd`` yields
that package."""
import importlib
import os
import sys

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)
sys.modules[__name__] = importlib.import_module("layered-prefill_amd")
