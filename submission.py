"""Drop-in for the reference's submission module: ``from submission import custom_kernel``
(README.md:94-95 of the reference shows the harness importing exactly this name)."""
import importlib
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
_pkg = importlib.import_module("amd-developer-challenge-2025_amd")

custom_kernel = _pkg.custom_kernel
grouped_kernel = _pkg.grouped_kernel
