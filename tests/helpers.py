"""Shared helpers for the tests: package loading and f32-valued operand views."""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pkg(sub=None):
    """The product package lives in a directory whose name is not an identifier."""
    name = "tpu-mlir_amd" if sub is None else "tpu-mlir_amd." + sub
    return importlib.import_module(name)


def f32_valued_a16(cfg):
    """Native-dtype synthetic operands expanded to the interpreter's f32-valued convention."""
    return pkg("synth").f32_valued_a16(cfg)
