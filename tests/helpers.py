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
    """Expand native-dtype synthetic operands to the interpreter's f32-valued convention
    (every tensor a float array; packed bytes 0..255, bf16 values widened)."""
    S = pkg("synth")
    x = S.bf16_to_f32(cfg["x"])
    w = cfg["weight"].astype(np.float32)
    scale = S.bf16_to_f32(cfg["scale"])
    zp = cfg["zp"].astype(np.float32)
    bias = None if cfg.get("bias") is None else S.bf16_to_f32(cfg["bias"])
    return x, w, scale, zp, bias
