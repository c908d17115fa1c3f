"""Helpers shared by the GPU parity tests (imported only by tests marked ``gpu``)."""
from __future__ import annotations

import sys

import numpy as np

import oracle
from helpers import logical, rng


_dev = None


def device():
    """One Rocm context per test process; fails loudly when the HIP library is missing."""
    global _dev
    if _dev is None:
        from dfdx_amd import Rocm

        _dev = Rocm(0)
    return _dev


def announce(*what):
    """Name the case on stdout before touching the GPU, so a fault can be attributed."""
    print("[gpu-case]", *what, flush=True)
    sys.stdout.flush()


def make_operand(g, rows, cols, transposed, dtype, pad=0, scale=1.0, dist="normal"):
    """Storage + strides of a (rows, cols) matrix view; `transposed` stores it as (cols, rows)."""
    r, c = (cols, rows) if transposed else (rows, cols)
    ld = c + pad
    vals = g.standard_normal((r, ld)) if dist == "normal" else g.uniform(-1.0, 1.0, (r, ld))
    st = oracle.to_storage((vals * scale).reshape(-1), dtype)
    strides = (1, ld) if transposed else (ld, 1)
    return st, strides


def values(st, dtype, shape, strides, offset=0):
    return logical(oracle.to_f64(st, dtype), shape, strides, offset)
