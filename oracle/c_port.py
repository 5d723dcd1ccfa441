"""ctypes binding of the C restatement (oracle/c/w3_oracle.c). Test infrastructure, as everything under oracle/."""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from functools import lru_cache
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIBRARY = HERE / "_build" / "libw3_oracle.so"


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-s"], check=True)
    return LIBRARY


class Experts(C.Structure):
    _fields_ = [("planes13", C.c_void_p), ("scales13", C.c_void_p), ("row13", C.c_void_p), ("planes2", C.c_void_p), ("scales2", C.c_void_p),
                ("row2", C.c_void_p), ("levels13", C.c_void_p), ("levels2", C.c_void_p), ("experts", C.c_int), ("base", C.c_int),
                ("hidden", C.c_int), ("inter", C.c_int), ("gated", C.c_int)]


@lru_cache(maxsize=1)
def lib() -> C.CDLL:
    if not LIBRARY.exists():
        build()
    h = C.CDLL(str(LIBRARY))
    h.w3o_moe_layer.restype = C.c_int
    h.w3o_last_unpack_seconds.restype = C.c_double
    return h


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _levels(codebook) -> np.ndarray:
    out = np.zeros(8, np.float32)
    out[:len(codebook)] = codebook
    return out


def codes(planes: np.ndarray, rows: int, k: int, bits: int = 3) -> np.ndarray:
    planes = np.ascontiguousarray(planes, np.uint32)
    out = np.empty((rows, k), np.uint8)
    lib().w3o_codes(_p(planes), C.c_int64(rows), k, bits, _p(out))
    return out


def dequantize(w3: dict) -> np.ndarray:
    planes, scales = np.ascontiguousarray(w3["planes"], np.uint32), np.ascontiguousarray(w3["scales"], np.uint8)
    row, lv = np.ascontiguousarray(w3["row_scale"], np.float32), _levels(w3["codebook"])
    n, k = w3["out_features"], w3["in_features"]
    out = np.empty((n, k), np.float32)
    lib().w3o_dequantize(_p(planes), _p(scales), _p(row), _p(lv), C.c_int64(n), k, planes.shape[2], _p(out))
    return out


class HostExperts:
    """Stacked experts in the checkpoint layout as contiguous numpy arrays (kept alive for the C calls)."""

    def __init__(self, planes13, scales13, row13, planes2, scales2, row2, codebook, fc2_codebook, hidden, inter, gated, base=0):
        self.arrays = [np.ascontiguousarray(a, t) for a, t in ((planes13, np.uint32), (scales13, np.uint8), (row13, np.float32),
                                                             (planes2, np.uint32), (scales2, np.uint8), (row2, np.float32))]
        self.levels = [_levels(codebook), _levels(fc2_codebook)]
        self.struct = Experts(*[_p(a) for a in self.arrays], _p(self.levels[0]), _p(self.levels[1]), self.arrays[2].shape[0], base, hidden, inter,
                              int(gated))


def moe_layer(experts: HostExperts, x_bits: np.ndarray, ids: np.ndarray, weights: np.ndarray, shared: HostExperts | None = None,
              gate_vec: np.ndarray | None = None):
    """x_bits uint16 [m, hidden] (BF16 bit patterns) -> (uint16 [m, hidden], distinct experts run)."""
    x_bits = np.ascontiguousarray(x_bits, np.uint16)
    ids = np.ascontiguousarray(ids, np.int32)
    weights = np.ascontiguousarray(weights, np.float32)
    m, topk = ids.shape
    out = np.empty_like(x_bits)
    gv = None if gate_vec is None else np.ascontiguousarray(gate_vec, np.float32)
    d = lib().w3o_moe_layer(C.byref(experts.struct), C.byref(shared.struct) if shared else None, _p(gv) if gv is not None else None, _p(x_bits),
                            _p(ids), _p(weights), m, topk, _p(out))
    return out, d


def last_unpack_seconds() -> float:
    """Seconds the last moe_layer call spent unpacking weights (the rest is matmuls, activation and combine)."""
    return float(lib().w3o_last_unpack_seconds())


def linear(w3: dict, x_bits: np.ndarray) -> np.ndarray:
    planes, scales = np.ascontiguousarray(w3["planes"], np.uint32), np.ascontiguousarray(w3["scales"], np.uint8)
    row, lv = np.ascontiguousarray(w3["row_scale"], np.float32), _levels(w3["codebook"])
    x_bits = np.ascontiguousarray(x_bits, np.uint16)
    n, k = w3["out_features"], w3["in_features"]
    y = np.empty((x_bits.shape[0], n), np.uint16)
    lib().w3o_linear(_p(planes), _p(scales), _p(row), _p(lv), n, k, planes.shape[2], _p(x_bits), x_bits.shape[0], _p(y))
    return y


def threads() -> int:
    return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
