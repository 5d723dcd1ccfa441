"""ctypes binding of libhibana_hip.so (the C ABI declared in include/hibana_hip.h)."""
from __future__ import annotations

import ctypes as C
from functools import lru_cache
from pathlib import Path

import torch

LIBRARY = Path(__file__).resolve().parent / "libhibana_hip.so"

HB_OK, HB_EINVAL, HB_ENULL, HB_EWORKSPACE, HB_ELAUNCH, HB_ESCRATCH = 0, -1, -2, -3, -4, -5


class HbW3Experts(C.Structure):
    _fields_ = [("fc1", C.c_void_p), ("fc1_rows", C.c_void_p), ("fc2", C.c_void_p), ("fc2_rows", C.c_void_p),
                ("fc1_lut", C.c_int64), ("fc2_lut", C.c_int64), ("experts", C.c_int), ("base", C.c_int),
                ("hidden", C.c_int), ("inter", C.c_int), ("hidden_out", C.c_int), ("gated", C.c_int)]


class HbNvfp4Experts(C.Structure):
    _fields_ = [("fc1", C.c_void_p), ("fc1_scale2", C.c_void_p), ("fc2", C.c_void_p), ("fc2_scale2", C.c_void_p),
                ("experts", C.c_int), ("base", C.c_int), ("hidden", C.c_int), ("inter", C.c_int),
                ("hidden_out", C.c_int), ("gated", C.c_int)]


class HbLatentWeights(C.Structure):
    _fields_ = [("gate_fc1", C.c_void_p), ("bias", C.c_void_p), ("fc2", C.c_void_p), ("routed", C.POINTER(HbNvfp4Experts)),
                ("shared_up", C.c_void_p), ("shared_down", C.c_void_p), ("shared_up_scale", C.c_float), ("shared_down_scale", C.c_float),
                ("experts_total", C.c_int), ("latent", C.c_int), ("hidden", C.c_int), ("shared_inter", C.c_int)]


_P, _I, _L, _Z, _F = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
_LW = C.POINTER(HbLatentWeights)
_EX = C.POINTER(HbW3Experts)
_EX4 = C.POINTER(HbNvfp4Experts)
# name -> (restype, argtypes): every symbol include/hibana_hip.h declares
SIGNATURES = {
    "hb_version": (_I, []),
    "hb_error_string": (C.c_char_p, [_I]),
    "hb_tune": (_I, [C.c_char_p, _I]),
    "hb_debug_events": (_I, [_P, _I]),
    "hb_debug_trace": (_I, [_P, _L]),
    "hb_debug_stream_read": (_I, [_P, _Z, _P, _P]),
    "hb_debug_ring_skeleton": (_I, [_P, _Z, _P, _I, _P, _Z, _P, _Z, _P, _Z, _P]),
    "hb_debug_workspace_layout": (_I, [_I, _I, _EX, _I, C.POINTER(C.c_int64)]),
    "hb_workspace_reset": (_I, [_P, _Z, _P]),
    "hb_workspace_status": (_I, [_P, C.POINTER(C.c_int32), _I, _P]),
    "hb_debug_mfma_rate": (_L, [_I, _I, _P, _P]),
    "hb_w3_tiled_bytes": (_Z, [_L, _I, _I]),
    "hb_w3_repack": (_I, [_P, _P, _L, _I, _I, _I, _P, _P]),
    "hb_w3_pack_codes": (_I, [_P, _P, _L, _I, _I, _P, _P, _P]),
    "hb_w3_unpack": (_I, [_P, _L, _I, _I, _P, _P, _P]),
    "hb_w3_unpack_planes": (_I, [_P, _P, _L, _I, _I, _P, _P, _P]),
    "hb_w3_dequant": (_I, [_P, _P, _L, _L, _I, _I, _P, _P]),
    "hb_w3_gemm": (_I, [_P, _I, _P, _P, _L, _I, _I, _I, _P, _P]),
    "hb_w3_quant_groups": (_I, [_P, _L, _I, _P, _P, _P]),
    "hb_w3_quant_rows": (_I, [_P, _L, _I, _P, _P, _P]),
    "hb_w3_gemm_e4m3": (_I, [_P, _P, _I, _P, _P, _L, _I, _I, _I, _P, _P]),
    "hb_w3_moe_workspace_bytes": (_Z, [_I, _I, _EX, _I]),
    "hb_w3_moe": (_I, [_EX, _P, _P, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "hb_w3_moe_layer": (_I, [_EX, _EX, _P, _P, _P, _P, _I, _I, _P, _P, _Z, _P]),
    "hb_w3_moe_layer_static": (_I, [_EX, _EX, _P, _P, _P, _P, _I, _I, _P, _P]),
    "hb_w3_moe_layer_e4m3": (_I, [_EX, _EX, _P, _P, _P, _P, _I, _I, _P, _P, _Z, _P]),
    "hb_w3_moe_layer_logits": (_I, [_EX, _EX, _P, _P, _P, _I, _I, _I, _P, _P, _P, _P, _Z, _P]),
    "hb_w3_moe_layer_budget": (_I, [_EX, _EX, _P, _P, _P, _I, _I, _I, _I, _I, _P, _I, _I, _I, _P, _P, _P, _P, _Z, _P]),
    "hb_w3_moe_layer_logits_e4m3": (_I, [_EX, _EX, _P, _P, _P, _I, _I, _I, _P, _P, _P, _P, _Z, _P]),
    "hb_moe_combine_pairs": (_I, [_P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P]),
    "hb_silu_and_mul": (_I, [_P, _L, _I, _I, _P, _P]),
    "hb_silu_mul": (_I, [_P, _L, _I, _I, _P, _P]),
    "hb_relu2": (_I, [_P, _L, _I, _L, _P]),
    "hb_silu_mul_quant_groups": (_I, [_P, _L, _I, _I, _I, _P, _P, _P]),
    "hb_route_softmax_topk": (_I, [_P, _I, _I, _I, _P, _I, _I, _P, _P, _P]),
    "hb_route_budget_workspace_bytes": (_L, [_I]),
    "hb_route_budget": (_I, [_P, _I, _I, _I, _I, _I, _P, _I, _I, _I, _I, _P, _L, _P, _P, _P]),
    "hb_route_budget_sigmoid_workspace_bytes": (_L, [_I, _I]),
    "hb_route_budget_sigmoid": (_I, [_P, _L, _P, _I, _I, _I, _I, _I, _I, _P, _I, _I, _I, _I, _P, _L, _P, _P, _P, _P]),
    "hb_route_sigmoid_topk": (_I, [_P, _L, _P, _I, _I, _I, _I, _P, _I, _I, _P, _P, _P, _P]),
    "hb_nvfp4_tiled_bytes": (_Z, [_L, _I]),
    "hb_nvfp4_repack": (_I, [_P, _P, _I, _L, _I, _P, _P]),
    "hb_nvfp4_dequant": (_I, [_P, _F, _L, _I, _P, _P]),
    "hb_nvfp4_gemm": (_I, [_P, _I, _P, _F, _I, _I, _I, _P, _P]),
    "hb_nvfp4_gemm_workspace_bytes": (_Z, [_I, _I, _I]),
    "hb_nvfp4_gemm_ws": (_I, [_P, _I, _P, _F, _I, _I, _I, _P, _P, _Z, _P]),
    "hb_nvfp4_moe_workspace_bytes": (_Z, [_I, _I, _EX4]),
    "hb_nvfp4_moe": (_I, [_EX4, _P, _P, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "hb_latent_workspace_bytes": (_Z, [_LW, _I, _I]),
    "hb_latent_router": (_I, [_LW, _P, _I, _I, _P, _I, _I, _I, _P, _P, _P, _P, _P, _Z, _P]),
    "hb_latent_block": (_I, [_LW, _P, _P, _P, _P, _I, _I, _I, _P, _P, _Z, _P]),
    "hb_latent_shared_up": (_I, [_LW, _P, _I, _I, _P, _Z, _P]),
    "hb_latent_out": (_I, [_LW, _P, _I, _I, _P, _P, _Z, _P]),
}


@lru_cache(maxsize=1)
def lib() -> C.CDLL:
    """The loaded library; raises if it has not been built (python -m hibana_amd.build)."""
    if not LIBRARY.exists():
        raise RuntimeError(f"{LIBRARY} is missing: build it with `python -m hibana_amd.build` (hipcc, gfx950); there is no fallback path")
    handle = C.CDLL(str(LIBRARY))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype, fn.argtypes = restype, argtypes
    return handle


def check(code: int, what: str) -> None:
    """Map a status code to the reference's error behaviour: ValueError for calls the kernels do not take,
    RuntimeError for the rest."""
    if code == HB_OK:
        return
    text = lib().hb_error_string(code).decode()
    if code in (HB_EINVAL, HB_ESCRATCH):
        raise ValueError(f"{what}: {text}")
    raise RuntimeError(f"{what}: {text}")


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


WORKSPACE_ZERO_BYTES = 1 << 20
_workspaces: dict[tuple[int, int, str], torch.Tensor] = {}


def workspace(device: torch.device, need: int, kind: str = "moe") -> torch.Tensor:
    """A workspace of at least `need` bytes for a call on the current stream of `device`: one buffer a (device, stream,
    kind of call), kept between calls and grown when a call needs more, handed over with its head zero as the library
    asks (its arrival counters and fault word; every call leaves them zero again). Calls on one stream follow one
    another, so they can share it; calls on different streams get different buffers and share nothing. `kind` keeps
    apart calls that are in progress together on one stream (a latent block's workspace lives across several calls,
    among them a routed one)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (index, torch.cuda.current_stream(device).cuda_stream, kind)
    have = _workspaces.get(key)
    if have is None or have.numel() < need:
        have = torch.empty(max(need, 4096), dtype=torch.uint8, device=device)
        have[:WORKSPACE_ZERO_BYTES].zero_()  # a fill kernel on the current stream (capturable); the rest needs no start value
        _workspaces[key] = have
    return have


def workspace_status(ws: torch.Tensor | None) -> int:
    """The fault word of a workspace (None: the library's own scratch) once the current stream's work is done: 0, or
    HB_FAULT_* bits."""
    word = C.c_int32(-1)
    check(lib().hb_workspace_status(ptr(ws), C.byref(word), 1, stream()), "workspace_status")
    return word.value


def workspace_reset(ws: torch.Tensor | None) -> None:
    check(lib().hb_workspace_reset(ptr(ws), 0 if ws is None else ws.numel(), stream()), "workspace_reset")


def need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("hibana_amd kernels run on the GPU only: got a CPU tensor (there is no CPU fallback)")
