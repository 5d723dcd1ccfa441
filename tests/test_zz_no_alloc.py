"""hb_w3_moe_layer_static (the entry point that allocates nothing: its workspace is a device array of the library) gives
hb_w3_moe_layer's bits, on two calls in a row, the second with a smaller input; a call beyond the array is refused."""
import ctypes as C

import pytest
import torch

from tests.util import random_experts

pytestmark = pytest.mark.gpu


def _both(ex, sh, gate, x, ids, weights):
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    lib = _lib.lib()
    m, k = ids.shape
    st, ss = w3_moe._struct(ex), w3_moe._struct(sh)
    need = lib.hb_w3_moe_workspace_bytes(m, k, C.byref(st), 1)
    assert 0 < need <= 8 << 20
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    want = torch.zeros((m, ex.shape2[0]), dtype=torch.bfloat16, device="cuda")
    got = torch.zeros_like(want)
    _lib.check(lib.hb_w3_moe_layer(C.byref(st), C.byref(ss), _lib.ptr(gate), _lib.ptr(x), _lib.ptr(ids), _lib.ptr(weights), m, k, _lib.ptr(want),
                                   _lib.ptr(ws), need, _lib.stream()), "moe_layer")
    _lib.check(lib.hb_w3_moe_layer_static(C.byref(st), C.byref(ss), _lib.ptr(gate), _lib.ptr(x), _lib.ptr(ids), _lib.ptr(weights), m, k,
                                          _lib.ptr(got), _lib.stream()), "moe_layer_static")
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_entry_point_matches_the_workspace_one():
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, _ = random_experts(16, 256, 128, True, 51)
    sh, _ = random_experts(1, 256, 128, True, 52)
    w3_moe.tile(ex), w3_moe.tile(sh)
    g = torch.Generator().manual_seed(53)
    gate = (torch.randn(256, generator=g) * 0.05).cuda()
    for m in (40, 3):  # the second call is smaller: what the first left in the array beyond it must not matter
        x = torch.randn(m, 256, generator=g).bfloat16().cuda()
        ids = torch.stack([torch.randperm(16, generator=g)[:4] for _ in range(m)]).to(torch.int32).cuda()
        weights = torch.rand(m, 4, generator=g).cuda()
        got, want = _both(ex, sh, gate, x, ids, weights)
        assert want.float().abs().max() > 0 and torch.equal(got, want), m
    # beyond the array: refused with its own code, nothing enqueued
    m = 4096
    x = torch.zeros(m, 256, dtype=torch.bfloat16, device="cuda")
    ids = torch.zeros(m, 4, dtype=torch.int32, device="cuda")
    weights = torch.zeros(m, 4, device="cuda")
    out = torch.zeros(m, 256, dtype=torch.bfloat16, device="cuda")
    st, ss = w3_moe._struct(ex), w3_moe._struct(sh)
    lib = _lib.lib()
    assert lib.hb_w3_moe_workspace_bytes(m, 4, C.byref(st), 1) > 8 << 20
    code = lib.hb_w3_moe_layer_static(C.byref(st), C.byref(ss), None, _lib.ptr(x), _lib.ptr(ids), _lib.ptr(weights), m, 4, _lib.ptr(out), _lib.stream())
    assert code == _lib.HB_ESCRATCH and b"scratch" in lib.hb_error_string(code)
    with pytest.raises(ValueError):
        _lib.check(code, "moe_layer_static")
