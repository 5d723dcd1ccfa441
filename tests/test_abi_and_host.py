"""CPU checks: the C ABI library loads and exports every symbol include/hibana_hip.h declares, argument validation
that needs no GPU, and the host-side logic that mirrors the reference interface."""
import ctypes as C
import os
import re

import pytest
import torch

from hibana_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "hibana_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hb_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 20
    handle = C.CDLL(str(_lib.LIBRARY))
    for name in names:
        assert hasattr(handle, name), name
    assert sorted(_lib.SIGNATURES) == names  # the Python binding covers the header, nothing more, nothing less


def test_a_build_without_debug_hooks_exports_none_of_them():
    """-DHB_NO_DEBUG_HOOKS: hb_tune and every hb_debug_* are gone (a serving process cannot race on them), the rest of
    the header is there; the default build has all of it. Host-only compiles: no device code is built here."""
    from hibana_amd import build
    hooks = {n for n in _declared() if n == "hb_tune" or n.startswith("hb_debug_")}
    assert len(hooks) >= 7
    assert build.host_symbols(no_debug_hooks=True) == set(_declared()) - hooks
    assert build.host_symbols(no_debug_hooks=False) == set(_declared())


def test_validation_without_a_gpu():
    lib = _lib.lib()
    assert lib.hb_version() >= 1000
    assert lib.hb_error_string(0) == b"ok" and b"workspace" in lib.hb_error_string(_lib.HB_EWORKSPACE)
    assert lib.hb_w3_tiled_bytes(1024, 2048, 3) == 1024 * 2048 * 3 // 8 + 1024 * 2048 // 32
    assert lib.hb_w3_tiled_bytes(1024, 2048, 2) == 1024 * 2048 * 2 // 8 + 1024 * 2048 // 32  # a two-bit matrix at its own density
    assert lib.hb_w3_tiled_bytes(96, 2048, 3) == 0 and lib.hb_w3_tiled_bytes(128, 100, 3) == 0 and lib.hb_w3_tiled_bytes(128, 128, 4) == 0
    assert lib.hb_nvfp4_tiled_bytes(128, 256) == 128 * 256 // 2 + 128 * 256 // 16
    assert lib.hb_nvfp4_tiled_bytes(128, 64) == 0
    assert lib.hb_tune(b"no_such_knob", 1) == _lib.HB_EINVAL and lib.hb_tune(b"w3_ksplit", 17) == _lib.HB_EINVAL
    assert lib.hb_tune(b"w3_ksplit", 4) == 0 and lib.hb_tune(b"w3_ksplit", 0) == 0
    assert lib.hb_w3_repack(None, None, 128, 128, 3, 3, None, None) == _lib.HB_ENULL
    assert lib.hb_w3_repack(256, 256, 128, 128, 3, 2, 256, None) == _lib.HB_EINVAL  # codes are widened, never narrowed
    assert lib.hb_w3_gemm(None, 1, None, None, 0, 128, 128, 3, None, None) == _lib.HB_ENULL
    assert lib.hb_nvfp4_gemm(None, 1, None, 1.0, 128, 128, 0, None, None) == _lib.HB_ENULL
    assert lib.hb_w3_moe_workspace_bytes(4, 2, None, 0) == 0
    ex = _lib.HbW3Experts(256, 256, 256, 256, 0, 0, 8, 0, 256, 128, 256, 1)  # (no call below reads through the pointers)
    need = lib.hb_w3_moe_workspace_bytes(32, 10, C.byref(ex), 1)
    assert need >= (320 + 32) * (128 * 2 + 256 * 4)
    bad = _lib.HbW3Experts(256, 256, 256, 256, 0, 0, 8, 0, 200, 128, 256, 1)  # hidden not a multiple of 128
    assert lib.hb_w3_moe_workspace_bytes(32, 10, C.byref(bad), 1) == 0
    assert lib.hb_w3_moe(C.byref(bad), None, None, None, 1, 1, 0, None, None, 0, None) == _lib.HB_EINVAL
    # pointers off the boundaries the kernels' vector accesses need are refused before anything is launched
    odd = _lib.HbW3Experts(264, 256, 256, 256, 0, 0, 8, 0, 256, 128, 256, 1)  # fc1 on an 8-byte boundary only
    assert lib.hb_w3_moe_workspace_bytes(32, 10, C.byref(odd), 1) == 0
    assert lib.hb_w3_gemm(258, 1, 256, 256, 0, 128, 128, 3, 256, None) == _lib.HB_EINVAL  # x on a 2-byte boundary
    assert lib.hb_w3_gemm(256, 1, 256, 256, 0, 128, 128, 4, 256, None) == _lib.HB_EINVAL  # tiles of two or three bits
    assert lib.hb_w3_moe(C.byref(ex), 256, 256, 256, 1, 1, 0, 256, 264, 1 << 30, None) == _lib.HB_EINVAL  # workspace on 8
    assert lib.hb_nvfp4_gemm(256, 1, 260, 1.0, 128, 128, 0, 256, None) == _lib.HB_EINVAL  # tile layout on 4
    # the dense product with a workspace: sizes only (no launch without a GPU)
    assert lib.hb_nvfp4_gemm_workspace_bytes(8, 25600, 5120) == 0 and lib.hb_nvfp4_gemm_workspace_bytes(2048, 25600, 5120) == 0
    # the header words and 100 arrival counters (a multiple of 256 bytes), then 100 tiles x 4 shares of K x 4 wavefronts x 4 row tiles x 4 x 64 lanes x 16 B
    assert lib.hb_nvfp4_gemm_workspace_bytes(64, 25600, 5120) == 512 + 100 * 4 * 4 * 4 * 4 * 64 * 16
    assert lib.hb_nvfp4_gemm_workspace_bytes(64, 100, 5120) == 0
    assert lib.hb_nvfp4_gemm_ws(None, 64, None, 1.0, 128, 128, 0, None, None, 0, None) == _lib.HB_ENULL
    assert lib.hb_relu2(None, 1, 2, 2, None) == _lib.HB_ENULL and lib.hb_relu2(256, 1, 3, 4, None) == _lib.HB_EINVAL
    assert lib.hb_silu_mul(None, 1, 2, 0, None, None) == _lib.HB_ENULL and lib.hb_silu_mul(256, 1, 3, 0, 256, None) == _lib.HB_EINVAL
    # budgeted routing: 20 candidates a row, whole requests, a workspace for the candidates
    assert lib.hb_route_budget_workspace_bytes(12) == 12 * 20 * 8 and lib.hb_route_budget_workspace_bytes(0) == 0
    assert lib.hb_route_budget(None, 12, 512, 10, 4, 64, None, 1, 0, 0, 0, 256, 1920, 256, 256, None) == _lib.HB_ENULL
    for r, e, k, keep, steps in [(12, 19, 10, 4, 1), (12, 1025, 10, 4, 1), (12, 512, 21, 4, 1), (12, 512, 10, 21, 1), (12, 512, 10, 4, 5)]:
        assert lib.hb_route_budget(256, r, e, k, keep, 64, None, steps, 0, 0, 0, 256, 1920, 256, 256, None) == _lib.HB_EINVAL
    assert lib.hb_route_budget(256, 12, 512, 10, 4, 64, None, 1, 0, 0, 0, 256, 1919, 256, 256, None) == _lib.HB_EWORKSPACE
    assert lib.hb_w3_moe_layer_budget(None, None, None, 256, 256, 512, 4, 10, 4, 64, None, 1, 0, 0, 256, 256, 256, 256, 1 << 20, None) == _lib.HB_ENULL
    assert lib.hb_route_budget_sigmoid_workspace_bytes(12, 22) == 12 * 22 * 12
    assert lib.hb_route_budget_sigmoid(None, 640, 256, 12, 512, 22, 128, 6, 64, None, 1, 1, 0, 0, 256, 3168, 256, 256, 256, None) == _lib.HB_ENULL
    for e, k, keep, fallback, stride in [(512, 33, 6, 0, 640), (1025, 22, 6, 0, 1200), (512, 22, 23, 0, 640), (512, 22, 6, 7, 640), (512, 22, 6, 0, 639)]:
        assert lib.hb_route_budget_sigmoid(256, stride, 256, 12, e, k, 128, keep, 64, None, 1, 1, 0, fallback, 256, 1 << 20, 256, 256, 256, None) == _lib.HB_EINVAL
    assert lib.hb_route_budget_sigmoid(256, 640, 256, 12, 512, 22, 128, 6, 64, None, 1, 1, 0, 0, 256, 3167, 256, 256, 256, None) == _lib.HB_EWORKSPACE
    # the small latent block: shapes and pointers are checked before anything is launched
    nv = _lib.HbNvfp4Experts(256, 256, 256, 256, 8, 0, 256, 128, 256, 0)
    lw = _lib.HbLatentWeights(256, 256, 256, C.pointer(nv), 256, 256, 1.0, 1.0, 8, 256, 512, 640)
    need = lib.hb_latent_workspace_bytes(C.byref(lw), 4, 2)
    assert need >= 4 * (256 + 640 + 512) * 2 and lib.hb_latent_workspace_bytes(C.byref(lw), 17, 2) == 0  # at most sixteen rows
    assert lib.hb_latent_workspace_bytes(None, 4, 2) == 0
    assert lib.hb_latent_router(None, 256, 4, 2, None, 1, 1, -1, 256, 256, 256, 256, 256, need, None) == _lib.HB_ENULL
    assert lib.hb_latent_router(C.byref(lw), 256, 4, 2, None, 1, 1, -1, 256, 256, 256, 256, 256, need - 1, None) == _lib.HB_EWORKSPACE
    assert lib.hb_latent_router(C.byref(lw), 256, 4, 2, None, 1, 1, 9, 256, 256, 256, 256, 256, need, None) == _lib.HB_EINVAL  # pad_id past "no expert"
    assert lib.hb_latent_block(C.byref(lw), 256, 256, 256, 256, 17, 2, 0, 256, 256, need, None) == _lib.HB_EINVAL
    bare = _lib.HbLatentWeights(256, 256, 256, None, None, None, 0.0, 0.0, 8, 256, 512, 0)  # 3-bit experts, no shared expert
    assert lib.hb_latent_block(C.byref(bare), 256, 256, 256, 256, 4, 2, 0, 256, 256, 1 << 20, None) == _lib.HB_ENULL
    assert lib.hb_latent_shared_up(C.byref(bare), 256, 4, 2, 256, 1 << 20, None) == _lib.HB_ENULL
    lopsided = _lib.HbLatentWeights(256, 256, 256, None, 256, None, 1.0, 0.0, 8, 256, 512, 640)  # an up projection without its down
    assert lib.hb_latent_workspace_bytes(C.byref(lopsided), 4, 2) == 0
    with pytest.raises(ValueError):
        _lib.check(_lib.HB_EINVAL, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.HB_ELAUNCH, "x")


def test_host_logic_mirrors_the_reference_interface(monkeypatch):
    from hibana_amd.kernels import ops, w3, w3_moe
    from hibana_amd.weights import modelopt
    from hibana_amd.weights.linear import Linear
    from oracle import layers, nvfp4_format as onv, w3_format as ow3
    assert w3.MAX_ROWS == 128 and w3.GROUP == 32 and w3.CHUNK == 128 and w3.DEFAULT_CODEBOOK == "lloyd"
    assert w3.CODEBOOKS == ow3.CODEBOOKS and w3_moe.EXPERTS == 512 and w3_moe.ORDER_IN_KERNEL == 640 and w3_moe.WIDE_ROWS == 1024
    for name, levels in w3.CODEBOOKS.items():
        assert w3.lut_of(levels) == ow3.lut_of(levels), name
    with pytest.raises(ValueError):
        w3._codebook((-3.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.3))
    with pytest.raises(ValueError):
        w3._codebook((1.0, 0.5, 2.0, 3.0))
    assert w3_moe.fc1_order(128).tolist() == layers.fc1_order(128).tolist()
    assert w3.pair_order(512, 64).tolist() == ow3.pair_order(512, 64).tolist() == modelopt.pair_order(512, 64).tolist()
    s = torch.arange(130 * 6, dtype=torch.float32).reshape(130, 6)
    sw = modelopt.swizzle_block_scales(s)
    assert sw.shape == (256, 8) and (sw.numpy() == onv.swizzle_block_scales(s.numpy())).all()
    assert torch.equal(modelopt.unswizzle_block_scales(sw, 130, 6), s)
    with pytest.raises(RuntimeError):
        ops.silu_and_mul(torch.randn(3, 256).bfloat16())  # a kernel: no CPU path
    with pytest.raises(ValueError):
        ops.silu_and_mul(torch.randn(3, 256))  # not BF16
    monkeypatch.delenv("HIBANA_W3_DECODE", raising=False)
    assert not w3.enabled()
    monkeypatch.setenv("HIBANA_W3_DECODE", "1")
    assert w3.enabled()
    lin = modelopt.Nvfp4Linear(torch.zeros(128, 64, dtype=torch.uint8), torch.zeros(128, 8).to(torch.float8_e4m3fn), torch.tensor(2.0),
                               torch.tensor(4.0), 128, 128)
    assert isinstance(lin, Linear) and lin.global_scale == 8.0 and lin.bytes == 128 * 64 + 128 * 8 and lin.w3 is None
    assert not ops.w3_decode(lin, 4)
    lin.w3 = object()
    assert ops.w3_decode(lin, 4) and not ops.w3_decode(lin, 129) and not ops.w3_decode(lin, 4, rows=2)
    # the ops have no CPU path: they raise rather than fall back
    with pytest.raises(RuntimeError):
        modelopt.unpack_fp4(torch.zeros(64, 64, dtype=torch.uint8), torch.zeros(64, 8, dtype=torch.uint8))
    with pytest.raises(RuntimeError):
        ops.route_topk(torch.zeros(2, 8), 2)
    with pytest.raises(RuntimeError):
        w3.pack_codes(torch.zeros(128, 128, dtype=torch.uint8), torch.zeros(128, 4).to(torch.float8_e4m3fn), torch.ones(128))
    with pytest.raises(ValueError):
        w3.pack_codes(torch.full((128, 128), 9, dtype=torch.uint8), torch.zeros(128, 4).to(torch.float8_e4m3fn), torch.ones(128))
    with pytest.raises(ValueError):
        w3.quant_rows(torch.zeros(1, 32))  # not BF16
    with pytest.raises(RuntimeError):
        w3.quant_rows(torch.zeros(1, 32, dtype=torch.bfloat16))  # no CPU path
    with pytest.raises(ValueError):
        w3.quant_groups(torch.zeros(1, 32))  # not BF16
    with pytest.raises(RuntimeError):
        w3.quant_groups(torch.zeros(1, 32, dtype=torch.bfloat16))  # no CPU path


def test_budgeted_selection_settings_and_which_forwards_take_it(monkeypatch):
    """`MoeLayer`'s keep / budget / per_request as the reference resolves them, the guarantee by the call's shape (the
    values of tests/unit/test_moe_selection.py:150-171 of the reference), and the routing call each forward makes."""
    from types import SimpleNamespace

    from hibana_amd.model import flashnext_moe
    from hibana_amd.model.flashnext_moe import MoeLayer

    def layer(keep=4, budget=64, per_request=12, topk=10):
        it = MoeLayer.__new__(MoeLayer)
        it.router = torch.zeros(512, 32, dtype=torch.bfloat16)
        it.topk = topk
        it.keep = keep if keep < topk else 0
        it.budget = budget if it.keep else 0
        it.per_request = per_request
        return it

    assert [layer(keep=k).keep for k in (0, 1, 4, 9, 10, 12)] == [0, 1, 4, 9, 0, 0]
    assert (layer(keep=0).budget, layer(keep=10).budget, layer(keep=4).budget) == (0, 0, 64)
    shapes = [(1, 1), (1, 5), (1, 8), (4, 5), (1, 9), (2, 9), (8, 5), (16, 4), (64, 4), (128, 1)]  # requests x rows a request
    assert [layer().guarantee(r * s, s) for r, s in shapes] == [4, 4, 4, 4, 3, 2, 3, 2, 2, 2]
    assert layer(keep=1).guarantee(256, 4) == 1 and layer(per_request=0).guarantee(5, 5) == 4
    calls = []
    stub = SimpleNamespace(
        route_budget=lambda logits, k, keep, budget, slots=None, steps=1, repeat=False, per_request=0, min_cap=0:
            calls.append(("budget", k, keep, budget, slots, steps, repeat, per_request, min_cap)) or "budget",
        route_topk=lambda logits, k, slots=None, steps=1, repeat=False: calls.append(("topk", k, slots, steps)) or f"top{k}")
    monkeypatch.setattr(flashnext_moe, "ops", stub)
    x = torch.zeros(20, 32, dtype=torch.bfloat16)
    verify_slots, decode_slots = torch.tensor([3, 1, 4, 0], dtype=torch.int32), torch.tensor([7] * 13 + [0] * 7, dtype=torch.int32)
    assert layer().route(x, SimpleNamespace(mode="verify", seq_slots=verify_slots, verify_steps=5)) == "budget"
    assert layer().route(x, SimpleNamespace(mode="decode", slots=decode_slots)) == "budget"
    assert calls == [("budget", 10, 4, 64, verify_slots, 5, False, 12, 16), ("budget", 10, 4, 64, decode_slots, 1, False, 12, 16)]
    del calls[:]
    assert layer(budget=0).route(x, SimpleNamespace(mode="decode", slots=decode_slots)) == "top4"  # keep alone: each token's top 4
    assert layer().route(x, SimpleNamespace(mode="prefill")) == "top10"
    assert layer(keep=0, budget=0).route(x, SimpleNamespace(mode="decode", slots=decode_slots)) == "top10"
    assert [c[:2] for c in calls] == [("topk", 4), ("topk", 10), ("topk", 10)] and calls[2][2] is decode_slots


def test_latent_block_budget_settings_and_fallback():
    """`NemotronMoe`'s keep / budget / per_request and the guarantee it falls back to (cap / rows within
    [SHARE_MIN, keep), hibana/model/nemotron/moe.py:464-474), worked out by hand from the rule."""
    from types import SimpleNamespace

    from hibana_amd.model.nemotron_moe import NemotronMoe

    def block(keep, budget, per_request, topk=22):
        it = NemotronMoe.__new__(NemotronMoe)
        it.topk = topk
        it.keep = keep if keep < topk else 0
        it.budget = budget if it.keep else 0
        it.per_request = per_request
        return it

    assert [block(k, 64, 0).keep for k in (0, 6, 21, 22, 30)] == [0, 6, 21, 0, 0] and block(22, 64, 0).budget == 0
    b = block(12, 64, 12)
    assert b.fallback(4, 1) == 0     # cap min(64, 48): 48 // 4 = 12, the floor itself
    assert b.fallback(16, 1) == 8    # cap 64: 64 // 16 = 4, raised to SHARE_MIN
    assert b.fallback(6, 1) == 10    # cap 64: 64 // 6 = 10
    assert b.fallback(16, 8) == 8    # two requests: cap 24, 24 // 16 = 1, raised to SHARE_MIN
    assert block(12, 0, 12).fallback(16, 1) == 0 and block(6, 64, 0).fallback(16, 1) == 0  # no cap; SHARE_MIN is the floor itself
    assert b.selects(SimpleNamespace(mode="decode")) and b.selects(SimpleNamespace(mode="verify"))
    assert not b.selects(SimpleNamespace(mode="prefill")) and not b.selects(None) and not block(0, 64, 12).selects(SimpleNamespace(mode="decode"))


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0 and "ONE GPU" in run.stderr
