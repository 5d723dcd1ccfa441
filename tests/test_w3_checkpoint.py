"""The calibrated 3-bit checkpoint format: round trips, identity checks and expert ranges on the CPU (as
tests/unit/test_w3_calibration.py:38-53 and tests/unit/test_w3_moe_pack.py:56-66 of the reference do), the load-time
repack on the GPU."""
import json
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import w3_format as ow3
from tests.util import random_w3, to_device_w3


def _write(tmp_path, entries, revision="rev"):
    (tmp_path / "manifest.json").write_text(json.dumps({"format": 1, "target_revision": revision, "weights": entries}))


def _same(a, b):
    return all(torch.equal(getattr(a, f).view(torch.uint8), getattr(b, f).view(torch.uint8)) for f in ("planes", "scales", "row_scale"))


def test_round_trip_and_identity_checks(tmp_path):
    from hibana_amd.weights.w3_checkpoint import CalibratedWeights, save_weight
    weight = to_device_w3(random_w3(128, 256, 1, "zero8")[0], "cpu")
    entry = save_weight(tmp_path / "layer.safetensors", weight)
    assert entry["out_features"] == 128 and entry["in_features"] == 256 and entry["codebook"] == list(ow3.CODEBOOKS["zero8"])
    _write(tmp_path, {"layer": entry})
    linear = SimpleNamespace(weight=torch.zeros(1), out_features=128, in_features=256)
    ck = CalibratedWeights(tmp_path, "rev")
    loaded = ck.load("layer", linear)
    assert _same(loaded, weight) and loaded.codebook == weight.codebook and loaded.lut == weight.lut and loaded.tiled is None
    assert len(ck.identity) == 64 and ck.paths(["layer"])[0] == (tmp_path / "layer.safetensors", entry["sha256"])
    with pytest.raises(ValueError, match="shape"):
        ck.load("layer", SimpleNamespace(weight=torch.zeros(1), out_features=256, in_features=256))
    (tmp_path / "layer.safetensors").write_bytes(b"corrupt")
    with pytest.raises(ValueError, match="checksum"):
        CalibratedWeights(tmp_path, "rev").load("layer", linear)
    with pytest.raises(ValueError, match="revision"):
        CalibratedWeights(tmp_path, "another")
    _write(tmp_path, {"layer": dict(entry, file="../layer.safetensors")})
    with pytest.raises(ValueError, match="inside"):
        CalibratedWeights(tmp_path, "rev").load("layer", linear)


def test_wrong_tensor_shapes_are_rejected(tmp_path):
    from hibana_amd.weights.w3_checkpoint import CalibratedWeights, save_weight
    weight = to_device_w3(random_w3(128, 128, 2)[0], "cpu")
    entry = save_weight(tmp_path / "w.safetensors", weight)
    _write(tmp_path, {"w": dict(entry, in_features=256)})
    with pytest.raises(ValueError, match="invalid"):
        CalibratedWeights(tmp_path, "rev").load("w", SimpleNamespace(weight=torch.zeros(1), out_features=128, in_features=256))


def test_paired_rows_are_interleaved_on_load(tmp_path):
    from hibana_amd.kernels import w3
    from hibana_amd.weights.w3_checkpoint import CalibratedWeights, save_weight
    packed = random_w3(256, 128, 3)[0]
    weight = to_device_w3(packed, "cpu")
    _write(tmp_path, {"mlp": save_weight(tmp_path / "mlp.safetensors", weight)})
    linear = SimpleNamespace(weight=torch.zeros(1), out_features=256, in_features=128, pairs=32)
    loaded = CalibratedWeights(tmp_path, "rev").load("mlp", linear)
    want = ow3.interleave_rows(packed, 32)
    assert np.array_equal(loaded.planes.view(torch.int32).numpy().view(np.uint32), want["planes"])
    assert np.array_equal(loaded.scales.numpy(), want["scales"]) and np.array_equal(loaded.row_scale.numpy(), want["row_scale"])
    assert _same(loaded, w3.interleave_rows(weight, 32))


def _expert_checkpoint(tmp_path, e, hidden, inter):
    from hibana_amd.kernels import w3_moe
    from hibana_amd.weights.w3_checkpoint import save_weight
    from tests.util import random_experts
    ex, per = random_experts(e, hidden, inter, True, 7, device="cpu")
    entries = {f"layers.3.experts.{key}": save_weight(tmp_path / f"layers.3.experts.{key}.safetensors", ex.stacked(key == "w13"))
               for key in ("w13", "w2")}
    _write(tmp_path, entries, "r")
    return ex, per


def test_expert_entries_round_trip_and_ranges(tmp_path):
    from hibana_amd.weights.w3_checkpoint import CalibratedWeights
    e, hidden, inter = 4, 128, 128
    ex, _ = _expert_checkpoint(tmp_path, e, hidden, inter)
    ck = CalibratedWeights(tmp_path, "r")
    assert ck.expert_layers() == {3} and ck.expert_names(3) == ["layers.3.experts.w13", "layers.3.experts.w2"]
    back = ck.load_experts(3, e, inter, hidden, torch.device("cpu"))
    for name in ("planes13", "scales13", "row13", "planes2", "scales2", "row2"):
        assert torch.equal(getattr(back, name).view(torch.uint8), getattr(ex, name).view(torch.uint8)), name
    assert back.codebook == ex.codebook and back.lut == ex.lut and back.base == 0 and back.tiled13 is None
    part = ck.load_experts(3, e, inter, hidden, torch.device("cpu"), lo=1, hi=3)
    assert part.experts == 2 and part.base == 1
    for name in ("planes13", "scales13", "row13", "planes2", "scales2", "row2"):
        assert torch.equal(getattr(part, name).view(torch.uint8), getattr(ex, name)[1:3].view(torch.uint8)), name


@pytest.mark.gpu
def test_loading_on_the_gpu_repacks_once_and_serves(tmp_path):
    from hibana_amd.kernels import w3, w3_moe
    from hibana_amd.weights.w3_checkpoint import CalibratedWeights, save_weight
    from oracle import layers
    from tests.util import MAX_REL, NORM_REL, errors, oracle_expert_getter
    packed = random_w3(128, 256, 11)[0]
    _write(tmp_path, {"lin": save_weight(tmp_path / "lin.safetensors", to_device_w3(packed, "cpu"))}, "r")
    linear = SimpleNamespace(weight=torch.zeros(1).cuda(), out_features=128, in_features=256)
    loaded = CalibratedWeights(tmp_path, "r").load("lin", linear)
    assert loaded.planes is None and loaded.scales is None and loaded.tiled is not None  # one copy, in the kernels' layout
    assert np.array_equal(w3.dequantize(loaded).cpu().numpy().view(np.uint32), ow3.dequantize(packed).view(np.uint32))
    x = torch.randn(3, 256, generator=torch.Generator().manual_seed(0)).bfloat16()
    mx, nr = errors(w3.w3_linear(x.cuda(), loaded), layers.dense_ref(x, ow3.dequantize(packed)))
    assert mx < MAX_REL and nr < NORM_REL

    e, hidden, inter = 4, 128, 128
    sub = tmp_path / "experts"
    sub.mkdir()
    _, per = _expert_checkpoint(sub, e, hidden, inter)
    ex = CalibratedWeights(sub, "r").load_experts(3, e, inter, hidden, torch.device("cuda"), lo=1, hi=4)
    assert ex.planes13 is None and ex.tiled13 is not None and ex.base == 1 and ex.experts == 3
    ids = torch.tensor([[1, 3], [0, 2], [3, 1]], dtype=torch.int32)  # expert 0 is not held here: its pair adds nothing
    wt = torch.tensor([[0.5, 0.5], [0.25, 0.75], [0.9, 0.1]])
    got = w3_moe.w3_moe(ex, x[:, :hidden].contiguous().cuda(), ids.cuda(), wt.cuda())
    get = oracle_expert_getter(per, True, inter)
    want = layers.moe_layer_ref(x[:, :hidden].contiguous(), ids.numpy(), wt, lambda i: get(i + 1), True, e_lo=1, e_n=3)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
