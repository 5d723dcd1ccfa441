"""Every served op is capturable in a HIP graph and its replays give the eager call's bits: no host synchronization, no
host-side decision on device data on the call path (the reference's convention for its kernels; replay-bitwise as
tests/gpu/test_w3_calibration.py:23-45 of the reference). Each graph is replayed several times with eager work and
synchronizations in between, its output cleared before every replay."""
import numpy as np
import pytest
import torch

from oracle import nvfp4_format as onv
from tests.test_gpu_nvfp4_moe import _experts, _stack
from tests.util import random_w3, to_device_w3

pytestmark = pytest.mark.gpu


def _replays_equal_eager(call, replays: int = 3):
    eager = call().clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = call()
    for i in range(replays):
        captured.zero_()
        scratch = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), i
        del scratch
    return eager


def _nvfp4_linear(n, k, seed):
    from hibana_amd.weights import modelopt
    (w, s, g), = [_stack(1, n, k, seed)]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    return modelopt.Nvfp4Linear(dev(w[0]), dev(onv.swizzle_block_scales(s[0])).view(torch.float8_e4m3fn), torch.tensor(float(g[0])).cuda(),
                                torch.tensor(1.0).cuda(), n, k).tile()  # tile(): the load-time step that reads the global scale once


@pytest.mark.parametrize("m", [1, 8, 40, 200])
def test_nvfp4_linear_is_capturable(m):
    from hibana_amd.kernels import ops
    lin = _nvfp4_linear(512, 384, 3)
    x = torch.randn(m, 384, generator=torch.Generator().manual_seed(m)).bfloat16().cuda()
    y = _replays_equal_eager(lambda: ops.nvfp4_linear(x, lin))
    assert y.float().abs().max() > 0
    _replays_equal_eager(lambda: ops.nvfp4_linear(x, lin, relu2=True))


@pytest.mark.parametrize("m", [1, 5, 64, 128])
def test_w3_linear_is_capturable(m):
    from hibana_amd.kernels import w3
    dev = w3.tile(to_device_w3(random_w3(512, 384, 5)[0]))
    x = torch.randn(m, 384, generator=torch.Generator().manual_seed(m)).bfloat16().cuda()
    y = _replays_equal_eager(lambda: w3.w3_linear(x, dev))
    assert y.float().abs().max() > 0
    q, s = w3.quant_groups(x)
    _replays_equal_eager(lambda: w3.w3_linear(q, dev, s))


@pytest.mark.parametrize("m", [1, 20, 300])
def test_nvfp4_experts_are_capturable(m):
    ex, _ = _experts(8, 256, 384, False, 5)
    g = torch.Generator().manual_seed(m)
    lat = torch.randn(m, 256, generator=g).bfloat16().cuda()
    ids = torch.stack([torch.randperm(8, generator=g)[:3] for _ in range(m)]).to(torch.int32).cuda()
    w = torch.rand(m, 3, generator=g).cuda()
    y = _replays_equal_eager(lambda: ex(lat, ids, w))
    assert y.float().abs().max() > 0


@pytest.mark.parametrize("m", [2, 48])
def test_latent_block_with_a_shared_expert_is_capturable(m):
    from hibana_amd.model import nemotron_moe
    e, hidden, latent, inter, topk, sh_inter = 16, 512, 256, 384, 4, 640
    ex, _ = _experts(e, latent, inter, False, 31, scaling=2.0)
    g = torch.Generator().manual_seed(17)
    gate_fc1 = torch.cat([torch.randn(e, hidden, generator=g) * 0.05, torch.randn(latent, hidden, generator=g) * 0.04]).bfloat16().cuda()
    fc2 = (torch.randn(hidden, latent, generator=g) * 0.04).bfloat16().cuda()
    block = nemotron_moe.NemotronMoe(gate_fc1, (torch.randn(e, generator=g) * 0.05).cuda(), fc2, ex, topk, _nvfp4_linear(sh_inter, hidden, 40),
                                     _nvfp4_linear(hidden, sh_inter, 41))
    x = torch.randn(m, hidden, generator=g).bfloat16().cuda()
    y = _replays_equal_eager(lambda: block(x))
    assert y.float().abs().max() > 0


@pytest.mark.parametrize("m", [1, 32])
def test_w3_moe_layer_from_logits_is_capturable(m):
    from hibana_amd.kernels import w3_moe
    from tests.util import random_experts
    ex, _ = random_experts(16, 256, 128, True, 7)
    sh, _ = random_experts(1, 256, 128, True, 8)
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, 256, generator=g).bfloat16().cuda()
    logits = torch.randn(m, 16, generator=g).cuda()
    gate = (torch.randn(256, generator=g) * 0.05).cuda()
    _replays_equal_eager(lambda: w3_moe.moe_layer_logits(ex, x, logits, 4, shared=sh, gate_vec=gate))
    _replays_equal_eager(lambda: w3_moe.moe_layer_logits(ex, x, logits, 4, shared=sh, gate_vec=gate, e4m3=True))
