"""The C restatement of the CPU path against the numpy/torch oracle (CPU)."""
import numpy as np
import torch

from oracle import c_port, layers, w3_format as ow3
from tests.util import random_w3


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).numpy().view(np.uint16)


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_codes_and_dequantize_are_bit_exact():
    for n, k, book in ((128, 256, "uniform"), (256, 384, "lloyd"), (128, 128, "lloyd2"), (384, 640, "zero8")):
        packed, q, raw, row = random_w3(n, k, 4, book)
        assert np.array_equal(c_port.codes(packed["planes"], n, k, packed["planes"].shape[2]), q)
        assert np.array_equal(c_port.dequantize(packed).view(np.uint32), ow3.dequantize(packed).view(np.uint32))


def test_linear_and_moe_layer_follow_the_oracle():
    packed, *_ = random_w3(256, 512, 5)
    x = torch.randn(5, 512, generator=torch.Generator().manual_seed(1)).bfloat16()
    want = layers.dense_ref(x, ow3.dequantize(packed))
    got = _bf16(c_port.linear(packed, _bits(x)))
    assert float((got.float() - want.float()).abs().max() / want.float().abs().max()) < 2 ** -7
    for gated in (True, False):
        e, hidden, inter = 6, 256, 128
        n1 = 2 * inter if gated else inter
        per = [(random_w3(n1, hidden, 100 + 2 * i)[0], random_w3(hidden, inter, 101 + 2 * i, "zero8")[0]) for i in range(e + 1)]
        stack = lambda idx, name, sel: np.stack([per[i][idx][name] for i in sel])  # noqa: E731
        routed = c_port.HostExperts(*(stack(0, f, range(e)) for f in ("planes", "scales", "row_scale")),
                                    *(stack(1, f, range(e)) for f in ("planes", "scales", "row_scale")),
                                    per[0][0]["codebook"], per[0][1]["codebook"], hidden, inter, gated)
        shared = c_port.HostExperts(*(stack(0, f, [e]) for f in ("planes", "scales", "row_scale")),
                                    *(stack(1, f, [e]) for f in ("planes", "scales", "row_scale")),
                                    per[0][0]["codebook"], per[0][1]["codebook"], hidden, inter, gated)
        g = torch.Generator().manual_seed(7)
        m, k = 9, 3
        x = torch.randn(m, hidden, generator=g).bfloat16()
        ids = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(m)]).numpy().astype(np.int32)
        ids[1, 2] = 512
        weights = torch.softmax(torch.randn(m, k, generator=g), -1)
        gate = torch.randn(hidden, generator=g) * 0.05
        inverse = np.argsort(layers.fc1_order(inter)) if gated else np.arange(inter)
        get = lambda i: (ow3.dequantize(per[i][0])[inverse], ow3.dequantize(per[i][1]))  # noqa: E731
        for sh, gv in ((None, None), (shared, None), (shared, gate)):
            want = layers.moe_layer_ref(x, ids, weights, get, gated, shared=get(e) if sh else None, gate_vec=gv, e_n=e)
            got, distinct = c_port.moe_layer(routed, _bits(x), ids, weights.numpy(), sh, None if gv is None else gv.numpy())
            assert distinct == len(set(ids.reshape(-1).tolist()) - {512})
            got = _bf16(got)
            assert float((got.float() - want.float()).norm() / want.float().norm()) < 4e-3
            assert float((got.float() - want.float()).abs().max() / want.float().abs().max()) < 2e-2
