"""GPU tests: the index bit-stream packer and the dense expansion of a packed weight against the
oracle's bit-stream functions (bit-exact)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import oracle_np as o

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("count", [1, 7, 8, 9, 1000, 64 * 1152 + 3])
def test_pack_lowbit_matches_the_oracle_and_round_trips(bits, count):
    from orbitquant_amd import ops

    rng = np.random.default_rng(bits * 1000 + count)
    values = rng.integers(0, 256, size=count, dtype=np.uint8)       # high bits set: the packer keeps the low `bits` only
    packed = ops.pack_lowbit(torch.from_numpy(values).to("cuda:0"), bits)
    want = o.pack_bits(values & ((1 << bits) - 1), bits)
    assert np.array_equal(packed.cpu().numpy(), want)
    back = ops.unpack_lowbit(packed, bits, count)
    assert np.array_equal(back.cpu().numpy(), values & ((1 << bits) - 1))


def test_pack_lowbit_of_nothing():
    from orbitquant_amd import ops

    assert ops.pack_lowbit(torch.empty(0, dtype=torch.uint8, device="cuda:0"), 3).numel() == 0


@pytest.mark.parametrize("bits,N,K", [(2, 64, 1152), (3, 33, 70), (4, 16, 4608), (6, 5, 3), (8, 7, 24), (3, 3, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_dequantize_packed_weight(bits, N, K, dtype):
    from orbitquant_amd import ops

    rng = np.random.default_rng(bits + N + K)
    idx = rng.integers(0, 1 << bits, size=(N, K), dtype=np.uint8)
    cents = np.sort(rng.standard_normal(1 << bits)).astype(np.float32)
    norms = torch.from_numpy(rng.uniform(0.1, 4.0, N).astype(np.float32)).to(torch.bfloat16)
    packed = torch.from_numpy(o.pack_bits(idx.reshape(-1), bits))
    got = ops.dequantize_packed_weight(packed.to("cuda:0"), norms.to("cuda:0"), torch.from_numpy(cents).to("cuda:0"), bits=bits,
                                       out_features=N, in_features=K, dtype=dtype)
    want = torch.from_numpy(cents[idx] * norms.float().numpy()[:, None]).to(dtype)   # one fp32 product, one rounding
    assert got.shape == (N, K) and got.dtype == dtype
    assert torch.equal(got.cpu(), want)
