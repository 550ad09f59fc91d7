"""GPU test of oq_quantized_linear_static, the entry point that allocates nothing: its scratch
(activation codes and token norms between the two launches) is a buffer inside the library's
device image instead of a workspace the caller brings.  The contract is bit identity with
oq_quantized_linear on the same inputs, also when a call with a smaller input follows a larger
one (the buffer keeps the previous call's contents), and a clear refusal beyond the buffer's size.

Everything goes through the C ABI with raw pointers; outputs are allocated here, by the caller."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20  # OQ_STATIC_SCRATCH_BYTES of include/orbitquant_hip.h


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


def make_layer(dev, k, n, wbits, abits, dtype, seed):
    from orbitquant_amd.codebooks import get_codebook
    from orbitquant_amd.rotations import get_rpbh_rotation

    rot, acb, wcb = get_rpbh_rotation(k, 0, "paper"), get_codebook(k, abits), get_codebook(k, wbits)
    g = torch.Generator().manual_seed(seed)
    return dict(
        k=k, n=n, wbits=wbits, abits=abits, dtype=dtype, block=rot.block_size, inv=float(rot.normalization),
        perm=rot.permutation.to(torch.int32).to(dev), signs=rot.signs.to(torch.int8).to(dev),
        bounds=acb.boundaries.to(dev), cents=acb.centroids.to(dev), wcents=wcb.centroids.to(dev),
        packed=torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=g, dtype=torch.uint8).to(dev),
        rn=(0.02 * (1 + 0.1 * torch.randn(n, generator=g))).to(torch.bfloat16).to(dev),
        bias=torch.randn(n, generator=g).to(dtype).to(dev))


def make_tokens(dev, layer, m, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, layer["k"], generator=g)
    x[torch.rand(m, layer["k"], generator=g) < 0.01] *= 20
    return x.to(layer["dtype"]).to(dev)


def call(layer, x, *, static):
    """One call through the C ABI into a caller-allocated output; returns (status, output)."""
    from orbitquant_amd import _lib

    lib = _lib.load()
    dt = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[x.dtype]
    m, k, n = x.shape[0], layer["k"], layer["n"]
    out = torch.full((m, n), float("nan"), dtype=x.dtype, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    head = (x.data_ptr(), dt, None, m, k, layer["perm"].data_ptr(), layer["signs"].data_ptr(),
            layer["bounds"].data_ptr(), layer["cents"].data_ptr(), layer["abits"], layer["block"], 1e-10, layer["inv"],
            layer["plan"].data_ptr() if layer.get("plan") is not None else None, layer["packed"].data_ptr(), layer["wbits"], layer["rn"].data_ptr(), layer["wcents"].data_ptr(),
            layer["bias"].data_ptr(), dt, n)
    if static:
        rc = lib.oq_quantized_linear_static(*head, out.data_ptr(), dt, None, stream)
    else:
        nibble = layer["abits"] <= 4 and k % 2 == 0
        codes = torch.empty((m, k // 2 if nibble else k), dtype=torch.uint8, device=x.device)
        norms = torch.empty(m, dtype=torch.float32, device=x.device)
        rc = lib.oq_quantized_linear(*head, codes.data_ptr(), norms.data_ptr(), out.data_ptr(), dt, None, None, 0, stream)
    torch.cuda.synchronize()
    return rc, out


@pytest.mark.parametrize("k,n,wbits,abits,dtype,sizes", [
    (1152, 384, 4, 4, torch.bfloat16, (96, 7)),      # tile kernel, then the streaming kernel on fewer tokens
    (4096, 512, 3, 6, torch.bfloat16, (40, 24)),     # one code per byte (six-bit activations)
    (3072, 256, 2, 3, torch.float16, (33, 1)),       # two launches, then the single launch of one token
    (1152, 128, 4, 4, torch.float32, (20, 3)),
    (4096, 256, 4, 4, torch.bfloat16, (128, 64)),    # few tiles, many K-steps: the allocating call shares K between workgroups
])
def test_static_scratch_equals_caller_scratch(dev, k, n, wbits, abits, dtype, sizes):
    layer = make_layer(dev, k, n, wbits, abits, dtype, seed=k + n)
    for i, m in enumerate(sizes):  # two calls in a row, the second with the smaller input
        x = make_tokens(dev, layer, m, seed=100 + i)
        rc_ref, want = call(layer, x, static=False)
        rc, got = call(layer, x, static=True)
        assert rc_ref == 0 and rc == 0
        assert not torch.isnan(got.float()).any()
        if k == 4096 and m == 128:
            # the call that may allocate adds partial sums of K from a buffer of the library's own; the static call
            # never takes one: same products, another order of the last additions
            assert (got.float() - want.float()).abs().max().item() <= want.float().abs().max().item() * 2.0 ** -7
            continue
        assert torch.equal(got, want), f"m={m}: {(got.float() - want.float()).abs().max().item()}"


def test_static_scratch_fills_to_its_limit_and_refuses_beyond(dev, library_switch):
    from orbitquant_amd import _lib

    library_switch("OQ_GEMM_WG_SPLIT", "1")   # the allocating call as one launch over K, like the static one

    lib = _lib.load()
    k = 4096
    layer = make_layer(dev, k, 128, 4, 4, torch.bfloat16, seed=5)
    # nibble codes: m * k / 2 bytes rounded up to 256, plus 4 m bytes of norms
    m_max = SCRATCH_BYTES // (k // 2 + 4)
    while ((m_max * (k // 2) + 255) // 256) * 256 + 4 * m_max > SCRATCH_BYTES:
        m_max -= 1
    x = make_tokens(dev, layer, m_max + 1, seed=9)
    rc_ref, want = call(layer, x[:m_max], static=False)
    rc, got = call(layer, x[:m_max], static=True)
    assert rc_ref == 0 and rc == 0 and torch.equal(got, want)
    rc, _ = call(layer, x, static=True)
    assert rc == 2, "one token more than fits must be refused as unsupported"
    message = lib.oq_last_error().decode()
    assert "scratch" in message and str(SCRATCH_BYTES) in message
