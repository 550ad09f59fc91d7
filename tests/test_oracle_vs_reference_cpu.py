"""The oracle against the reference's own CPU kernels (oracle/_ref/liboq_ref_cpu.so, compiled
from the reference checkout by oracle/build.py).  Skipped where that library is not built.

The reference CPU quantizer multiplies by 1/(norm+eps) where the Python specification (and the
oracle) divides, and sums squares in an ISA-specific order, so values agree to rounding and a
code may flip only for a coordinate that sits on a bucket boundary to within rounding:
the test demands >= 99.99 % identical values and that every differing value is the neighbouring
centroid.  The packed matmul is compared within fp32 accumulation-order noise.
"""

import numpy as np
import pytest
import torch

from oracle import oracle_c, oracle_np, ref_cpu

pytestmark = pytest.mark.skipif(not ref_cpu.available(), reason="oracle/_ref/liboq_ref_cpu.so not built")


@pytest.mark.parametrize("dim,block,bits,dtype", [
    (1152, 64, 4, torch.float32), (1152, 128, 4, torch.bfloat16), (4608, 512, 4, torch.bfloat16),
    (3072, 1024, 3, torch.bfloat16), (5120, 1024, 6, torch.float16), (4096, 4096, 4, torch.bfloat16),
])
def test_quantize_activations_matches_reference_cpu(dim, block, bits, dtype):
    gen = torch.Generator().manual_seed(dim + bits)
    x = torch.randn(64, dim, generator=gen)
    x = torch.where(torch.rand(64, dim, generator=gen) < 0.01, x * 20, x).to(dtype)
    x[3] = 0
    perm, signs, _, _ = oracle_np.rpbh_constants(dim, 0, block)
    cents, bounds = oracle_np.lloyd_max_tables(dim, bits)
    inv = np.float32(1.0 / np.sqrt(block))
    ref = ref_cpu.quantize_activations_cpu(
        x, torch.from_numpy(perm.astype(np.int64)), torch.from_numpy(signs), torch.from_numpy(cents),
        torch.from_numpy(bounds), eps=1e-10, inv_sqrt_block=float(inv), block_size=block)
    codes, s = oracle_c.rotate_quantize(x.float().numpy(), perm.astype(np.int32), signs, bounds, block, 1e-10, inv)
    # recover the reference's codes from its values (centroids are well separated)
    s64 = np.maximum(s.astype(np.float64), 1e-300)[:, None]
    ref_unit = ref.double().numpy() / s64
    ref_codes = np.abs(ref_unit[:, :, None] - cents.astype(np.float64)[None, None, :]).argmin(-1)
    live = s > 0
    same = ref_codes[live] == codes[live]
    assert same.mean() >= 0.9999
    assert np.abs(ref_codes[live].astype(int) - codes[live].astype(int)).max() <= 1   # only boundary ties differ
    assert not ref[3].any()                                                              # zero token -> zeros
    # and the values themselves agree to rounding of the token norm / output dtype
    mine = torch.from_numpy(cents[codes] * s[:, None]).to(dtype).double().numpy()
    tol = {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
    agree = np.abs(mine - ref.double().numpy()) <= tol * np.abs(mine) + 1e-30
    assert agree[live][same].all()


@pytest.mark.parametrize("bits", [2, 3, 4, 6, 8])
@pytest.mark.parametrize("m,k,n", [(5, 256, 37), (33, 1152, 96)])
def test_matmul_packed_weight_matches_reference_cpu(bits, m, k, n):
    gen = np.random.default_rng(bits * 100 + m)
    idx = gen.integers(0, 1 << bits, size=(n, k), dtype=np.int64)
    packed = oracle_np.pack_bits(idx.reshape(-1), bits)
    cents = np.sort(gen.standard_normal(1 << bits)).astype(np.float32) * 0.1
    r = np.linspace(0.5, 1.5, n).astype(np.float32)
    bias = gen.standard_normal(n).astype(np.float32)
    x = gen.standard_normal((m, k)).astype(np.float32)
    ref = ref_cpu.matmul_packed_weight(torch.from_numpy(x), torch.from_numpy(packed), torch.from_numpy(r),
                                       torch.from_numpy(cents), bits=bits, out_features=n, in_features=k,
                                       bias=torch.from_numpy(bias)).numpy()
    mine = oracle_c.matmul_packed_weight(x, packed, r, cents, bias, bits, n)
    exact = (x.astype(np.float64) @ cents[idx].astype(np.float64).T) * r + bias
    scale = np.linalg.norm(x, axis=1)[:, None] * (np.linalg.norm(cents[idx], axis=1) * r)[None, :] / np.sqrt(k)
    assert np.max(np.abs(ref - exact) / scale) < 1e-5
    assert np.max(np.abs(mine - exact) / scale) < 1e-5
    assert np.max(np.abs(mine - ref) / scale) < 1e-5
