"""Seeded random shapes through oq_packed_linear against the oracle, drawn around the token counts at
which the dispatcher changes kernels (1, 16/17: row blocks of the streaming kernel; 64/65: tile kernel;
a few hundred tokens on long rows: K shared between workgroups) and with ragged N, every weight width
and both code formats.  The named tests cover each kernel on chosen shapes; this one looks for a
shape nobody chose."""

from __future__ import annotations

import numpy as np
import pytest
import torch

import test_gpu_parity as tp

pytestmark = pytest.mark.gpu

TOKENS = [1, 2, 5, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 300, 511, 600]


def draw_cases(count: int, seed: int):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        m = int(rng.choice(TOKENS))
        k = int(rng.choice([128, 256, 384, 512, 1024, 1152, 2048, 3072, 4096, 6144]))
        if m > 200 and k > 2048:
            k = int(rng.choice([512, 1024, 2048]))          # keeps the oracle within seconds
        n = int(rng.choice([8, 16, 24, 40, 64, 96, 120, 128, 136, 200, 256, 264, 520]))
        wbits = int(rng.choice([2, 3, 4, 6, 8]))
        abits = int(rng.choice([2, 3, 4, 4, 4, 6, 8]))
        cases.append((m, n, k, wbits, abits, bool(rng.integers(2)), bool(rng.integers(2))))
    return cases


CASES = draw_cases(72, seed=20240611)


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


@pytest.mark.parametrize(("m", "n", "k", "wbits", "abits", "with_bias", "fp32_out"), CASES)
def test_packed_linear_random_shape(dev, m, n, k, wbits, abits, with_bias, fp32_out):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k + wbits * 7 + abits)
    layer = tp.make_layer(rng, n, k, wbits, abits, with_bias=with_bias)
    _, x32 = tp.make_x(rng, m, k, torch.bfloat16)
    if m > 2:
        x32[m // 2] = 0
    codes, s = tp.oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    out_dtype = torch.float32 if fp32_out else torch.bfloat16
    want = tp.oracle_linear(layer, codes, s, out_dtype)
    formats = ["u8"] if abits > 4 else ["nibble", "u8"]
    for fmt in formats:
        got = tp.run_packed_linear(dev, layer, codes, s, fmt, out_dtype)
        assert got.dtype == out_dtype and tuple(got.shape) == (m, n)
        tp.check_outputs(got, want, s, layer["r"].float().numpy(), k, f"{fmt} codes")
        if m > 2:   # a zero token gives exactly the bias
            expect = np.zeros(n) if layer["bias"] is None else torch.from_numpy(layer["bias"]).to(out_dtype).float().numpy()
            assert np.array_equal(got[m // 2].float().cpu().numpy(), expect)
        assert torch.equal(got, tp.run_packed_linear(dev, layer, codes, s, fmt, out_dtype))   # reproducible
