"""GPU parity: the HIP path (through the C ABI) against the CPU oracle.

Bars: activation codes, token norms and packed-index decode bit-exact; matmul
outputs within max-abs-error <= 2e-2 * ||x|| * ||w_row|| / sqrt(K) per element and
cosine similarity >= 0.9999 against the fp64 statement of the dequantized path.
"""

from __future__ import annotations

import math

import numpy as np
import pytest
import torch

from oracle import oracle_c, oracle_np as o
from parity_util import cosine, output_error, outside_rounded_bound, reference_tables

pytestmark = pytest.mark.gpu

F32 = np.float32


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


_TABLES: dict = {}


def tables(dim, bits):
    """The reference generator's own table where the golden file holds one (every configuration
    dimension), the oracle's elsewhere."""
    key = (dim, bits)
    if key not in _TABLES:
        _TABLES[key] = reference_tables(dim, bits)
    return _TABLES[key]


def make_x(rng, m, k, dtype, kind="outliers"):
    x = rng.standard_normal((m, k)).astype(F32)
    if kind == "outliers":
        x[rng.random(x.shape) < 0.01] *= 20
    elif kind == "student":
        x = rng.standard_t(4, size=(m, k)).astype(F32)
    t = torch.from_numpy(x).to(dtype)
    return t, t.float().numpy()


def gpu_rotate_quantize(dev, xt, perm, signs, bounds, block, eps, inv, cents=None, fmt="u8", values=None):
    from orbitquant_amd import ops

    return ops.rotate_quantize(
        xt.to(dev), torch.from_numpy(perm.astype(np.int32)).to(dev), torch.from_numpy(signs).to(dev),
        torch.from_numpy(bounds).to(dev), block_size=block, eps=eps, inv_sqrt_block=float(inv),
        centroids=None if cents is None else torch.from_numpy(cents).to(dev), code_format=fmt, values=values)


# --------------------------------------------------------------- rotate+quantize

RQ_CASES = [
    # dim, block, a_bits, dtype, rows
    (24, 8, 4, torch.float32, 7),
    (37, 1, 4, torch.float32, 3),
    (64, 64, 2, torch.bfloat16, 5),
    (512, 512, 4, torch.bfloat16, 4),
    (1152, 64, 4, torch.float32, 33),      # C1
    (1152, 128, 4, torch.bfloat16, 40),    # C2 fc1
    (4608, 512, 4, torch.bfloat16, 21),    # C2 fc2
    (3072, 1024, 3, torch.bfloat16, 17),   # C3
    (12288, 4096, 3, torch.bfloat16, 5),   # C3 fc2
    (5120, 1024, 6, torch.bfloat16, 9),    # C4 fc1
    (13824, 512, 6, torch.bfloat16, 5),    # C4 fc2
    (4096, 4096, 4, torch.bfloat16, 16),   # C5
    (14336, 2048, 4, torch.bfloat16, 4),   # C5 down
    (16384, 16384, 4, torch.float16, 2),
    (2048, 2, 8, torch.float16, 3),
]


@pytest.mark.parametrize(("dim", "block", "abits", "dtype", "rows"), RQ_CASES)
def test_rotate_quantize_codes_and_norms_bit_exact(dev, dim, block, abits, dtype, rows):
    rng = np.random.default_rng(dim * 31 + block)
    perm, signs, block, inv = o.rpbh_constants(dim, 0, block)
    cents, bounds = tables(max(dim, 3), abits)
    xt, x32 = make_x(rng, rows, dim, dtype)
    xt[rows // 2] = 0
    x32[rows // 2] = 0
    want_codes, want_norms = oracle_c.rotate_quantize(x32, perm, signs, bounds, block, 1e-10, inv)
    codes, values, norms = gpu_rotate_quantize(dev, xt, perm, signs, bounds, block, 1e-10, inv, cents, "u8", "scaled")
    assert np.array_equal(norms.cpu().numpy().view(np.int32), want_norms.view(np.int32))
    got = codes.cpu().numpy()
    mism = int((got != want_codes).sum())
    assert mism == 0, f"{mism} code mismatches of {got.size}"
    want_values = torch.from_numpy(cents[want_codes] * want_norms[:, None]).to(dtype)
    assert torch.equal(values.cpu(), want_values)
    assert not values[rows // 2].any()
    if abits <= 4 and dim % 2 == 0:
        nib, unit, norms2 = gpu_rotate_quantize(dev, xt, perm, signs, bounds, block, 1e-10, inv, cents, "nibble", "unit_bf16")
        assert np.array_equal(nib.cpu().numpy(), o.pack_nibbles(want_codes))
        assert torch.equal(norms2, norms)
        assert torch.equal(unit.cpu(), torch.from_numpy(cents[want_codes]).to(torch.bfloat16))


@pytest.mark.parametrize("dim", [512, 4096, 16384])
def test_rotate_quantize_one_hot_rows(dev, dim):
    # native tests/test_packed_matmul.py:688-733 (reference checkout): closed form per row
    gen = torch.Generator().manual_seed(dim)
    perm = torch.randperm(dim, generator=gen).numpy()
    signs = np.where(np.arange(dim) % 2 == 0, 1, -1).astype(np.int8)
    bounds = np.linspace(-0.2, 0.2, 15, dtype=F32)
    x = torch.zeros((2, dim), dtype=torch.bfloat16)
    x[0, 3] = 1
    x[1, dim - 7] = -1
    inv = F32(dim ** -0.5)
    nib, _, norms = gpu_rotate_quantize(dev, x, perm, signs, bounds, dim, 1e-12, inv, None, "nibble")
    assert norms.cpu().tolist() == [1.0, 1.0]
    rows = []
    for hot, val in ((3, 1.0), (dim - 7, -1.0)):
        c = int(np.nonzero(perm == hot)[0][0])
        j = np.arange(dim)
        parity = np.array([bin(v).count("1") & 1 for v in (c & j)])
        rot = (np.where(parity == 1, -1.0, 1.0) * val * signs[c]).astype(F32) * inv
        rows.append(np.searchsorted(bounds, rot, side="left").astype(np.uint8))
    assert np.array_equal(nib.cpu().numpy(), o.pack_nibbles(np.stack(rows)))


@pytest.mark.parametrize("kind", ["clustered", "duplicates", "one_sided", "wide_range", "two_levels", "sixty_four"])
def test_rotate_quantize_awkward_boundaries(dev, kind):
    """Boundary sets that defeat (or stress) the kernel's uniform cell table: the codes must still be
    the count of boundaries below each value, ties included."""
    rng = np.random.default_rng(len(kind))
    dim, block, rows = 256, 64, 24
    if kind == "clustered":       # several boundaries closer together than a cell: binary-search fallback
        bounds = np.array([-0.3, -0.1, -1e-6, 0.0, 1e-7, 2e-7, 3e-7, 0.05, 0.05001, 0.1, 0.11, 0.2, 0.21, 0.3, 0.31], dtype=F32)
    elif kind == "duplicates":
        bounds = np.array([-0.2, -0.1, -0.1, 0.0, 0.0, 0.0, 0.1, 0.1, 0.15, 0.2, 0.25, 0.3, 0.3, 0.4, 0.5], dtype=F32)
    elif kind == "one_sided":
        bounds = np.linspace(0.01, 0.2, 15, dtype=F32)
    elif kind == "wide_range":    # every value falls into the first or last cells
        bounds = np.linspace(-1e6, 1e6, 15, dtype=F32)
    elif kind == "two_levels":
        bounds = np.array([0.0], dtype=F32)
    else:
        bounds = np.sort(rng.standard_normal(63).astype(F32) * 0.08)
    perm, signs, block, inv = o.rpbh_constants(dim, 3, block)
    x32 = rng.standard_normal((rows, dim)).astype(F32)
    x32[1] = 0
    # rows that land exactly on boundaries after rotation are rare; force ties through a one-hot row whose
    # rotated entries are +-inv and boundaries that include those very values
    x32[2] = 0
    x32[2, 5] = 1.0
    if kind == "clustered":
        bounds[0], bounds[-1] = -inv, inv
        bounds = np.sort(bounds)
    xt = torch.from_numpy(x32)
    want_codes, want_norms = oracle_c.rotate_quantize(x32, perm, signs, bounds, block, 1e-10, inv)
    codes, _, norms = gpu_rotate_quantize(dev, xt, perm, signs, bounds, block, 1e-10, inv, None, "u8")
    assert np.array_equal(norms.cpu().numpy().view(np.int32), want_norms.view(np.int32))
    assert np.array_equal(codes.cpu().numpy(), want_codes)


def test_rotate_quantize_full_size_c2_bit_exact(dev):
    # BASELINE config 2, second quantizer: [2048, 4608] bf16 with outlier columns x30
    rng = np.random.default_rng(2)
    m, dim = 2048, 4608
    perm, signs, block, inv = o.rpbh_constants(dim, 0)
    cents, bounds = tables(dim, 4)
    x = rng.standard_normal((m, dim)).astype(F32)
    x[:, rng.choice(dim, 23, replace=False)] *= 30
    xt = torch.from_numpy(x).to(torch.bfloat16)
    want_codes, want_norms = oracle_c.rotate_quantize(xt.float().numpy(), perm, signs, bounds, block, 1e-10, inv)
    codes, _, norms = gpu_rotate_quantize(dev, xt, perm, signs, bounds, block, 1e-10, inv)
    assert np.array_equal(norms.cpu().numpy().view(np.int32), want_norms.view(np.int32))
    assert int((codes.cpu().numpy() != want_codes).sum()) == 0
    # batch independence: any slice of rows gives the same codes
    part, _, _ = gpu_rotate_quantize(dev, xt[100:117], perm, signs, bounds, block, 1e-10, inv)
    assert torch.equal(part, codes[100:117])


def test_rotate_quantize_rejects_bad_arguments(dev):
    perm, signs, block, inv = o.rpbh_constants(64, 0, 64)
    _, bounds = tables(64, 4)
    x = torch.zeros((2, 64), dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        gpu_rotate_quantize(dev, x, perm, signs, bounds, 48, 1e-10, inv)       # not a power of two
    _, b6 = tables(64, 6)
    with pytest.raises(ValueError):
        gpu_rotate_quantize(dev, x, perm, signs, b6, 64, 1e-10, inv, fmt="nibble")   # 64 levels in a nibble


# ---------------------------------------------------------------------- unpack

@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_unpack_lowbit_bit_exact(dev, bits):
    from orbitquant_amd import ops

    values = (np.arange(100003) * 7 % (1 << bits)).astype(np.uint8)
    packed = o.pack_bits(values, bits)
    got = ops.unpack_lowbit(torch.from_numpy(packed).to(dev), bits, values.size)
    assert np.array_equal(got.cpu().numpy(), values)


# ---------------------------------------------------------------- packed linear

def make_layer(rng, n, k, wbits, abits, block="paper", scale=0.02, with_bias=True):
    perm, signs, block, inv = o.rpbh_constants(k, 0, block)
    cw, bw = tables(k, wbits)
    ca, ba = tables(k, abits)
    w = (rng.standard_normal((n, k)) * scale).astype(F32)
    packed, r_bf16, idx = o.quantize_weight(w, perm, signs, bw, block, 1e-10, wbits)
    bias = rng.standard_normal(n).astype(F32) * 0.1 if with_bias else None
    return dict(perm=perm, signs=signs, block=block, inv=inv, cw=cw, bw=bw, ca=ca, ba=ba, packed=packed,
                r=r_bf16, idx=idx, bias=bias, n=n, k=k, wbits=wbits, abits=abits)


def check_outputs(got, want, s, r, k, what=""):
    """`got`: the kernel's output tensor.  fp32 outputs must meet the bound as it stands; 16-bit
    outputs with the half-ulp of their own format added (the message reports both)."""
    out_dtype = got.dtype
    got = got.float().cpu().numpy()
    is16 = out_dtype != torch.float32
    strict, rounded = output_error(got, want, s, r, k, is16, out_dtype == torch.bfloat16)
    assert rounded <= 1.0, f"{what}: max error is {rounded:.3f} of the bound ({strict:.3f} without the output format's half-ulp)"
    if is16:   # every stored output must be the rounding of a value within the stated bound: any excess is output rounding alone
        bad = outside_rounded_bound(got, want, s, r, k, out_dtype == torch.bfloat16)
        assert bad == 0, f"{what}: {bad} outputs are not the rounding of any value within the bound"
    cos = cosine(got, want)
    assert cos >= 0.9999, f"{what}: cosine {cos}"
    return rounded, cos


def run_packed_linear(dev, layer, codes_np, s_np, fmt, out_dtype=torch.bfloat16):
    from orbitquant_amd import ops

    if fmt == "nibble":
        codes_t = torch.from_numpy(o.pack_nibbles(codes_np))
    else:
        codes_t = torch.from_numpy(codes_np)
    bias = None if layer["bias"] is None else torch.from_numpy(layer["bias"]).to(out_dtype).to(dev)
    return ops.packed_linear(
        codes_t.to(dev), torch.from_numpy(s_np).to(dev), torch.from_numpy(layer["ca"]).to(dev),
        torch.from_numpy(layer["packed"]).to(dev), layer["r"].to(dev), torch.from_numpy(layer["cw"]).to(dev),
        code_format=fmt, activation_bits=layer["abits"], weight_bits=layer["wbits"],
        out_features=layer["n"], in_features=layer["k"], bias=bias, output_dtype=out_dtype)


def oracle_linear(layer, codes, s, out_dtype):
    bias = layer["bias"]
    if bias is not None:
        bias = torch.from_numpy(bias).to(out_dtype).float().numpy()
    return oracle_c.linear_from_codes(codes, s, layer["ca"], layer["packed"], layer["wbits"],
                                      layer["r"].float().numpy(), layer["cw"], bias, layer["n"])


GEMM_CASES = [
    # m, n, k, wbits, abits, block, bias, out dtype
    (256, 1152, 1152, 4, 4, 64, True, torch.float32),      # C1 full size
    (300, 200, 1152, 4, 4, "paper", True, torch.bfloat16), # ragged M and N
    (130, 258, 256, 4, 4, "paper", False, torch.bfloat16),
    (257, 384, 3072, 3, 3, "paper", True, torch.bfloat16), # C3 widths
    (129, 96, 4608, 2, 4, "paper", True, torch.bfloat16),
    (200, 160, 1024, 6, 4, "paper", False, torch.float16),
    (100, 130, 512, 8, 4, "paper", True, torch.bfloat16),
    (64, 64, 64, 4, 2, "paper", True, torch.bfloat16),
    (33, 70, 192, 3, 4, "paper", True, torch.bfloat16),
]


@pytest.mark.parametrize(("m", "n", "k", "wbits", "abits", "block", "with_bias", "out_dtype"), GEMM_CASES)
def test_packed_linear_tile_kernel(dev, m, n, k, wbits, abits, block, with_bias, out_dtype):
    rng = np.random.default_rng(m * 7 + n * 3 + k + wbits)
    layer = make_layer(rng, n, k, wbits, abits, block, with_bias=with_bias)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    x32[1] = 0
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, out_dtype)
    got = run_packed_linear(dev, layer, codes, s, "nibble", out_dtype)
    assert got.dtype == out_dtype and tuple(got.shape) == (m, n)
    check_outputs(got, want, s, layer["r"].float().numpy(), k, "nibble")
    # zero token -> exactly the bias (tests/test_paper_reference_oracle.py:202-203, reference checkout)
    zero_row = got[1].float().cpu().numpy()
    expect = np.zeros(n) if layer["bias"] is None else torch.from_numpy(layer["bias"]).to(out_dtype).float().numpy()
    assert np.array_equal(zero_row, expect)
    # one code per byte takes the shape-agnostic kernel: same answer
    got_u8 = run_packed_linear(dev, layer, codes, s, "u8", out_dtype)
    check_outputs(got_u8, want, s, layer["r"].float().numpy(), k, "u8")


@pytest.mark.parametrize(("m", "n", "k", "wbits", "abits"), [
    (300, 200, 1024, 4, 6), (130, 96, 256, 4, 8), (257, 384, 1536, 3, 6), (64, 64, 64, 2, 5), (100, 136, 512, 6, 6),
    (90, 72, 384, 8, 8), (515, 520, 1152, 4, 4)])
@pytest.mark.parametrize("tile", ["0", "1", "2", "3", "4"])
def test_packed_linear_byte_codes_tile_kernel(dev, m, n, k, wbits, abits, tile, library_switch):
    """One activation code per byte (a_bits up to 8) through the all-table tile kernel."""
    library_switch("OQ_GEMM_TILE", tile)
    rng = np.random.default_rng(m + 3 * n + k + wbits + abits + int(tile))
    layer = make_layer(rng, n, k, wbits, abits)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    x32[2] = 0
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, torch.bfloat16)
    got = run_packed_linear(dev, layer, codes, s, "u8")
    check_outputs(got, want, s, layer["r"].float().numpy(), k, f"u8 tile {tile}")
    expect = np.zeros(n) if layer["bias"] is None else torch.from_numpy(layer["bias"]).to(torch.bfloat16).float().numpy()
    assert np.array_equal(got[2].float().cpu().numpy(), expect)


@pytest.mark.parametrize("tile", ["0", "1", "2", "3"])
def test_packed_linear_every_tile_shape(dev, tile, library_switch):
    library_switch("OQ_GEMM_TILE", tile)
    rng = np.random.default_rng(int(tile) + 50)
    m, n, k = 515, 520, 1152
    layer = make_layer(rng, n, k, 4, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, torch.bfloat16)
    got = run_packed_linear(dev, layer, codes, s, "nibble")
    check_outputs(got, want, s, layer["r"].float().numpy(), k, f"tile {tile}")


@pytest.mark.parametrize("tile", ["0", "1", "2", "3", "4"])
@pytest.mark.parametrize(("m", "n", "k"), [(17, 8, 256), (33, 24, 512), (300, 8, 256)])
def test_packed_linear_tiny_outputs_every_tile(dev, m, n, k, tile, library_switch):
    """Outputs much smaller than a tile: every row / column clamp and store guard is exercised."""
    library_switch("OQ_GEMM_TILE", tile)
    rng = np.random.default_rng(m * 5 + n + k + int(tile))
    layer = make_layer(rng, n, k, 4, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, torch.float32)
    got = run_packed_linear(dev, layer, codes, s, "nibble", torch.float32)
    check_outputs(got, want, s, layer["r"].float().numpy(), k, f"tiny tile {tile}")


@pytest.mark.parametrize(("m", "n", "k", "wbits"), [(300, 200, 1024, 4), (128, 96, 256, 4), (515, 1152, 2304, 3), (130, 104, 512, 6)])
def test_packed_linear_k_split_kernel(dev, m, n, k, wbits, library_switch):
    """Four wavefronts share one output tile and a quarter of K each; partial tiles are summed through LDS."""
    library_switch("OQ_GEMM_TILE", "4")
    rng = np.random.default_rng(m + n + k)
    layer = make_layer(rng, n, k, wbits, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, torch.bfloat16)
    got = run_packed_linear(dev, layer, codes, s, "nibble")
    check_outputs(got, want, s, layer["r"].float().numpy(), k, "k-split")
    again = run_packed_linear(dev, layer, codes, s, "nibble")
    assert torch.equal(got, again)  # fixed summation order: bitwise reproducible


@pytest.mark.parametrize(("m", "n", "k", "wbits", "abits", "splits"), [
    (128, 256, 2048, 4, 4, 2), (65, 520, 4096, 4, 4, 4), (300, 136, 8192, 3, 3, 8), (129, 96, 4608, 2, 4, 3),
    (200, 264, 3072, 6, 4, 2), (130, 128, 2048, 8, 4, 2), (256, 384, 4096, 4, 6, 4), (100, 72, 2048, 3, 8, 2)])
def test_packed_linear_k_shared_between_workgroups(dev, m, n, k, wbits, abits, splits, library_switch):
    """Several workgroups per output tile, each over a part of K, fp32 partial tiles added by a second launch:
    against the oracle, against the single launch (same products, another summation order), and reproducible."""
    rng = np.random.default_rng(m + n + k + wbits)
    layer = make_layer(rng, n, k, wbits, abits)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    x32[2] = 0
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    fmt = "nibble" if abits <= 4 else "u8"
    want = oracle_linear(layer, codes, s, torch.bfloat16)
    library_switch("OQ_GEMM_WG_SPLIT", "1")
    single = run_packed_linear(dev, layer, codes, s, fmt)
    library_switch("OQ_GEMM_WG_SPLIT", str(splits))
    got = run_packed_linear(dev, layer, codes, s, fmt)
    check_outputs(got, want, s, layer["r"].float().numpy(), k, f"{splits} parts of K")
    assert torch.equal(got, run_packed_linear(dev, layer, codes, s, fmt))   # fixed order of the parts
    scale = single.float().abs().max().item()
    assert (got.float() - single.float()).abs().max().item() <= scale * 2.0 ** -7
    zero_row = got[2].float().cpu().numpy()      # a zero token gives exactly the bias
    assert np.array_equal(zero_row, torch.from_numpy(layer["bias"]).to(torch.bfloat16).float().numpy())
    fp32 = run_packed_linear(dev, layer, codes, s, fmt, torch.float32)
    check_outputs(fp32, oracle_linear(layer, codes, s, torch.float32), s, layer["r"].float().numpy(), k, "fp32 out")


def test_packed_linear_shares_k_under_graph_capture_too(dev, library_switch):
    """Which kernel a call takes depends on its arguments alone (the partial tiles live in a workspace the
    caller provides, here the wrapper, from torch's allocator): a captured call shares K like the eager one,
    and every replay returns the eager call's bits."""
    rng = np.random.default_rng(5)
    m, n, k = 128, 256, 8192
    layer = make_layer(rng, n, k, 4, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    library_switch("OQ_GEMM_WG_SPLIT", "1")
    single = run_packed_linear(dev, layer, codes, s, "nibble")
    library_switch("OQ_GEMM_WG_SPLIT", "8")
    split = run_packed_linear(dev, layer, codes, s, "nibble")
    assert not torch.equal(split, single)          # the eager call does share K here
    from orbitquant_amd import ops
    args = (torch.from_numpy(o.pack_nibbles(codes)).to(dev), torch.from_numpy(s).to(dev), torch.from_numpy(layer["ca"]).to(dev),
            torch.from_numpy(layer["packed"]).to(dev), layer["r"].to(dev), torch.from_numpy(layer["cw"]).to(dev))
    kw = dict(code_format="nibble", activation_bits=4, weight_bits=4, out_features=n, in_features=k,
              bias=torch.from_numpy(layer["bias"]).to(torch.bfloat16).to(dev), output_dtype=torch.bfloat16)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.packed_linear(*args, **kw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ops.packed_linear(*args, **kw)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, split)
        assert torch.equal(ops.packed_linear(*args, **kw), split)   # eager work between the replays


def test_workspace_is_the_callers_and_optional(dev, library_switch):
    """The C ABI allocates nothing.  Without a workspace (NULL, or one that is too small) oq_packed_linear is the
    single launch and oq_matmul_packed_weight stages activation rows through LDS; with the bytes the query
    functions name they share K between workgroups / read an operand-order copy.  Same results as the wrapper's."""
    from orbitquant_amd import _lib, ops

    lib = _lib.load()
    rng = np.random.default_rng(6)
    m, n, k = 128, 256, 8192
    layer = make_layer(rng, n, k, 4, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    library_switch("OQ_GEMM_WG_SPLIT", "1")
    single = run_packed_linear(dev, layer, codes, s, "nibble")
    library_switch("OQ_GEMM_WG_SPLIT", "8")
    split = run_packed_linear(dev, layer, codes, s, "nibble")
    t = dict(codes=torch.from_numpy(o.pack_nibbles(codes)).to(dev), s=torch.from_numpy(s).to(dev), ca=torch.from_numpy(layer["ca"]).to(dev),
             packed=torch.from_numpy(layer["packed"]).to(dev), r=layer["r"].to(dev), cw=torch.from_numpy(layer["cw"]).to(dev),
             bias=torch.from_numpy(layer["bias"]).to(torch.bfloat16).to(dev))
    need = int(lib.oq_packed_linear_workspace_bytes(m, n, k, 4, 1, 4))
    assert need == m * n * 4 * 8
    out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)

    def call(ws_ptr, ws_bytes):
        rc = lib.oq_packed_linear(t["codes"].data_ptr(), 1, t["s"].data_ptr(), t["ca"].data_ptr(), 4, t["packed"].data_ptr(), 4,
                                  t["r"].data_ptr(), t["cw"].data_ptr(), t["bias"].data_ptr(), 2, m, n, k, out.data_ptr(), 2,
                                  ws_ptr, ws_bytes, None)
        torch.cuda.synchronize()
        assert rc == 0
        return out.clone()
    assert torch.equal(call(None, 0), single)
    assert torch.equal(call(ws.data_ptr(), need - 1), single)        # too small: not used
    assert torch.equal(call(ws.data_ptr(), need), split)
    assert lib.oq_packed_linear_workspace_bytes(16, n, k, 4, 1, 4) == 0   # the streaming kernel needs none

    # float activations: the operand-order copy lives in the workspace; without one, the LDS-staged kernel, same sums
    m2, n2, k2 = 520, 200, 1152
    layer2 = make_layer(rng, n2, k2, 3, 4)
    x = torch.from_numpy(rng.standard_normal((m2, k2)).astype(F32)).to(torch.bfloat16).to(dev)
    packed, r, cw = torch.from_numpy(layer2["packed"]).to(dev), layer2["r"].to(dev), torch.from_numpy(layer2["cw"]).to(dev)
    want = ops.matmul_packed_weight_values(x, packed, r, cw, bits=3, out_features=n2, in_features=k2)
    need2 = int(lib.oq_matmul_packed_weight_workspace_bytes(m2, n2, k2, 3, 2))
    assert need2 == ((m2 + 31) // 32) * (k2 // 64) * 256 * 16
    out2 = torch.empty(m2, n2, dtype=torch.bfloat16, device=dev)
    ws2 = torch.empty(need2, dtype=torch.uint8, device=dev)
    for ws_ptr, ws_bytes in ((None, 0), (ws2.data_ptr(), need2), (ws2.data_ptr(), 64)):
        out2.zero_()
        rc = lib.oq_matmul_packed_weight(x.data_ptr(), 2, None, packed.data_ptr(), 3, r.data_ptr(), cw.data_ptr(), None, 0,
                                         m2, n2, k2, out2.data_ptr(), 2, ws_ptr, ws_bytes, None)
        torch.cuda.synchronize()
        assert rc == 0 and torch.equal(out2, want)


def test_packed_linear_chooses_shared_k_for_short_and_long_problems(dev):
    """The dispatcher's own choice on a short-and-long problem (few tiles, many K-steps) against the oracle."""
    rng = np.random.default_rng(77)
    m, n, k = 128, 512, 14336
    layer = make_layer(rng, n, k, 4, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16)
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    got = run_packed_linear(dev, layer, codes, s, "nibble")
    check_outputs(got, oracle_linear(layer, codes, s, torch.bfloat16), s, layer["r"].float().numpy(), k, "dispatcher's choice")


@pytest.mark.parametrize("m", [1, 4, 16, 3])
@pytest.mark.parametrize(("n", "k", "wbits"), [(4096, 4096, 2), (1000, 4096, 3), (4096, 14336, 3), (2048, 4096, 4), (512, 1152, 6), (256, 1024, 8)])
def test_packed_linear_small_m_stream_kernel(dev, m, n, k, wbits):
    rng = np.random.default_rng(m + n + k + wbits)
    layer = make_layer(rng, n, k, wbits, 4)
    _, x32 = make_x(rng, m, k, torch.bfloat16, kind="plain")
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, torch.bfloat16)
    got = run_packed_linear(dev, layer, codes, s, "nibble")
    check_outputs(got, want, s, layer["r"].float().numpy(), k, "small-M")
    again = run_packed_linear(dev, layer, codes, s, "nibble")
    assert torch.equal(got, again)      # fixed summation order: run-to-run identical


@pytest.mark.parametrize("m", [1, 16])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize(("n", "k", "wbits"), [(64, 128, 4), (40, 256, 3), (100, 384, 2), (4104, 640, 4), (24, 1408, 4)])
def test_packed_linear_small_m_short_rows(dev, m, n, k, wbits, with_bias, out_dtype):
    """Rows of one to eleven K-steps: some wavefronts of a workgroup own no K-step at all, others an
    odd number; bias absent, 16-bit and 32-bit (the kernel requests it long before it is used)."""
    rng = np.random.default_rng(m + n + k + wbits)
    layer = make_layer(rng, n, k, wbits, 4, with_bias=with_bias)
    _, x32 = make_x(rng, m, k, torch.bfloat16, kind="plain")
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, out_dtype)
    got = run_packed_linear(dev, layer, codes, s, "nibble", out_dtype)
    check_outputs(got, want, s, layer["r"].float().numpy(), k, "small-M short rows")
    assert torch.equal(got, run_packed_linear(dev, layer, codes, s, "nibble", out_dtype))


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize(("n", "k", "wbits", "abits"), [(2048, 4096, 4, 6), (1000, 1024, 3, 8), (512, 1152, 6, 5), (4096, 4096, 2, 7)])
def test_packed_linear_small_m_byte_codes(dev, m, n, k, wbits, abits):
    """Decode-sized inputs with activation codes wider than 4 bits (one code per byte)."""
    rng = np.random.default_rng(m + n + k + wbits + abits)
    layer = make_layer(rng, n, k, wbits, abits)
    _, x32 = make_x(rng, m, k, torch.bfloat16, kind="plain")
    codes, s = oracle_c.rotate_quantize(x32, layer["perm"], layer["signs"], layer["ba"], layer["block"], 1e-10, layer["inv"])
    want = oracle_linear(layer, codes, s, torch.bfloat16)
    got = run_packed_linear(dev, layer, codes, s, "u8")
    check_outputs(got, want, s, layer["r"].float().numpy(), k, "small-M byte codes")
    assert torch.equal(got, run_packed_linear(dev, layer, codes, s, "u8"))


# ------------------------------------------------- float-activation packed matmul

def _pack_loop(values, bits):
    out = bytearray((len(values) * bits + 7) // 8)
    for i, v in enumerate(values):
        start = i * bits
        out[start // 8] |= (v << (start % 8)) & 0xFF
        if start % 8 + bits > 8:
            out[start // 8 + 1] |= v >> (8 - start % 8)
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


@pytest.mark.parametrize("bits", [2, 3, 4, 6])
@pytest.mark.parametrize(("rows", "k", "n"), [(9, 16, 7), (9, 19, 7), (15, 37, 29), (65, 64, 70), (1, 32, 32)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_matmul_packed_weight_reference_vectors(dev, bits, rows, k, n, dtype):
    """Vectors of the reference's native tests (tests/test_packed_matmul.py:365-452,567-602 of
    the native package): indices = arange % 2^b, centroids = linspace(-1, 1),
    row_norms = linspace(0.5, 1.5), tolerance 2e-2 (3e-2 for bf16)."""
    from orbitquant_amd import ops

    torch.manual_seed(1000 + bits * 100 + rows * 10 + k + n)
    x = torch.randn(rows, k).to(dtype)
    idx = (np.arange(n * k) % (1 << bits)).astype(np.uint8)
    packed = _pack_loop(idx.tolist(), bits)
    r = torch.linspace(0.5, 1.5, n).to(torch.bfloat16)
    cents = torch.linspace(-1.0, 1.0, 1 << bits)
    bias = torch.randn(n).to(dtype)
    w = r.float()[:, None] * cents[torch.from_numpy(idx.reshape(n, k)).long()]
    want = torch.nn.functional.linear(x.float(), w, bias.float())
    got = ops.matmul_packed_weight_values(
        x.to(dev), torch.from_numpy(packed).to(dev), r.to(dev), cents.to(dev), bits=bits,
        out_features=n, in_features=k, bias=bias.to(dev))
    assert got.dtype == dtype and tuple(got.shape) == (rows, n)
    tol = 3e-2 if dtype == torch.bfloat16 else 2e-2
    assert torch.allclose(got.float().cpu(), want, atol=tol, rtol=tol)


def test_matmul_packed_weight_mfma_path_realistic(dev):
    from orbitquant_amd import ops

    rng = np.random.default_rng(77)
    m, n, k = 333, 1536, 1536
    layer = make_layer(rng, n, k, 4, 4)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(F32)).to(torch.bfloat16)
    got = ops.matmul_packed_weight_values(
        x.to(dev), torch.from_numpy(layer["packed"]).to(dev), layer["r"].to(dev),
        torch.from_numpy(layer["cw"]).to(dev), bits=4, out_features=n, in_features=k,
        bias=torch.from_numpy(layer["bias"]).to(torch.bfloat16).to(dev))
    bias = torch.from_numpy(layer["bias"]).to(torch.bfloat16).float().numpy()
    want = o.matmul_packed_weight_f32(x.float().numpy(), layer["packed"], layer["r"].float().numpy(), layer["cw"], 4, n, bias)
    s = np.linalg.norm(x.float().numpy(), axis=1)
    check_outputs(got, want, s, layer["r"].float().numpy(), k, "float-activation MFMA")


# ------------------------------------------------------------------ whole module

@pytest.mark.parametrize(("name", "k", "n", "m", "dtype"), [
    ("w4a4", 1152, 1152, 256, torch.float32),
    ("w3a3", 3072, 512, 200, torch.bfloat16),
    ("w2a4", 4096, 1024, 4, torch.bfloat16),
    ("w2a3", 1024, 256, 40, torch.bfloat16),
    ("w4a6", 5120, 384, 100, torch.bfloat16),
])
def test_orbit_linear_end_to_end(dev, name, k, n, m, dtype):
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(5)
    cfg = recipe(name)
    lin = torch.nn.Linear(k, n)
    with torch.no_grad():
        lin.weight.mul_(0.6)
    layer = OrbitLinear.from_linear(lin, config=cfg).to(dev)
    assert sorted(layer.state_dict().keys()) == ["bias", "packed_weight_indices", "row_norms"]
    x = torch.randn(2, m // 2, k).to(dtype)
    x[0, 0] = 0
    y = layer(x.to(dev))
    assert y.dtype == dtype and tuple(y.shape) == (2, m // 2, n)

    perm, signs, block, inv = o.rpbh_constants(k, 0)
    ca, ba = tables(k, cfg.activation_bits)
    cw, _ = tables(k, cfg.weight_bits)
    x32 = x.reshape(-1, k).float().numpy()
    codes, s = oracle_c.rotate_quantize(x32, perm, signs, ba, block, 1e-10, inv)
    packed = layer.packed_weight_indices.cpu().numpy()
    r = layer.row_norms.float().cpu().numpy()
    bias = lin.bias.detach().to(dtype).float().numpy()
    want = oracle_c.linear_from_codes(codes, s, ca, packed, cfg.weight_bits, r, cw, bias, n)
    check_outputs(y.reshape(-1, n), want, s, r, k, name)
    assert np.array_equal(y[0, 0].float().cpu().numpy(), bias)

    # the weights the module holds are the oracle's (offline quantization parity)
    w_packed, w_r, _ = o.quantize_weight(lin.weight.detach().numpy(), perm, signs, tables(k, cfg.weight_bits)[1], block, 1e-10, cfg.weight_bits)
    assert np.array_equal(packed, w_packed) and torch.equal(layer.row_norms.cpu(), w_r)


def test_orbit_linear_torch_compile_fullgraph(dev):
    # tests/test_torch_compile.py:30-90 of the reference: compiled == eager exactly
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(9)
    layer = OrbitLinear.from_linear(torch.nn.Linear(512, 256), config=recipe("w4a4")).to(dev)
    x = torch.randn(3, 20, 512, dtype=torch.bfloat16, device=dev)
    eager = layer(x)
    compiled = torch.compile(layer, fullgraph=True)
    assert torch.equal(compiled(x), eager)


def test_state_dict_roundtrip(dev):
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(3)
    cfg = recipe("w3a3")
    a = OrbitLinear.from_linear(torch.nn.Linear(256, 128), config=cfg).to(dev)
    b = OrbitLinear.from_linear(torch.nn.Linear(256, 128), config=cfg).to(dev)
    b.load_state_dict(a.state_dict(), strict=True)
    x = torch.randn(17, 256, dtype=torch.bfloat16, device=dev)
    assert torch.equal(a(x), b(x))


# -------------------------------------------- drop-in package (reference API names)

@pytest.mark.parametrize(("dim", "threads"), [(512, 128), (4096, 256), (16384, 512)])
def test_dropin_quantize_activations_packed_w4_and_int8(dev, dim, threads):
    """Reference native tests (tests/test_packed_matmul.py:773-821 of the native package):
    the int8 form equals codes[index] of the packed form, norms identical."""
    import orbitquant_packed_matmul as pkg

    torch.manual_seed(dim)
    x = torch.randn((2, dim), dtype=torch.bfloat16)
    perm = torch.randperm(dim)
    signs = torch.where(torch.arange(dim) % 2 == 0, 1, -1).to(torch.int8)
    bounds = torch.linspace(-0.2, 0.2, 15)
    codes = torch.tensor([-120, -92, -68, -49, -34, -22, -12, -4, 4, 12, 22, 34, 49, 68, 92, 120], dtype=torch.int8)
    kw = dict(eps=1e-12, inv_sqrt_block=dim ** -0.5, threads=threads)
    packed, norms = pkg.quantize_activations_packed_w4(x.to(dev), perm.to(dev), signs.to(dev), bounds.to(dev), **kw)
    q8, norms8 = pkg.quantize_activations_int8(x.to(dev), perm.to(dev), signs.to(dev), bounds.to(dev), codes.to(dev), **kw)
    assert packed.dtype == torch.uint8 and tuple(packed.shape) == (2, dim // 2) and tuple(norms.shape) == (2,)
    idx = torch.empty((2, dim), dtype=torch.long, device=dev)
    idx[:, 0::2] = packed & 15
    idx[:, 1::2] = packed >> 4
    assert torch.equal(q8, codes.to(dev)[idx]) and torch.equal(norms8, norms)
    want_codes, want_norms = oracle_c.rotate_quantize(x.float().numpy(), perm.numpy(), signs.numpy(), bounds.numpy(), dim, 1e-12, F32(dim ** -0.5))
    assert np.array_equal(packed.cpu().numpy(), o.pack_nibbles(want_codes))
    assert np.array_equal(norms.cpu().numpy(), want_norms)
    # int32 and int64 permutations give the same result (tests/test_packed_matmul.py:736-770)
    packed32, _ = pkg.quantize_activations_packed_w4(x.to(dev), perm.to(torch.int32).to(dev), signs.to(dev), bounds.to(dev), **kw)
    assert torch.equal(packed32, packed)


@pytest.mark.parametrize(("rows", "out_features"), [(128, 128), (256, 128), (130, 258)])
def test_dropin_matmul_packed_w4a4_int8_exact_integer_reference(dev, rows, out_features):
    # reference native tests/test_packed_matmul.py:605-685: fixed int8 code table, scales 0.005
    import orbitquant_packed_matmul as pkg

    k = 256
    torch.manual_seed(0)
    a_idx = torch.randint(0, 16, (rows, k), dtype=torch.uint8)
    w_idx = torch.randint(0, 16, (out_features, k), dtype=torch.uint8)
    pa = (a_idx[:, 0::2] | (a_idx[:, 1::2] << 4)).contiguous()
    pw = (w_idx[:, 0::2] | (w_idx[:, 1::2] << 4)).contiguous()
    codes = torch.tensor([-104, -79, -62, -48, -36, -25, -15, -5, 5, 15, 25, 36, 48, 62, 79, 104], dtype=torch.int8)
    tn = torch.linspace(0.5, 1.0, rows)
    rn = torch.linspace(0.5, 1.5, out_features).to(torch.bfloat16)
    got = pkg.matmul_packed_w4a4_int8(pa.to(dev), pw.to(dev), tn.to(dev), rn.to(dev), codes.to(dev), codes.to(dev),
                                      activation_scale=0.005, weight_scale=0.005, out_features=out_features, in_features=k)
    ref = codes[a_idx.long()].float() @ codes[w_idx.long()].float().T
    ref = ref * tn[:, None] * rn.float()[None, :] * (0.005 * 0.005)
    assert got.dtype == torch.bfloat16
    assert torch.allclose(got.float().cpu(), ref, atol=0.25, rtol=1e-2)


def test_dropin_matmul_packed_weight_rows_1536(dev):
    # reference native tests/test_packed_matmul.py:222-279: realistic 1536 rows 16/24/32/33
    import orbitquant_packed_matmul as pkg

    rng = np.random.default_rng(1536)
    layer = make_layer(rng, 1536, 1536, 4, 4)
    for rows in (16, 24, 32, 33):
        x = torch.from_numpy(rng.standard_normal((rows, 1536)).astype(F32)).to(torch.bfloat16)
        got = pkg.matmul_packed_weight(x.to(dev), torch.from_numpy(layer["packed"]), layer["r"], torch.from_numpy(layer["cw"]),
                                       bits=4, out_features=1536, in_features=1536)
        want = o.matmul_packed_weight_f32(x.float().numpy(), layer["packed"], layer["r"].float().numpy(), layer["cw"], 4, 1536)
        s = np.linalg.norm(x.float().numpy(), axis=1)
        check_outputs(got, want, s, layer["r"].float().numpy(), 1536, f"rows {rows}")


@pytest.mark.parametrize("bits", [2, 3, 4, 6, 8])
@pytest.mark.parametrize(("m", "n", "k"), [(300, 200, 256), (512, 1152, 4608), (257, 96, 64), (2048, 384, 1152)])
def test_matmul_packed_weight_large_m_bf16(dev, bits, m, n, k, library_switch):
    """bf16 activations take the operand-order pass + tile kernel: against the oracle, and
    bit for bit against the code kernel fed with the codes whose centroids are those activations (both as
    one launch over all of K: the code kernel would share K between workgroups on some of these shapes)."""
    from orbitquant_amd import ops

    library_switch("OQ_GEMM_WG_SPLIT", "1")

    rng = np.random.default_rng(bits * 7 + m)
    layer = make_layer(rng, n, k, bits, 4)
    ca = torch.from_numpy(layer["ca"]).to(torch.bfloat16)             # sixteen bf16 values
    codes = rng.integers(0, 16, size=(m, k), dtype=np.uint8)
    x = ca[torch.from_numpy(codes).long()] if m != 300 else torch.from_numpy(rng.standard_normal((m, k)).astype(F32)).to(torch.bfloat16)
    scale = torch.from_numpy(rng.uniform(0.5, 2.0, m).astype(F32))
    bias = torch.from_numpy(layer["bias"]).to(torch.bfloat16)
    args = dict(bits=bits, out_features=n, in_features=k, bias=bias.to(dev), token_scale=scale.to(dev))
    got = ops.matmul_packed_weight_values(x.to(dev), torch.from_numpy(layer["packed"]).to(dev), layer["r"].to(dev),
                                          torch.from_numpy(layer["cw"]).to(dev), **args)
    want = o.matmul_packed_weight_f32(x.float().numpy(), layer["packed"], layer["r"].float().numpy(), layer["cw"], bits, n, None)
    want = want * scale.numpy()[:, None] + bias.float().numpy()[None, :]
    s = np.linalg.norm(x.float().numpy(), axis=1) * scale.numpy()
    check_outputs(got, want, s, layer["r"].float().numpy(), k, f"large-M float activations W{bits}")
    if m != 300:
        nib = torch.from_numpy((codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8))
        by_codes = ops.packed_linear(nib.to(dev), scale.to(dev), torch.from_numpy(layer["ca"]).to(dev), torch.from_numpy(layer["packed"]).to(dev),
                                     layer["r"].to(dev), torch.from_numpy(layer["cw"]).to(dev), code_format="nibble", activation_bits=4,
                                     weight_bits=bits, out_features=n, in_features=k, bias=bias.to(dev), output_dtype=torch.bfloat16)
        assert torch.equal(got, by_codes)


@pytest.mark.parametrize("bits,m", [(2, 520), (3, 520), (4, 520), (6, 520), (8, 520), (4, 3), (3, 40), (2, 130)])
def test_matmul_packed_weight_large_m_bf16_under_graph_capture(dev, bits, m):
    """The float-activation call on bf16 values under stream capture: the wrapper's workspace comes from the
    graph's memory pool, the call takes the kernels the eager call takes, and the replayed graph returns
    the bits of the eager call, replay after replay."""
    from orbitquant_amd import ops

    rng = np.random.default_rng(bits + m)
    n, k = 200, 1152
    layer = make_layer(rng, n, k, bits, 4)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(F32)).to(torch.bfloat16).to(dev)
    packed, r, cw = torch.from_numpy(layer["packed"]).to(dev), layer["r"].to(dev), torch.from_numpy(layer["cw"]).to(dev)
    scale = torch.from_numpy(rng.uniform(0.5, 2.0, m).astype(F32)).to(dev)

    def call():
        return ops.matmul_packed_weight_values(x, packed, r, cw, bits=bits, out_features=n, in_features=k, token_scale=scale)
    eager = call()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call()
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        assert torch.equal(call(), eager)   # eager work between the replays
