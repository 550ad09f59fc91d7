"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each test checks the oracle against something it did not produce: a vector held
by the reference's own tests, a closed form, a brute-force evaluation, a library
routine, or an invariant.  Reference locations are given per test
(paths relative to the reference checkout).
"""

from __future__ import annotations

import hashlib
import json
import math

import numpy as np
import pytest
import torch

from oracle import oracle_c, oracle_np as o

F32 = np.float32


# ------------------------------------------------------------------ codebooks

# tests/test_codebooks.py:39-65 (golden dim=32, bits=3, tolerance 1e-6)
GOLDEN_32_3_CENTROIDS = [-0.36626825, -0.23246057, -0.13175610, -0.04285152,
                         0.04285152, 0.13175610, 0.23246057, 0.36626825]
GOLDEN_32_3_BOUNDARIES = [-0.29936442, -0.18210834, -0.08730381, 0.0,
                          0.08730381, 0.18210834, 0.29936442]


def test_codebook_matches_reference_golden_dim32_bits3():
    cents, bounds = o.lloyd_max_tables(32, 3)
    assert np.abs(cents - np.array(GOLDEN_32_3_CENTROIDS, F32)).max() <= 1e-6
    assert np.abs(bounds - np.array(GOLDEN_32_3_BOUNDARIES, F32)).max() <= 1e-6


def _trapezoid_interval_mean(dim, left, right):
    # independent of the incomplete-beta route (tests/test_paper_reference_oracle.py:76-83)
    grid = np.linspace(left, right, 20001)
    density = np.clip(1 - grid * grid, 0, None) ** ((dim - 3) / 2)
    return np.trapezoid(grid * density, grid) / np.trapezoid(density, grid)


@pytest.mark.parametrize("bits", [2, 3, 4, 6])
def test_codebook_is_lloyd_max_fixed_point_by_numeric_integration(bits):
    # tests/test_paper_reference_oracle.py:399-425 (dim=64, tol 2e-6 / 2e-8)
    cents, bounds = o.lloyd_max_tables(64, bits)
    c64 = cents.astype(np.float64)
    assert np.abs(bounds - ((c64[:-1] + c64[1:]) / 2)).max() <= 2e-8
    assert np.array_equal(cents, -cents[::-1])
    edges = np.concatenate(([-1.0], (c64[:-1] + c64[1:]) / 2, [1.0]))
    means = [_trapezoid_interval_mean(64, edges[i], edges[i + 1]) for i in range(c64.size)]
    assert np.abs(np.array(means) - c64).max() <= 2e-6


def test_codebook_lloyd_condition_dim128_bits6():
    # tests/test_codebooks.py:105-128 (1e-7)
    cents, _ = o.lloyd_max_tables(128, 6)
    pos = cents[32:].astype(np.float64)
    edges = np.concatenate(([0.0], (pos[:-1] + pos[1:]) / 2, [1.0]))
    means = [_trapezoid_interval_mean(128, edges[i], edges[i + 1]) for i in range(pos.size)]
    assert np.abs(np.array(means) - pos).max() <= 1e-7


def test_codebook_tables_against_reference_generated_fixture(golden_dir):
    """fp32 bit patterns written by tests/golden/make_codebook_golden.py from the
    reference generator.  Bits 2/3/4: identical.  Bits 6: the reference stops its
    iteration ~1e-12 short of the fixed point, so an independent solver may differ
    by one fp32 ulp in a few entries; more than one ulp anywhere is a failure."""
    tables = json.loads((golden_dir / "codebooks_v2.json").read_text())["tables"]
    for dim in (24, 1152, 3072, 4096, 5120, 14336):
        for bits in (2, 3, 4, 6):
            want = tables[f"dim{dim}_bits{bits}"]
            wc = np.array(want["centroids_u32"], dtype=np.int32).view(F32)
            wb = np.array(want["boundaries_u32"], dtype=np.int32).view(F32)
            cents, bounds = o.lloyd_max_tables(dim, bits)
            if bits < 6:
                assert np.array_equal(cents, wc) and np.array_equal(bounds, wb), (dim, bits)
            else:
                ulp_c = np.abs(cents.view(np.int32) - wc.view(np.int32)).max()
                ulp_b = np.abs(bounds.view(np.int32) - wb.view(np.int32)).max()
                assert ulp_c <= 1 and ulp_b <= 1, (dim, bits, ulp_c, ulp_b)


# ------------------------------------------------------------------- rotation

def test_paper_block_table():
    # tests/test_paper_methodology.py:101-117, tests/test_rpbh.py:77-81
    table = {1536: 512, 3072: 1024, 3840: 256, 8960: 256, 9216: 1024, 10240: 2048,
             12288: 4096, 15360: 1024, 24: 8}
    for dim, block in table.items():
        assert o.paper_block(dim) == block


def test_rotation_draws_match_fixture(golden_dir):
    draws = json.loads((golden_dir / "rotations.json").read_text())["draws"]
    for key, want in draws.items():
        dim = int(key.split("_")[0][3:])
        seed = int(key.split("seed")[1])
        perm, signs, _, _ = o.rpbh_constants(dim, seed)
        assert hashlib.sha256(perm.astype("<i8").tobytes()).hexdigest() == want["perm_sha256"]
        assert hashlib.sha256(signs.astype("i1").tobytes()).hexdigest() == want["signs_sha256"]
        assert perm[:16].tolist() == want["perm_head"]
        assert sorted(perm.tolist()) == list(range(dim))
        assert set(signs.tolist()) <= {-1, 1}


def test_rotation_explicit_h4():
    # tests/test_rpbh.py:31-50: dim=8, seed=5, block=4, explicit 4x4 Hadamard
    perm, signs, block, inv = o.rpbh_constants(8, 5, 4)
    x = (np.arange(16, dtype=F32).reshape(2, 8) - 3).astype(F32)
    h4 = np.array([[1, 1, 1, 1], [1, -1, 1, -1], [1, 1, -1, -1], [1, -1, -1, 1]], F32)
    signed = x[:, perm] * signs.astype(F32)
    expected = (signed.reshape(2, 2, 4) @ h4.T * F32(0.5)).reshape(2, 8)
    assert np.array_equal(o.rotate(x, perm, signs, block, inv), expected)


def _dense_rotation(perm, signs, block):
    # tests/test_paper_reference_oracle.py:15-42: P^T . D . H_block, built densely
    dim = perm.size
    gather = np.zeros((dim, dim))
    gather[perm, np.arange(dim)] = 1
    h = o.hadamard_dense(block) / math.sqrt(block)
    blocks = np.kron(np.eye(dim // block), h)
    return gather @ np.diag(signs.astype(np.float64)) @ blocks


@pytest.mark.parametrize(("dim", "seed", "block"), [(24, 17, "paper"), (16, 7, 8), (64, 3, 64), (96, 1, 32)])
def test_rotation_matches_dense_matrix(dim, seed, block):
    perm, signs, block, inv = o.rpbh_constants(dim, seed, block)
    rng = np.random.default_rng(101)
    x = rng.standard_normal((5, dim)).astype(F32)
    dense = _dense_rotation(perm, signs, block)
    got = o.rotate(x, perm, signs, block, inv)
    assert np.abs(got - x.astype(np.float64) @ dense).max() <= 2e-6
    # orthogonal: norm preserving, and linear(xR, WR) == linear(x, W) (tests/test_rpbh.py:6-16,53-65)
    assert np.abs(dense @ dense.T - np.eye(dim)).max() <= 1e-12
    w = rng.standard_normal((7, dim)).astype(F32)
    folded = got.astype(np.float64) @ o.rotate(w, perm, signs, block, inv).astype(np.float64).T
    assert np.abs(folded - x.astype(np.float64) @ w.astype(np.float64).T).max() <= 1e-4


def test_fwht_matches_brute_force_hadamard_exactly_on_integers():
    # integer inputs: every partial sum is exact in fp32, so equality is exact
    rng = np.random.default_rng(0)
    for n in (1, 2, 8, 64, 256):
        x = rng.integers(-50, 50, size=(3, n)).astype(F32)
        assert np.array_equal(o.fwht_np(x), (x.astype(np.float64) @ o.hadamard_dense(n)).astype(F32))


def test_fwht_stage_order_low_distance_first():
    # With non-associative fp32 inputs the stage order is observable: compare with
    # an explicit per-stage evaluation written from rotations/fwht.py:19-25.
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(16) * np.array([1e8, 1, 1e-8, 1] * 4)).astype(F32)
    y = x.copy()
    d = 1
    while d < 16:
        nxt = np.empty_like(y)
        for j in range(16):
            nxt[j] = y[j] + y[j + d] if (j & d) == 0 else y[j - d] - y[j]
        y = nxt
        d *= 2
    assert np.array_equal(o.fwht_np(x[None])[0], y)


# ------------------------------------------------------------ bucketize, bits

def test_bucketize_ties_go_low_and_equal_nearest_centroid():
    # tests/test_kernels.py:689-702 (values exactly on boundaries);
    # tests/test_paper_reference_oracle.py:45-51 (exhaustive argmin)
    cents, bounds = o.lloyd_max_tables(64, 4)
    assert o.bucketize(bounds, bounds).tolist() == list(range(15))
    above = np.nextafter(bounds, F32(np.inf))
    assert o.bucketize(above, bounds).tolist() == list(range(1, 16))
    rng = np.random.default_rng(3)
    v = (rng.standard_normal(20000) * 0.15).astype(F32)
    nearest = np.abs(v[:, None].astype(np.float64) - cents[None, :].astype(np.float64)).argmin(axis=1)
    assert np.array_equal(o.bucketize(v, bounds), nearest.astype(np.uint8))
    assert np.array_equal(o.bucketize(v, bounds), torch.bucketize(torch.from_numpy(v), torch.from_numpy(bounds)).numpy().astype(np.uint8))


def _pack_loop(values, bits):
    # independent writer: one value at a time (native tests/test_packed_matmul.py:20-30)
    out = bytearray((len(values) * bits + 7) // 8)
    for i, v in enumerate(values):
        start = i * bits
        out[start // 8] |= (v << (start % 8)) & 0xFF
        if start % 8 + bits > 8:
            out[start // 8 + 1] |= v >> (8 - start % 8)
    return np.frombuffer(bytes(out), dtype=np.uint8)


def _unpack_loop(payload, bits, count):
    # independent reader (tests/test_paper_reference_oracle.py:54-73)
    data = list(payload) + [0]
    vals = []
    for i in range(count):
        off = i * bits
        word = data[off // 8] | (data[off // 8 + 1] << 8)
        vals.append((word >> (off % 8)) & ((1 << bits) - 1))
    return np.array(vals, dtype=np.uint8)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_bitstream_pack_unpack_against_loop_reader_writer(bits):
    # tests/test_kernels.py:810-824 vector: arange(1027)*3 % 2^bits
    values = (np.arange(1027) * 3 % (1 << bits)).astype(np.uint8)
    packed = o.pack_bits(values, bits)
    assert np.array_equal(packed, _pack_loop(values.tolist(), bits))
    assert np.array_equal(o.unpack_bits(packed, bits, 1027), values)
    assert np.array_equal(_unpack_loop(packed.tolist(), bits, 1027), values)
    assert np.array_equal(oracle_c.unpack(packed, bits, 1027), values)


def test_bitstream_known_bytes():
    # 3-bit values 1,2,3,4,5 -> bits: 001 010 011 100 101 (LSB first per value)
    # stream (value i at bit 3i): byte0 = 1 | 2<<3 | (3&3)<<6 = 0xD1, byte1 = 3>>2 | 4<<1 | 5<<4 = 0x58
    assert o.pack_bits([1, 2, 3, 4, 5], 3).tolist() == [0xD1, 0x58]
    assert o.pack_bits([0xA, 0x5, 0xF], 4).tolist() == [0x5A, 0x0F]
    assert o.pack_bits([3, 0, 1, 2], 2).tolist() == [0b10010011]


def test_bitstream_long_roundtrip():
    # tests/test_bitpack.py:6-25 sizes (100 003 values)
    rng = np.random.default_rng(9)
    for bits in (2, 3, 4, 6):
        values = rng.integers(0, 1 << bits, size=100003).astype(np.uint8)
        assert np.array_equal(o.unpack_bits(o.pack_bits(values, bits), bits, values.size), values)


# ---------------------------------------------------- activation quantization

def test_sumsq_order_is_close_to_exact_and_c_matches_numpy():
    rng = np.random.default_rng(11)
    for k in (1, 7, 24, 1152, 2048, 2049, 5120, 14336):
        x = rng.standard_normal((4, k)).astype(F32)
        got = o.sumsq_v1(x)
        exact = (x.astype(np.float64) ** 2).sum(axis=1)
        assert np.abs(got - exact).max() <= 4e-7 * exact.max()
        assert np.abs(o.token_norms(x) - torch.from_numpy(x).norm(dim=-1).numpy()).max() <= 2e-6 * np.sqrt(exact.max())


def test_sumsq_small_hand_case():
    # 9 elements: lanes 0 and 1 hold data; lane 0: ((1+4)+(9+16))+((25+36)+(49+64)) = 204, lane 1: 81
    x = np.arange(1, 10, dtype=F32)[None]
    assert o.sumsq_v1(x)[0] == F32(285.0)


@pytest.mark.parametrize("dim", [512, 4096])
def test_activation_codes_one_hot_closed_form(dim):
    """native tests/test_packed_matmul.py:688-733: one-hot rows, alternating signs,
    boundaries = linspace(-0.2, 0.2, 15), full-row block.  For a one-hot row the
    rotated vector is one row of the Hadamard matrix: value(j) = sign * v/|v| *
    (-1)^popcount(c & j) / sqrt(dim), with c the slot the hot input is gathered to."""
    gen = torch.Generator().manual_seed(dim)
    perm = torch.randperm(dim, generator=gen).numpy()
    signs = np.where(np.arange(dim) % 2 == 0, 1, -1).astype(np.int8)
    bounds = np.linspace(-0.2, 0.2, 15, dtype=F32)
    x = np.zeros((2, dim), F32)
    x[0, 3] = 1
    x[1, dim - 7] = -1
    inv = F32(dim ** -0.5)
    codes, norms = o.quantize_codes(x, perm, signs, bounds, dim, 1e-12, inv)
    assert norms.tolist() == [1.0, 1.0]
    for row, (hot, val) in enumerate(((3, 1.0), (dim - 7, -1.0))):
        c = int(np.nonzero(perm == hot)[0][0])
        parity = np.array([bin(c & j).count("1") & 1 for j in range(dim)])
        rot = (np.where(parity == 1, -1.0, 1.0) * val * signs[c]).astype(F32) * inv
        want = np.array([(bounds < v).sum() for v in rot], dtype=np.uint8)
        assert np.array_equal(codes[row], want)
    c_codes, c_norms = oracle_c.rotate_quantize(x, perm, signs, bounds, dim, 1e-12, inv)
    assert np.array_equal(c_codes, codes) and np.array_equal(c_norms, norms)


@pytest.mark.parametrize(("dim", "block", "bits"), [(24, 8, 4), (1152, 64, 4), (3072, 1024, 3), (4608, 512, 6), (4096, 4096, 4)])
def test_c_oracle_equals_numpy_oracle_bit_for_bit(dim, block, bits):
    perm, signs, block, inv = o.rpbh_constants(dim, 0, block)
    _, bounds = o.lloyd_max_tables(dim, bits)
    rng = np.random.default_rng(dim + bits)
    x = rng.standard_normal((9, dim)).astype(F32)
    x[rng.random(x.shape) < 0.01] *= 20
    x[2] = 0
    codes, norms = o.quantize_codes(x, perm, signs, bounds, block, 1e-10, inv)
    c_codes, c_norms = oracle_c.rotate_quantize(x, perm, signs, bounds, block, 1e-10, inv)
    assert np.array_equal(codes, c_codes)
    assert np.array_equal(norms.view(np.int32), c_norms.view(np.int32))


def test_activation_quantization_invariants():
    # tests/test_kernels.py:68-122: scale equivariance, batch independence, zero token
    dim, block = 96, 32
    perm, signs, block, inv = o.rpbh_constants(dim, 4, block)
    cents, bounds = o.lloyd_max_tables(dim, 4)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((6, dim)).astype(F32)
    x[4] = 0
    codes, norms = o.quantize_codes(x, perm, signs, bounds, block, 1e-10, inv)
    codes4, norms4 = o.quantize_codes(x * F32(4), perm, signs, bounds, block, 1e-10, inv)
    assert np.array_equal(codes, codes4)                 # power-of-two scale: exact
    assert np.array_equal(norms4, norms * F32(4))
    one, one_norm = o.quantize_codes(x[1:2], perm, signs, bounds, block, 1e-10, inv)
    assert np.array_equal(one[0], codes[1]) and one_norm[0] == norms[1]
    values = o.quantize_values(x, perm, signs, cents, bounds, block, 1e-10)
    assert not values[4].any() and norms[4] == 0
    # eps is added to the norm: a tiny token divided by (s + eps), not by s
    tiny = np.full((1, dim), 1e-12, F32)
    _, s = o.quantize_codes(tiny, perm, signs, bounds, block, 1e-10, inv)
    unit = tiny / (s + F32(1e-10))[:, None]
    assert np.abs(unit).max() < 0.02


def test_activation_values_match_independent_reference_dim24():
    """native tests/test_packed_matmul.py:97-134: tanh(linspace) centroids, dim=24,
    block=8, nearest-centroid by exhaustive argmin, tolerance 2e-3."""
    torch.manual_seed(41)
    dim, block = 24, 8
    x = torch.randn(2, 3, dim)
    x[0, 0].zero_()
    perm = torch.randperm(dim).numpy()
    signs = (torch.randint(0, 2, (dim,), dtype=torch.int8) * 2 - 1).numpy()
    cents = torch.tanh(torch.linspace(-1.7, 1.7, 16)).numpy()
    bounds = ((cents[:-1] + cents[1:]) / 2).astype(F32)
    flat = x.reshape(-1, dim).numpy()
    got = o.quantize_values(flat, perm, signs, cents, bounds, block, 1e-10)
    norms = np.linalg.norm(flat.astype(np.float64), axis=1, keepdims=True)
    unit = flat / (norms + 1e-10)
    rot = (unit[:, perm] * signs).reshape(-1, 3, block) @ o.hadamard_dense(block) / block ** 0.5
    idx = np.abs(rot.reshape(-1, dim)[..., None] - cents.astype(np.float64)).argmin(-1)
    want = cents[idx] * norms
    assert np.abs(got - want).max() <= 2e-3
    assert not got[0].any()


# ------------------------------------------------------------- whole layer

@pytest.mark.parametrize(("wbits", "abits", "with_bias"), [(4, 4, True), (3, 3, False), (2, 4, True), (2, 3, False), (4, 6, True)])
def test_whole_layer_against_dense_algorithm(wbits, abits, with_bias):
    """tests/test_paper_reference_oracle.py:122-203: dim=24, seed=29, zero weight row,
    zero token; weight indices by exhaustive nearest centroid on the dense rotation,
    bf16 row norms, output within 2e-5, zero token -> bias exactly."""
    torch.manual_seed(202)
    lin = torch.nn.Linear(24, 5, bias=with_bias)
    with torch.no_grad():
        lin.weight[1].zero_()
    acts = torch.randn(2, 2, 24)
    acts[0, 0].zero_()
    w = lin.weight.detach().numpy().astype(F32)
    bias = lin.bias.detach().numpy() if with_bias else None
    perm, signs, block, inv = o.rpbh_constants(24, 29)
    cw, bw = o.lloyd_max_tables(24, wbits)
    ca, ba = o.lloyd_max_tables(24, abits)
    dense = _dense_rotation(perm, signs, block)

    packed, r_bf16, idx = o.quantize_weight(w, perm, signs, bw, block, 1e-10, wbits)
    rot_w = w.astype(np.float64) @ dense
    raw = np.linalg.norm(rot_w, axis=1)
    dirs = rot_w / np.maximum(raw, 1e-10)[:, None]
    want_idx = np.abs(dirs[..., None] - cw.astype(np.float64)).argmin(-1)
    assert np.array_equal(idx, want_idx.astype(np.uint8))
    assert np.array_equal(o.unpack_bits(packed, wbits, idx.size).reshape(idx.shape), idx)
    assert torch.equal(r_bf16, torch.from_numpy(raw.astype(F32)).to(torch.bfloat16))

    x = acts.reshape(-1, 24).numpy()
    codes, s = o.quantize_codes(x, perm, signs, ba, block, 1e-10, inv)
    y = o.linear_from_codes_f64(codes, s, ca, idx, r_bf16.float().numpy(), cw, bias)

    rot_x = x.astype(np.float64) @ dense
    tn = np.linalg.norm(rot_x, axis=1, keepdims=True)
    dx = rot_x / (tn + 1e-10)
    qa = ca.astype(np.float64)[np.abs(dx[..., None] - ca.astype(np.float64)).argmin(-1)] * tn
    qw = r_bf16.float().numpy().astype(np.float64)[:, None] * cw.astype(np.float64)[want_idx]
    want = qa @ qw.T + (0 if bias is None else bias.astype(np.float64))
    assert np.abs(y - want).max() <= 2e-5
    zero_tok = np.zeros(5) if bias is None else bias.astype(np.float64)
    assert np.array_equal(y[0], zero_tok)
    assert not y[:, 1].any() if bias is None else np.array_equal(y[:, 1], np.full(4, bias[1], np.float64))

    # C oracle agrees with the numpy statement
    yc = oracle_c.linear_from_codes(codes, s, ca, packed, wbits, r_bf16.float().numpy(), cw, bias, 5)
    assert np.abs(yc - y).max() <= 1e-12


@pytest.mark.parametrize("bits", [2, 3, 4, 6])
def test_matmul_packed_weight_arange_indices(bits):
    # native tests/test_packed_matmul.py:365-405: indices = arange % 2^b,
    # centroids = linspace(-1, 1), row_norms = linspace(0.5, 1.5), tol 2e-2
    torch.manual_seed(bits)
    rows, k, n = 9, 19, 7
    x = torch.randn(rows, k).numpy()
    idx = (np.arange(n * k) % (1 << bits)).astype(np.uint8).reshape(n, k)
    packed = _pack_loop(idx.reshape(-1).tolist(), bits)
    r = np.linspace(0.5, 1.5, n, dtype=F32)
    cents = np.linspace(-1, 1, 1 << bits, dtype=F32)
    bias = torch.randn(n).numpy()
    want = x.astype(np.float64) @ (r[:, None] * cents[idx]).astype(np.float64).T + bias
    got = oracle_c.matmul_packed_weight(x, packed, r, cents, bias, bits, n)
    assert np.abs(got - want).max() <= 1e-5
    assert np.abs(o.matmul_packed_weight_f32(x, packed, r, cents, bits, n, bias) - want).max() <= 1e-6
