"""CPU-side checks: the C ABI library loads and exports what the header declares,
and the host modules (codebooks, rotation, packing, weight quantizer, config,
module skeleton, drop-in package validation) agree with the oracle / fixtures."""

from __future__ import annotations

import ctypes
import hashlib
import json
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import oracle_np as o

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_symbol_the_header_declares():
    from orbitquant_amd import _lib

    header = (ROOT / "include" / "orbitquant_hip.h").read_text()
    body = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(oq_[a-z0-9_]+)\s*\(", body))
    assert declared == set(_lib.EXPORTS)
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared:
        assert hasattr(lib, name), name
    loaded = _lib.load()
    assert loaded.oq_version().decode().startswith("orbitquant-hip")


def test_debug_override_knows_its_switches():
    """oq_debug_override touches no GPU: known switches are accepted (and cleared again), others refused."""
    from orbitquant_amd import _lib

    lib = _lib.load()
    for name in (b"OQ_GEMM_TILE", b"OQ_GEMM_WG_SPLIT", b"OQ_GEMV_CFG", b"OQ_NO_TOKEN_LINEAR", b"OQ_GEMV_MAX_M"):
        assert lib.oq_debug_override(name, b"1") == 0
        assert lib.oq_debug_override(name, None) == 0
    assert lib.oq_debug_override(b"OQ_NO_SUCH_SWITCH", b"1") != 0 and b"unknown switch" in lib.oq_last_error()
    assert lib.oq_debug_override(None, b"1") != 0


def test_debug_override_is_refused_in_a_process_started_without_the_debug_variable():
    """A serving process cannot have its kernel variants switched at run time: without ORBITQUANT_DEBUG=1
    in its starting environment the call fails and says why."""
    import os
    import subprocess
    import sys

    code = ("from orbitquant_amd import _lib; lib = _lib.load(); rc = lib.oq_debug_override(b'OQ_GEMM_TILE', b'3'); "
            "print(rc, lib.oq_last_error().decode())")
    env = {k: v for k, v in os.environ.items() if k != "ORBITQUANT_DEBUG"}
    root = str(Path(__file__).resolve().parent.parent)
    done = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr
    rc, message = done.stdout.strip().split(" ", 1)
    assert int(rc) != 0 and "ORBITQUANT_DEBUG=1" in message


def test_product_codebooks_match_reference_generated_fixture(golden_dir):
    from orbitquant_amd.codebooks import get_codebook

    tables = json.loads((golden_dir / "codebooks_v2.json").read_text())["tables"]
    for dim, bits in [(24, 2), (24, 3), (24, 4), (24, 6), (32, 3), (1152, 2), (1152, 3), (1152, 4),
                      (3072, 3), (4096, 4), (14336, 3), (5120, 6), (13824, 6)]:
        want = tables[f"dim{dim}_bits{bits}"]
        book = get_codebook(dim, bits)
        assert book.centroids.view(torch.int32).tolist() == want["centroids_u32"], (dim, bits)
        assert book.boundaries.view(torch.int32).tolist() == want["boundaries_u32"], (dim, bits)


def test_product_codebook_newton_cross_check():
    from orbitquant_amd.codebooks import get_codebook, solve_fixed_point_newton

    for dim, bits in [(64, 4), (1152, 4), (3072, 3)]:
        positive = np.array(solve_fixed_point_newton(dim, bits))
        book = get_codebook(dim, bits).centroids.numpy().astype(np.float64)
        assert np.abs(book[book.size // 2:] - positive).max() <= 3e-8   # fp32 rounding of the table
        oc, ob = o.lloyd_max_tables(dim, bits)
        assert np.array_equal(oc, get_codebook(dim, bits).centroids.numpy())
        assert np.array_equal(ob, get_codebook(dim, bits).boundaries.numpy())


def test_product_rotation_matches_fixture_and_oracle(golden_dir):
    from orbitquant_amd.rotations import RPBHRotation, fwht, paper_block_size

    draws = json.loads((golden_dir / "rotations.json").read_text())["draws"]
    for key, want in draws.items():
        dim = int(key.split("_")[0][3:])
        seed = int(key.split("seed")[1])
        rot = RPBHRotation(dim, seed)
        assert hashlib.sha256(rot.permutation.numpy().astype("<i8").tobytes()).hexdigest() == want["perm_sha256"]
        assert hashlib.sha256(rot.signs.numpy().astype("i1").tobytes()).hexdigest() == want["signs_sha256"]
        assert rot.block_size == o.paper_block(dim) == paper_block_size(dim)
    rot = RPBHRotation(96, 3, 32)
    perm, signs, block, inv = o.rpbh_constants(96, 3, 32)
    x = torch.randn(5, 96)
    assert np.array_equal(rot.apply_to_activations(x).numpy(), o.rotate(x.numpy(), perm, signs, block, inv))
    assert np.array_equal(fwht(x[:, :64]).numpy(), o.fwht_np(x[:, :64].numpy()))
    back = rot.apply_inverse_to_activations(rot.apply_to_activations(x))
    assert torch.allclose(back, x, atol=1e-5)
    with pytest.raises(ValueError):
        RPBHRotation(96, 0, 64)
    with pytest.raises(ValueError):
        RPBHRotation(96, 0, 24)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 6, 8])
def test_product_packing_matches_oracle(bits):
    from orbitquant_amd.packing import pack_lowbit, packed_length, unpack_lowbit

    values = torch.from_numpy((np.arange(10007) * 5 % (1 << bits)).astype(np.uint8))
    packed = pack_lowbit(values, bits)
    assert packed.numel() == packed_length(values.numel(), bits)
    assert np.array_equal(packed.numpy(), o.pack_bits(values.numpy(), bits))
    assert torch.equal(unpack_lowbit(packed, bits, values.numel()), values)
    with pytest.raises(ValueError):
        pack_lowbit(torch.tensor([1 << bits]), bits)
    with pytest.raises(ValueError):
        pack_lowbit(values, 9)


@pytest.mark.parametrize(("name", "k", "n"), [("w4a4", 96, 33), ("w3a3", 64, 17), ("w2a4", 128, 9), ("w4a6", 24, 5)])
def test_weight_quantizer_matches_oracle_and_row_tiling(name, k, n):
    from orbitquant_amd import get_codebook, get_rpbh_rotation, quantize_weight, recipe

    cfg = recipe(name)
    torch.manual_seed(k + n)
    w = torch.randn(n, k) * 0.05
    w[2] = 0
    rot = get_rpbh_rotation(k, 0)
    book = get_codebook(k, cfg.weight_bits)
    packed, norms = quantize_weight(w, rotation=rot, codebook=book, bits=cfg.weight_bits, eps=cfg.activation_eps)
    tiled, norms2 = quantize_weight(w, rotation=rot, codebook=book, bits=cfg.weight_bits, eps=cfg.activation_eps, row_tile=8)
    assert torch.equal(packed, tiled) and torch.equal(norms, norms2)
    perm, signs, block, _ = o.rpbh_constants(k, 0)
    want_packed, want_norms, idx = o.quantize_weight(w.numpy(), perm, signs, book.boundaries.numpy(), block, cfg.activation_eps, cfg.weight_bits)
    assert np.array_equal(packed.numpy(), want_packed) and torch.equal(norms, want_norms)
    assert norms[2] == 0        # zero row keeps a zero norm -> dequantizes to zeros


def test_config_and_recipes():
    from orbitquant_amd import OrbitQuantConfig, recipe

    assert (recipe("W4A6").weight_bits, recipe("w4-a6").activation_bits) == (4, 6)
    assert recipe("w2a3", rotation_seed=7).rotation_seed == 7
    for bad in ({"weight_bits": 5}, {"activation_bits": 1}, {"codebook_version": 1}, {"block_size": 0},
                {"activation_eps": 0.0}, {"runtime_mode": "dequant_bf16"}):
        with pytest.raises(ValueError):
            OrbitQuantConfig(**bad)
    with pytest.raises(ValueError):
        recipe("w5a5")


def test_orbit_linear_skeleton_on_cpu():
    from orbitquant_amd import OrbitLinear, recipe

    lin = torch.nn.Linear(64, 10)
    layer = OrbitLinear.from_linear(lin, config=recipe("w3a3"))
    state = layer.state_dict()
    assert sorted(state) == ["bias", "packed_weight_indices", "row_norms"]
    assert state["packed_weight_indices"].dtype == torch.uint8 and state["packed_weight_indices"].numel() == 240
    assert state["row_norms"].dtype == torch.bfloat16
    assert layer._rotation_permutation.dtype == torch.int32 and layer._rotation_signs.dtype == torch.int8
    layer.to(torch.bfloat16)       # constants survive dtype casts
    assert layer._activation_codebook_boundaries.dtype == torch.float32
    assert layer.packed_weight_indices.dtype == torch.uint8
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        layer(torch.randn(2, 64))
    with pytest.raises(ValueError):
        layer(torch.randn(2, 63))
    with pytest.raises(TypeError):
        OrbitLinear.from_linear(torch.nn.Conv1d(3, 3, 1), config=recipe("w4a4"))
    with pytest.raises(ValueError):
        OrbitLinear(in_features=64, out_features=10, config=recipe("w3a3"), bias=None,
                    packed_weight_indices=torch.zeros(10, dtype=torch.uint8), row_norms=state["row_norms"])


def test_fake_impl_gives_shape_and_dtype():
    from orbitquant_amd import OrbitLinear, recipe

    layer = OrbitLinear.from_linear(torch.nn.Linear(64, 10), config=recipe("w4a4"))
    meta = [t.to("meta") for t in (
        layer._rotation_permutation, layer._rotation_signs, layer._activation_codebook_centroids,
        layer._activation_codebook_boundaries, layer.packed_weight_indices.data, layer.row_norms.data,
        layer._weight_codebook_centroids)]
    x = torch.empty(3, 5, 64, dtype=torch.bfloat16, device="meta")
    y = torch.ops.orbitquant_amd.quantized_linear(x, *meta, None, 64, 1e-10, 0.125, 4, 4, 10)
    assert tuple(y.shape) == (3, 5, 10) and y.dtype == torch.bfloat16


def test_dropin_package_surface_and_validation():
    import orbitquant_packed_matmul as pkg

    for name in ("supports_device", "matmul_packed_weight", "quantize_activations_packed_w4",
                 "quantize_activations_int8", "matmul_packed_w4a4_int8", "quantize_activations_cpu",
                 "matmul_packed_adaln_int4_cpu", "supports_cpu_activation", "supports_cpu_adaln"):
        assert callable(getattr(pkg, name))
    assert pkg.supports_device("cpu") is False and pkg.supports_cpu_activation() is False
    with pytest.raises(ValueError):
        pkg.supports_device("tpu")
    x = torch.zeros(2, 16)
    with pytest.raises(ValueError):
        pkg.matmul_packed_weight(x, torch.zeros(8, dtype=torch.uint8), torch.ones(1), torch.zeros(16), bits=9,
                                 out_features=1, in_features=16)
    with pytest.raises(ValueError):
        pkg.matmul_packed_weight(x, torch.zeros(8, dtype=torch.uint8), torch.ones(1), torch.zeros(16), bits=4,
                                 out_features=1, in_features=32)
    with pytest.raises(RuntimeError):
        pkg.matmul_packed_weight(x, torch.zeros(8, dtype=torch.uint8), torch.ones(1), torch.zeros(16), bits=4,
                                 out_features=1, in_features=16)
    with pytest.raises(RuntimeError):
        pkg.quantize_activations_packed_w4(x, torch.arange(16), torch.ones(16), torch.zeros(15), inv_sqrt_block=0.25)


def test_activation_table_on_the_cpu():
    """The table handed to the quantize kernel is the function itself on all 65536 bit patterns."""
    from orbitquant_amd import ops

    gelu = torch.nn.functional.gelu
    for dtype in (torch.bfloat16, torch.float16):
        table = ops.activation_table(gelu, dtype, "cpu")
        assert table.dtype == dtype and table.shape == (65536,)
        for value in (0.0, 1.0, -1.0, 0.37, -3.5, 100.0):
            t = torch.tensor([value], dtype=dtype)
            bits = int(t.view(torch.int16).item()) & 0xFFFF
            assert torch.equal(table[bits : bits + 1], gelu(t))
        assert torch.isnan(table[(torch.tensor([float("nan")], dtype=dtype).view(torch.int16).item()) & 0xFFFF])
    with pytest.raises(ValueError):
        ops.activation_table(gelu, torch.float32, "cpu")
    with pytest.raises(ValueError):
        ops.activation_table(lambda t: t.float(), torch.bfloat16, "cpu")
