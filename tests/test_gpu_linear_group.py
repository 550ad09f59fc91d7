"""GPU tests of oq_packed_linear_group / OrbitLinearGroup: several packed linears on the same
activation codes through one native call.  The contract is bit identity with one
oq_packed_linear call per matrix (pinned to the oracle elsewhere), whether the group runs as a
single launch (decode sizes) or as one launch per matrix."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


def make_group(dev, m, k, shapes, abits, dtype, seed, block="paper"):
    """shapes: (out_features, weight_bits, with_bias) per matrix; one quantized input for all."""
    from orbitquant_amd import ops
    from orbitquant_amd.codebooks import get_codebook
    from orbitquant_amd.rotations import get_rpbh_rotation

    rot, acb = get_rpbh_rotation(k, 0, block), get_codebook(k, abits)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    x[torch.rand(m, k, generator=g) < 0.01] *= 20
    fmt = "nibble" if abits <= 4 else "u8"
    codes, _, norms = ops.rotate_quantize(
        x.to(dtype).to(dev), rot.permutation.to(torch.int32).to(dev), rot.signs.to(torch.int8).to(dev),
        acb.boundaries.to(dev), block_size=rot.block_size, eps=1e-10, inv_sqrt_block=rot.normalization, code_format=fmt)
    weights = []
    for n, wbits, with_bias in shapes:
        weights.append((
            torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=g, dtype=torch.uint8).to(dev),
            (0.02 * (1 + 0.1 * torch.randn(n, generator=g))).to(torch.bfloat16).to(dev),
            get_codebook(k, wbits).centroids.to(dev), wbits, n,
            torch.randn(n, generator=g).to(dtype).to(dev) if with_bias else None))
    return dict(codes=codes, norms=norms, cents=acb.centroids.to(dev), weights=weights, fmt=fmt, abits=abits, k=k, dtype=dtype)


def one_by_one(c):
    from orbitquant_amd import ops

    return [ops.packed_linear(c["codes"], c["norms"], c["cents"], w[0], w[1], w[2], code_format=c["fmt"],
                              activation_bits=c["abits"], weight_bits=w[3], out_features=w[4], in_features=c["k"],
                              bias=w[5], output_dtype=c["dtype"]) for w in c["weights"]]


def grouped(c):
    from orbitquant_amd import ops

    return ops.packed_linear_group(c["codes"], c["norms"], c["cents"], c["weights"], code_format=c["fmt"],
                                   activation_bits=c["abits"], in_features=c["k"], output_dtype=c["dtype"])


GROUPS = [
    # single launch, eight wavefronts per workgroup (rows shorter than 2048 values)
    dict(m=1, k=512, shapes=[(96, 2, False), (40, 2, True), (17, 3, False)], abits=4),
    dict(m=3, k=1024, shapes=[(256, 4, True), (256, 3, True)], abits=4),
    dict(m=16, k=384, shapes=[(64, 3, False), (64, 4, False), (64, 2, False), (33, 3, True)], abits=3),
    # single launch, sixteen wavefronts (K >= 2048, at most 4096 rows each); ragged row counts
    dict(m=1, k=4096, shapes=[(1024, 2, False), (256, 2, False), (250, 3, False)], abits=4),
    dict(m=5, k=2048, shapes=[(4096, 4, True), (1000, 3, False)], abits=4),
    # more rows than the rule for one / two rows-per-workgroup steps
    dict(m=2, k=512, shapes=[(5000, 3, False), (4200, 3, False)], abits=4),
    # 17 to 64 tokens: the single launch with two or four blocks of sixteen token rows per workgroup
    dict(m=17, k=512, shapes=[(96, 2, False), (40, 2, True), (17, 3, False)], abits=4),
    dict(m=32, k=4096, shapes=[(1024, 2, False), (256, 2, False), (250, 3, False)], abits=4),
    dict(m=64, k=2048, shapes=[(4096, 4, True), (1000, 3, False)], abits=4),
    dict(m=33, k=512, shapes=[(5000, 3, False), (4200, 3, False)], abits=4),
    dict(m=64, k=384, shapes=[(64, 3, False), (64, 4, False), (64, 2, False), (33, 3, True)], abits=3),
    dict(m=48, k=1024, shapes=[(9000, 4, True), (8200, 2, False)], abits=4),
    # groups that run as one launch per matrix: mixed K-splits, byte codes, wide weights, many tokens,
    # more than four matrices, a single matrix
    dict(m=1, k=4096, shapes=[(4096, 4, False), (4112, 4, False)], abits=4),
    dict(m=4, k=512, shapes=[(64, 4, False), (48, 3, True)], abits=6),
    dict(m=4, k=512, shapes=[(64, 6, False), (48, 8, True)], abits=4),
    dict(m=70, k=512, shapes=[(64, 4, False), (48, 3, True)], abits=4),
    dict(m=1, k=256, shapes=[(32, 2, False)] * 5, abits=4),
    dict(m=1, k=256, shapes=[(32, 4, True)], abits=4),
]


# every case in bf16, a third of them also with fp32 outputs and biases
@pytest.mark.parametrize("case,dtype", [(c, torch.bfloat16) for c in range(len(GROUPS))] +
                         [(c, torch.float32) for c in range(0, len(GROUPS), 3)])
def test_group_equals_one_call_per_matrix(dev, case, dtype):
    spec = GROUPS[case]
    c = make_group(dev, spec["m"], spec["k"], spec["shapes"], spec["abits"], dtype, seed=100 + case)
    want = one_by_one(c)
    got = grouped(c)
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert a.shape == b.shape and a.dtype == b.dtype
        assert torch.equal(a, b), f"matrix {i} of case {case}: {(a.float() - b.float()).abs().max().item()}"


@pytest.mark.parametrize("rows_per_step", ["1", "2", "4"])
def test_group_result_does_not_depend_on_rows_per_workgroup(dev, rows_per_step, library_switch):
    """The launch shape is a speed choice only."""
    c = make_group(dev, 3, 2048, [(1000, 2, False), (520, 3, True), (4096, 4, False)], 4, torch.bfloat16, seed=7)
    want = one_by_one(c)
    library_switch("OQ_GEMV_GROUP_R", rows_per_step)
    assert all(torch.equal(a, b) for a, b in zip(grouped(c), want))
    library_switch("OQ_NO_GEMV_GROUP", "1")          # and with the single launch switched off
    assert all(torch.equal(a, b) for a, b in zip(grouped(c), want))


@pytest.mark.parametrize("k,n,wbits", [(4096, 4096, 4), (4096, 14336, 3), (2048, 520, 2), (14336, 4096, 4), (1024, 96, 6),
                                        (512, 40, 8), (16384, 64, 4)])
def test_few_token_launch_equals_rows_of_a_batch(dev, k, n, wbits):
    """Launches of few tokens (M*K <= 16384) read their activation operands from values decoded once
    per workgroup; larger launches look every operand up in the table.  Token rows are independent, so
    a row computed alone, in a staged launch of few rows and in a sixteen-row batch must agree bit for bit."""
    from orbitquant_amd import ops

    c = make_group(dev, 16, k, [(n, wbits, True)], 4, torch.bfloat16, seed=900 + wbits)
    w = c["weights"][0]

    def run(rows):
        return ops.packed_linear(c["codes"][rows], c["norms"][rows], c["cents"], w[0], w[1], w[2], code_format="nibble",
                                 activation_bits=4, weight_bits=wbits, out_features=n, in_features=k, bias=w[5],
                                 output_dtype=torch.bfloat16)

    batch = run(slice(0, 16))
    few = max(1, min(16, 16384 // k))
    for start in (0, 16 - few):
        assert torch.equal(run(slice(start, start + few)), batch[start:start + few]), (start, few)
    assert torch.equal(run(slice(5, 6)), batch[5:6])
    if few >= 3:
        assert torch.equal(run(slice(2, 5)), batch[2:5])


@pytest.mark.parametrize("k,n,wbits,abits", [(4096, 4096, 4, 4), (512, 14336, 3, 4), (14336, 4096, 4, 4), (2048, 9000, 2, 3),
                                            (1024, 520, 6, 4), (512, 96, 8, 4), (1024, 4096, 4, 6), (4096, 600, 3, 6),
                                            (512, 9000, 4, 8)])
def test_seventeen_to_sixty_four_tokens_stream_like_sixteen(dev, k, n, wbits, abits):
    """17 to 64 tokens take the streaming kernel with two or four blocks of sixteen token rows per
    workgroup.  A token row's sums do not depend on the rows computed with it: every row of such a
    launch equals the same row from launches of at most sixteen tokens, bit for bit."""
    from orbitquant_amd import ops

    c = make_group(dev, 64, k, [(n, wbits, True)], abits, torch.bfloat16, seed=700 + wbits + abits)
    w = c["weights"][0]

    def run(lo, hi):
        return ops.packed_linear(c["codes"][lo:hi], c["norms"][lo:hi], c["cents"], w[0], w[1], w[2], code_format=c["fmt"],
                                 activation_bits=abits, weight_bits=wbits, out_features=n, in_features=k, bias=w[5],
                                 output_dtype=torch.bfloat16)

    want = torch.cat([run(lo, lo + 16) for lo in range(0, 64, 16)])
    assert torch.equal(run(0, 64), want)
    for lo, hi in ((0, 17), (3, 35), (10, 42), (15, 64), (31, 64)):
        assert torch.equal(run(lo, hi), want[lo:hi]), (lo, hi)


WHOLE = [
    # one token, wide rows: quantizer launch, then the whole group in one launch
    dict(m=1, k=4096, shapes=[(4096, 2, False), (1024, 2, True), (1000, 3, False)], dtype=torch.bfloat16, block="paper"),
    dict(m=1, k=4096, shapes=[(4096, 2, False), (4096, 2, False), (4096, 3, False)], dtype=torch.bfloat16, block="paper"),
    dict(m=1, k=2048, shapes=[(4096, 4, True), (4096, 3, True), (520, 4, True), (2048, 2, True)], dtype=torch.float16, block=128),
    dict(m=1, k=8192, shapes=[(3000, 3, False), (3000, 4, False)], dtype=torch.bfloat16, block=512),
    dict(m=1, k=3072, shapes=[(4096, 4, False), (1024, 4, False)], dtype=torch.bfloat16, block=1024),
    # other groups (some run as one launch per matrix)
    dict(m=1, k=4096, shapes=[(1024, 2, False), (1024, 3, False)], dtype=torch.bfloat16, block="paper"),
    dict(m=1, k=1024, shapes=[(4096, 2, False), (4096, 3, False)], dtype=torch.bfloat16, block="paper"),
    dict(m=4, k=4096, shapes=[(4096, 2, False), (1024, 2, True)], dtype=torch.bfloat16, block="paper"),
    dict(m=1, k=4096, shapes=[(4096, 2, False), (1024, 2, True)], dtype=torch.float32, block="paper"),
    dict(m=33, k=512, shapes=[(64, 4, False), (48, 3, True)], dtype=torch.float16, block="paper"),
]


# every case plain; every other 16-bit case also through an input map
@pytest.mark.parametrize("case,mapped", [(c, False) for c in range(len(WHOLE))] +
                         [(c, True) for c in range(0, len(WHOLE), 2) if WHOLE[c]["dtype"] != torch.float32])
def test_whole_forward_group_equals_one_call_per_matrix(dev, case, mapped):
    """ops.quantized_linear_group (oq_quantized_linear_group) against ops.quantized_linear per matrix,
    which is pinned to quantize + packed linear in test_gpu_token_linear.py."""
    from orbitquant_amd import ops
    from orbitquant_amd.codebooks import get_codebook
    from orbitquant_amd.rotations import get_rpbh_rotation

    spec = WHOLE[case]
    m, k, dtype = spec["m"], spec["k"], spec["dtype"]
    rot, acb = get_rpbh_rotation(k, 0, spec["block"]), get_codebook(k, 4)
    g = torch.Generator().manual_seed(500 + case)
    x = torch.randn(m, k, generator=g)
    x[torch.rand(m, k, generator=g) < 0.01] *= 20
    x = x.to(dtype).to(dev)
    weights = []
    for n, wbits, with_bias in spec["shapes"]:
        weights.append((
            torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=g, dtype=torch.uint8).to(dev),
            (0.02 * (1 + 0.1 * torch.randn(n, generator=g))).to(torch.bfloat16).to(dev),
            get_codebook(k, wbits).centroids.to(dev), wbits, n,
            torch.randn(n, generator=g).to(dtype).to(dev) if with_bias else None))
    table = ops.activation_table(torch.nn.functional.silu, dtype, dev) if mapped else None
    common = dict(block_size=rot.block_size, eps=1e-10, inv_sqrt_block=rot.normalization, activation_bits=4, input_map=table)
    perm, signs = rot.permutation.to(torch.int32).to(dev), rot.signs.to(torch.int8).to(dev)
    bounds, cents = acb.boundaries.to(dev), acb.centroids.to(dev)
    got = ops.quantized_linear_group(x, perm, signs, bounds, cents, weights, **common)
    for i, w in enumerate(weights):
        want = ops.quantized_linear(x, perm, signs, bounds, cents, w[0], w[1], w[2], weight_bits=w[3], out_features=w[4],
                                    bias=w[5], **common)
        assert got[i].shape == want.shape and got[i].dtype == want.dtype
        assert torch.equal(got[i], want), f"matrix {i} of case {case}: {(got[i].float() - want.float()).abs().max().item()}"


def test_linear_group_module(dev):
    """OrbitLinearGroup: outputs equal every member's own forward."""
    from orbitquant_amd import OrbitLinear, OrbitLinearGroup, OrbitQuantConfig

    torch.manual_seed(3)
    q, k = (OrbitLinear.from_linear(torch.nn.Linear(1024, n), config=OrbitQuantConfig(weight_bits=2, activation_bits=4)).to(dev)
            for n in (512, 128))
    v = OrbitLinear.from_linear(torch.nn.Linear(1024, 128, bias=False), config=OrbitQuantConfig(weight_bits=3, activation_bits=4)).to(dev)
    group = OrbitLinearGroup(q, k, v)
    for m, dtype in ((1, torch.bfloat16), (7, torch.float16), (64, torch.bfloat16), (2, torch.float32)):
        x = torch.randn(m, 1024, device=dev).to(dtype)
        want = [layer(x) for layer in (q, k, v)]
        got = group(x)
        assert len(got) == 3
        assert all(torch.equal(a, b) for a, b in zip(got, want)), (m, dtype)
    # three-dimensional input keeps its leading dimensions
    x = torch.randn(2, 3, 1024, device=dev, dtype=torch.bfloat16)
    assert [t.shape for t in group(x)] == [(2, 3, 512), (2, 3, 128), (2, 3, 128)]
    assert all(torch.equal(a, layer(x)) for a, layer in zip(group(x), (q, k, v)))
    # members must share the quantizer
    other = OrbitLinear.from_linear(torch.nn.Linear(2048, 64), config=OrbitQuantConfig(weight_bits=2, activation_bits=4)).to(dev)
    with pytest.raises(ValueError):
        OrbitLinearGroup(q, other)
    wider = OrbitLinear.from_linear(torch.nn.Linear(1024, 64), config=OrbitQuantConfig(weight_bits=2, activation_bits=3)).to(dev)
    with pytest.raises(ValueError):
        OrbitLinearGroup(q, wider)
    with pytest.raises(TypeError):
        OrbitLinearGroup(q, torch.nn.Linear(1024, 8))
    # a member with a fused output activation: the members run one after the other, same results
    k.fuse_output_activation(torch.nn.functional.gelu)
    x = torch.randn(1, 1024, device=dev, dtype=torch.bfloat16)
    assert all(torch.equal(a, layer(x)) for a, layer in zip(group(x), (q, k, v)))


def test_group_argument_checks(dev):
    from orbitquant_amd import _lib

    lib = _lib.load()
    c = make_group(dev, 1, 256, [(32, 4, False), (32, 4, False)], 4, torch.bfloat16, seed=1)
    outs = [torch.empty(1, 32, dtype=torch.bfloat16, device=dev) for _ in range(2)]
    ptrs = ctypes.c_void_p * 2

    def call(count=2, w_bits=(4, 4), out=None, a_bits=4, fmt=1):
        return lib.oq_packed_linear_group(
            c["codes"].data_ptr(), fmt, c["norms"].data_ptr(), c["cents"].data_ptr(), a_bits, count,
            ptrs(*[w[0].data_ptr() for w in c["weights"]]), (ctypes.c_int * 2)(*w_bits),
            ptrs(*[w[1].data_ptr() for w in c["weights"]]), ptrs(*[w[2].data_ptr() for w in c["weights"]]), None, 0, 1,
            (ctypes.c_int64 * 2)(32, 32), 256, out if out is not None else ptrs(*[o.data_ptr() for o in outs]), 2, None, 0, None)

    assert call() == 0
    assert call(count=0) == 1 and b"count" in lib.oq_last_error()
    assert call(count=65) == 1
    assert call(w_bits=(4, 9)) == 1 and b"bits" in lib.oq_last_error()
    assert call(out=ptrs(outs[0].data_ptr(), None)) == 1 and b"null" in lib.oq_last_error()
    assert call(a_bits=0) == 1
    assert call(fmt=7) == 1
    torch.cuda.synchronize()
    want = one_by_one(c)
    assert torch.equal(outs[0], want[0]) and torch.equal(outs[1], want[1])
