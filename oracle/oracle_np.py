"""CPU restatement (numpy) of the reference's quantized-linear forward.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
it is the checker that `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py` compare the HIP path against.

Every function cites the reference lines it restates (paths relative to the
reference checkout).  Arithmetic is fp32 with one rounding per operation unless
stated; numpy never contracts a multiply and an add into an FMA.

Sum-of-squares order ("sumsq-v1").  The reference takes the token norm with
`torch.norm` (src/orbitquant/functional.py:17), whose fp32 summation order is an
implementation detail of the torch build.  This oracle fixes one order, the HIP
kernel reproduces it, and the two must agree bit for bit:

  * pad the row with zeros to a multiple of 2048 and view it as
    [passes, 256 lanes, 8 elements];
  * per (pass, lane): s_e = x_e * x_e, then
    v = ((s0+s1)+(s2+s3)) + ((s4+s5)+(s6+s7));
  * per lane: q = v(pass 0) + v(pass 1) + ... (left to right);
  * across lanes: a balanced binary tree in lane order (pairs of neighbours
    first: q0+q1, q2+q3, ...; then pairs of those; ... 8 levels).

Parity status: rotation order, bucketize, bit packing, weight indices and the
whole-layer equation are pinned by the reference's own test vectors (see
tests/test_oracle_pins.py); the exact fp32 value of the token norm is pinned
only up to the summation order above.
"""

from __future__ import annotations

import math

import numpy as np
import torch

F32 = np.float32


# --------------------------------------------------------------------------
# constants
# --------------------------------------------------------------------------

def paper_block(dim: int) -> int:
    """rotations/rpbh.py:13-18 - largest power of two dividing dim."""
    block = 1
    while dim % (2 * block) == 0:
        block *= 2
    return block


def rpbh_constants(dim: int, seed: int, block: int | str = "paper"):
    """rotations/rpbh.py:55-72 - (perm int64, signs int8 in {-1,+1}, block, fp32 1/sqrt(block)).

    The draw is defined by torch's CPU generator: permutation first, signs
    second, from the same generator.
    """
    if block == "paper":
        block = paper_block(dim)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    perm = torch.randperm(dim, generator=gen, dtype=torch.long, device="cpu").numpy()
    bits = torch.randint(0, 2, (dim,), generator=gen, dtype=torch.int8, device="cpu").numpy()
    signs = (bits.astype(np.int8) * 2 - 1).astype(np.int8)
    return perm, signs, int(block), F32(1.0 / math.sqrt(block))


def lloyd_max_tables(dim: int, bits: int):
    """codebooks/lloyd_max.py:385-448 - v2 codebook -> (centroids f32, boundaries f32).

    Same iteration as the reference: quantile start on the positive half,
    Lloyd updates over-relaxed by 1.9 while the ordering survives, stop when a
    plain update moves less than 1e-13; mirror; fp64 midpoints; cast to fp32.
    The interval masses come from scipy's regularized incomplete beta instead of
    the reference's own continued fraction (lloyd_max.py:279-340).
    """
    from scipy.special import betainc, gammaln

    b = (dim - 1) / 2.0
    half = (1 << bits) // 2
    log_c = gammaln(dim / 2.0) - 0.5 * math.log(math.pi) - gammaln(b)

    def cdf(z):
        return betainc(0.5, b, np.square(z))

    # quantile start (lloyd_max.py:343-354) by bisection on the |z| cdf
    lo = np.zeros(half)
    hi = np.ones(half)
    target = (np.arange(half) + 0.5) / half
    for _ in range(96):
        mid = (lo + hi) / 2
        below = cdf(mid) < target
        lo = np.where(below, mid, lo)
        hi = np.where(below, hi, mid)
    cents = (lo + hi) / 2

    def conditional_means(c):
        edges = np.concatenate(([0.0], (c[:-1] + c[1:]) / 2, [1.0]))
        left, right = edges[:-1], edges[1:]
        prob = cdf(right) - cdf(left)
        prob[-1] = betainc(b, 0.5, 1.0 - left[-1] ** 2)  # upper tail without cancellation
        mass = 0.5 * prob
        with np.errstate(divide="ignore"):
            log_l = b * np.log1p(-np.square(left))
            log_r = np.where(right < 1.0, b * np.log1p(-np.square(np.minimum(right, 1 - 1e-300))), -np.inf)
            log_r[-1] = -np.inf
        moment = np.exp(log_c) * np.exp(log_l) * -np.expm1(log_r - log_l) / (2 * b)
        return moment / mass

    limit = max(1024, 6 * (1 << bits) ** 2)
    for _ in range(limit):
        nxt = conditional_means(cents)
        if np.max(np.abs(nxt - cents)) < 1e-13:
            cents = nxt
            break
        fast = cents + 1.9 * (nxt - cents)
        upper = np.concatenate((fast[1:], [1.0]))
        cents = fast if np.all((fast > 0.0) & (fast < upper)) else nxt
    else:
        raise RuntimeError("Lloyd-Max did not converge")
    full = np.concatenate((-cents[::-1], cents))
    bounds = (full[:-1] + full[1:]) / 2
    return full.astype(F32), bounds.astype(F32)


# --------------------------------------------------------------------------
# rotation
# --------------------------------------------------------------------------

def fwht_np(y: np.ndarray) -> np.ndarray:
    """rotations/fwht.py:19-25 - radix-2 butterflies, distance 1 first, fp32."""
    y = np.array(y, dtype=F32, copy=True)
    n = y.shape[-1]
    lead = y.shape[:-1]
    d = 1
    while d < n:
        v = y.reshape(-1, n // (2 * d), 2, d)
        left = v[:, :, 0, :].copy()
        right = v[:, :, 1, :].copy()
        v[:, :, 0, :] = left + right
        v[:, :, 1, :] = left - right
        y = v.reshape(*lead, n)
        d *= 2
    return y


def hadamard_dense(n: int) -> np.ndarray:
    """Sylvester matrix H[i, j] = (-1)^popcount(i & j), for brute-force checks."""
    idx = np.arange(n)
    return np.where(np.vectorize(lambda v: bin(v).count("1") & 1)(idx[:, None] & idx[None, :]), -1.0, 1.0)


def rotate(x32: np.ndarray, perm, signs, block: int, inv_sqrt_block) -> np.ndarray:
    """rotations/rpbh.py:74-84 - gather, sign, block FWHT, one multiply by fp32(1/sqrt(h))."""
    x32 = np.asarray(x32, dtype=F32)
    y = x32[..., perm] * signs.astype(F32)
    k = x32.shape[-1]
    y = fwht_np(y.reshape(*x32.shape[:-1], k // block, block)).reshape(x32.shape)
    return y * F32(inv_sqrt_block)


# --------------------------------------------------------------------------
# activation quantization
# --------------------------------------------------------------------------

def sumsq_v1(x32: np.ndarray) -> np.ndarray:
    """Sum of squares per row in the fixed order given in the module docstring."""
    x32 = np.asarray(x32, dtype=F32)
    m, k = x32.shape
    passes = max(1, -(-k // 2048))
    padded = np.zeros((m, passes * 2048), dtype=F32)
    padded[:, :k] = x32
    sq = (padded * padded).reshape(m, passes, 256, 8)
    p = sq[..., 0::2] + sq[..., 1::2]
    p = p[..., 0::2] + p[..., 1::2]
    v = p[..., 0] + p[..., 1]                      # [m, passes, 256]
    q = v[:, 0, :].copy()
    for c in range(1, passes):
        q = q + v[:, c, :]
    while q.shape[1] > 1:
        q = q[:, 0::2] + q[:, 1::2]
    return q[:, 0]


def token_norms(x32: np.ndarray) -> np.ndarray:
    return np.sqrt(sumsq_v1(x32)).astype(F32)


def bucketize(values: np.ndarray, boundaries: np.ndarray) -> np.ndarray:
    """codebooks/lloyd_max.py:40-42 - code = #{j : boundaries[j] < v}; ties to the lower code."""
    return np.searchsorted(np.asarray(boundaries, dtype=F32), np.asarray(values, dtype=F32), side="left").astype(np.uint8)


def quantize_codes(x, perm, signs, boundaries, block: int, eps: float, inv_sqrt_block=None):
    """functional.py:16-21 up to the codes: (codes u8 [M,K], raw norms f32 [M]).

    work = fp32(x); s = ||work||; unit = work / (s + eps) (true division, eps
    added in fp32); rotate; bucketize.  x: float32 array [M, K] (bf16/fp16
    inputs are upcast exactly by the caller).
    """
    x32 = np.asarray(x, dtype=F32)
    if inv_sqrt_block is None:
        inv_sqrt_block = F32(1.0 / math.sqrt(block))
    s = token_norms(x32)
    unit = x32 / (s + F32(eps))[:, None]
    rot = rotate(unit, perm, signs, block, inv_sqrt_block)
    return bucketize(rot, boundaries), s


def quantize_values(x, perm, signs, centroids, boundaries, block, eps):
    """functional.py:21-22 - centroid[code] * s in fp32 (caller casts to x's dtype)."""
    codes, s = quantize_codes(x, perm, signs, boundaries, block, eps)
    return np.asarray(centroids, dtype=F32)[codes] * s[:, None]


def pack_nibbles(codes: np.ndarray) -> np.ndarray:
    """Two 4-bit codes per byte, even k in the low nibble
    (native .../orbitquant_packed_matmul_cuda/packed_matmul.cu:648-656)."""
    return (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)


# --------------------------------------------------------------------------
# bit stream
# --------------------------------------------------------------------------

def pack_bits(values, bits: int) -> np.ndarray:
    """packing/bitpack.py:8-46 - value i at stream bits [i*b, i*b+b), little-endian."""
    flat = np.asarray(values, dtype=np.uint64).reshape(-1)
    out = np.zeros((flat.size * bits + 7) // 8 + 8, dtype=np.uint8)
    pos = np.arange(flat.size, dtype=np.uint64) * np.uint64(bits)
    byte = (pos >> np.uint64(3)).astype(np.int64)
    shift = pos & np.uint64(7)
    word = flat << shift                      # at most 15 significant bits
    np.add.at(out, byte, (word & np.uint64(0xFF)).astype(np.uint8))
    np.add.at(out, byte + 1, ((word >> np.uint64(8)) & np.uint64(0xFF)).astype(np.uint8))
    return out[: (flat.size * bits + 7) // 8].copy()


def unpack_bits(packed, bits: int, count: int) -> np.ndarray:
    """packing/bitpack.py:63-97; scalar form native .../packed_matmul_scalar.cpp:31-43."""
    buf = np.concatenate((np.asarray(packed, dtype=np.uint8).reshape(-1), np.zeros(2, np.uint8)))
    pos = np.arange(count, dtype=np.int64) * bits
    byte = pos >> 3
    shift = pos & 7
    word = buf[byte].astype(np.uint32) | (buf[byte + 1].astype(np.uint32) << 8)
    return ((word >> shift.astype(np.uint32)) & np.uint32((1 << bits) - 1)).astype(np.uint8)


# --------------------------------------------------------------------------
# weights and the linear itself
# --------------------------------------------------------------------------

def quantize_weight(weight, perm, signs, boundaries, block, eps, bits, norm_order="torch"):
    """layers.py:121-125,201-215 - (packed u8, row_norms bf16 as torch tensor, indices u8 [N,K]).

    r = ||W_row|| on the unrotated fp32 row; rotW = rotate(W); unit = rotW / max(r, eps);
    idx = bucketize(unit).  norm_order "torch": torch.norm, as the reference's host path;
    "sumsq_v1": the fixed order of `token_norms`, which is what the GPU kernel computes (the
    reference's device path has an order of its own too, triton_cuda.py:150-152).
    """
    w = torch.as_tensor(np.asarray(weight, dtype=F32))
    r = w.norm(dim=-1) if norm_order == "torch" else torch.from_numpy(token_norms(w.numpy()))
    rot = rotate(w.numpy(), perm, signs, block, F32(1.0 / math.sqrt(block)))
    unit = rot / np.maximum(r.numpy(), F32(eps))[:, None]
    idx = bucketize(unit, boundaries)
    return pack_bits(idx, bits), r.to(torch.bfloat16), idx


def dequantize_weight(packed, row_norms_f32, centroids, bits, n, k) -> np.ndarray:
    """layers.py:1060-1069 - W = r[:, None] * c_w[idx] in fp32."""
    idx = unpack_bits(packed, bits, n * k).reshape(n, k)
    return np.asarray(row_norms_f32, dtype=F32)[:, None] * np.asarray(centroids, dtype=F32)[idx]


def linear_from_codes_f64(codes, s, c_a, idx, r_w, c_w, bias=None) -> np.ndarray:
    """fp64 statement of y = (sum_k c_a[code]*c_w[idx]) * s[m] * r_w[n] + bias[n]
    (functional.py:21-22 + layers.py:1060-1070,1450-1455 without the dtype casts)."""
    a = np.asarray(c_a, dtype=np.float64)[codes]
    w = np.asarray(c_w, dtype=np.float64)[idx]
    y = (a @ w.T) * np.asarray(s, dtype=np.float64)[:, None] * np.asarray(r_w, dtype=np.float64)[None, :]
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)[None, :]
    return y


def matmul_packed_weight_f32(x32, packed, row_norms, centroids, bits, n, bias=None) -> np.ndarray:
    """native .../orbitquant_packed_matmul_cpu/packed_matmul_scalar.cpp:45-74:
    out[m,n] = (sum_k x[m,k] * c[idx[n,k]]) * r[n] + bias[n] (fp64 accumulation here)."""
    x32 = np.asarray(x32, dtype=F32)
    k = x32.shape[1]
    idx = unpack_bits(packed, bits, n * k).reshape(n, k)
    w = np.asarray(centroids, dtype=np.float64)[idx]
    y = (x32.astype(np.float64) @ w.T) * np.asarray(row_norms, dtype=np.float64)[None, :]
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)[None, :]
    return y


# --------------------------------------------------------------------------
# AdaLN INT4 group-scaled linear
# --------------------------------------------------------------------------

def bf16_round(a: np.ndarray) -> np.ndarray:
    """fp32 values rounded to bfloat16 (nearest even), returned as fp32."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=F32)).to(torch.bfloat16).float().numpy()


def adaln_quantize(weight, group_size: int):
    """src/orbitquant/adaln.py:17-35 - (packed u8, scales fp32 [N, groups], codes u8 [N, groups*group_size]).

    Rows are zero-padded to whole groups; per group scale = max(absmax, 1e-12) / 7 in fp32,
    code = clip(round_half_even(w / scale), -8, 7) + 8, two codes per byte, even index in the low nibble.
    """
    w = np.asarray(weight, dtype=F32)
    n, k = w.shape
    groups = (k + group_size - 1) // group_size
    padded = np.zeros((n, groups * group_size), dtype=F32)
    padded[:, :k] = w
    grouped = padded.reshape(n, groups, group_size)
    scales = (np.maximum(np.abs(grouped).max(axis=-1), F32(1e-12)) / F32(7.0)).astype(F32)
    signed = np.clip(np.rint(grouped / scales[..., None]), -8, 7).astype(np.int16)
    codes = (signed + 8).astype(np.uint8).reshape(n, groups * group_size)
    flat = codes.reshape(-1)
    packed = (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)
    return packed, scales, codes


def adaln_linear_f64(x, codes, scales_bf16, bias, in_features: int, group_size: int) -> np.ndarray:
    """The contract of the packed AdaLN linear before its final rounding (adaln.py:300-312 dequantization,
    cpu_msvc_avx2.cpp:186-236 of the reference): w = bf16((code - 8) * scale), y = x @ w.T + bias, here in fp64.
    x: bf16-representable fp32 [M, K]; scales_bf16: the stored scales as fp32 [N, groups]; bias fp32 [N] or None."""
    n = codes.shape[0]
    signed = codes.astype(np.int16).astype(F32) - F32(8)
    w = bf16_round((signed.reshape(n, -1, group_size) * np.asarray(scales_bf16, dtype=F32)[..., None]).reshape(n, -1))[:, :in_features]
    y = np.asarray(x, dtype=np.float64) @ w.astype(np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)[None, :]
    return y
