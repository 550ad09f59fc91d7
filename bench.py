"""Benchmark of the quantized-linear forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c5] [--m M]

Default workload: BASELINE.json configs[1] - the DiT-XL/2 MLP pair, W4A4, bf16,
M = 2048 tokens: fc1 1152->4608, GELU, fc2 4608->1152.  One step = rotate+quantize,
packed GEMM, GELU, rotate+quantize, packed GEMM, with the input already resident
in HBM.  Prints ONE JSON line; `value` is whole-step TFLOP/s counted as 2*M*N*K
per linear.  The `roofline` object is for the dominant kernel (the packed GEMM,
or the streaming kernel for the small-M workload c5), timed alone with events on
the launch stream.  `cpu_baseline` times the CPU oracle (a port of the
reference's CPU path) on a bounded row sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

# Kernel arguments in device memory instead of host memory (a switch of the HIP runtime, read when it loads, so
# it is set before torch is imported; a caller's own setting wins): the command processor then reads a launch's
# arguments without a trip over PCIe, which takes about 1.3 us off every launch of the step (86 -> 81 us measured
# on one box, alternating).  `config.hip_force_dev_kernarg` reports what the run had.
os.environ.setdefault("HIP_FORCE_DEV_KERNARG", "1")

import numpy as np  # noqa: E402
import torch  # noqa: E402

MFMA_BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--m", type=int, default=0, help="token count override (c5: 1, 4 or 16)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-grouped-launch", action="store_true",
                    help="c5: q, k and v share their input's quantization but each take a launch of their own")
    ap.add_argument("--no-shared-quantization", action="store_true",
                    help="c5: q, k and v each quantize their (common) input, as the reference's layers do")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of HIP-graph replays")
    ap.add_argument("--kernel-iters", type=int, default=50)
    ap.add_argument("--gemm-phases", action="store_true",
                    help="print where the time inside one packed-GEMM launch of the workload goes (in-kernel clock stamps); "
                         "needs a library built with -DOQ_GEMM_STAMPS: python -m orbitquant_amd.build --variant stamps "
                         "--flags=-DOQ_GEMM_STAMPS --only packed_gemm.hip, then ORBITQUANT_HIP_LIB=orbitquant_amd/liborbitquant_hip_stamps.so")
    ap.add_argument("--activation", default="output", choices=["output", "input", "separate"],
                    help="where the GELU between two linears runs: as a table lookup in the epilogue of the "
                         "matmul that produces its input (default), in the quantize kernel of the layer that "
                         "consumes it, or as torch's separate kernel (identical results all three ways)")
    ap.add_argument("--unfused-activation", action="store_true", help="same as --activation separate")
    return ap.parse_args()


# ---------------------------------------------------------------- workloads

def workload_spec(name: str, m_override: int):
    """-> dict(name, M, dtype, layers=[(K, N, wbits, abits, block, act_after)], x_kind)"""
    if name == "c1":
        return dict(name="c1 single W4A4 linear 1152->1152, fp32, block 64", M=m_override or 256,
                    dtype=torch.float32, x_kind="entry_outliers",
                    layers=[(1152, 1152, 4, 4, 64, None)], w_std=0.02)
    if name == "c2":
        return dict(name="c2 DiT-XL/2 MLP pair W4A4 bf16 (1152->4608, GELU, 4608->1152)", M=m_override or 2048,
                    dtype=torch.bfloat16, x_kind="column_outliers",
                    layers=[(1152, 4608, 4, 4, "paper", "gelu"), (4608, 1152, 4, 4, "paper", None)], w_std=0.02)
    if name == "c3":
        return dict(name="c3 Flux double-stream projections W3A3 bf16 (qkv, out, fc1, fc2)", M=m_override or 4608,
                    dtype=torch.bfloat16, x_kind="student_t",
                    layers=[(3072, 9216, 3, 3, "paper", "slice3072"), (3072, 3072, 3, 3, "paper", None),
                            (3072, 12288, 3, 3, "paper", "gelu"), (12288, 3072, 3, 3, "paper", None)], w_std=0.02)
    if name == "c4":
        return dict(name="c4 video-DiT FFN W4A6 bf16 (5120->13824, GELU, 13824->5120)", M=m_override or 32760,
                    dtype=torch.bfloat16, x_kind="entry_outliers",
                    layers=[(5120, 13824, 4, 6, "paper", "gelu"), (13824, 5120, 4, 6, "paper", None)], w_std=0.015)
    # c5: one interior layer group of the 40-layer decode stack (q,k W2; v,o W3; MLP W3) is
    # built per distinct matrix; see build_c5
    return dict(name="c5 small-M decode stack, mixed W2/W3/W4, A4", M=m_override or 1, dtype=torch.bfloat16,
                x_kind="plain", layers=[], w_std=0.02)


def make_input(spec, k, gen):
    m = spec["M"]
    x = torch.randn(m, k, generator=gen)
    kind = spec["x_kind"]
    if kind == "entry_outliers":
        mask = torch.rand(m, k, generator=gen) < 0.01
        x = torch.where(mask, x * 20, x)
    elif kind == "column_outliers":
        cols = torch.randperm(k, generator=gen)[: max(1, int(np.ceil(0.005 * k)))]
        x[:, cols] *= 30
    elif kind == "student_t":
        chi = torch.randn(m, k, 4, generator=gen).square().sum(-1)
        x = x / torch.sqrt(chi / 4)
    return x.to(spec["dtype"])


def random_packed_weight(n, k, bits, gen, device):
    """Synthetic quantized weight: uniform random indices (the matmul kernels do not care
    how indices were chosen) and row norms of N(0, std) rows."""
    nbytes = (n * k * bits + 7) // 8
    packed = torch.randint(0, 256, (nbytes,), generator=gen, dtype=torch.uint8)
    return packed.to(device)


def build_layers(spec, device, gen, real_quantization: bool, activation: str = "output"):
    from orbitquant_amd import OrbitLinear, OrbitQuantConfig

    layers = []
    for (k, n, wbits, abits, block, act) in spec["layers"]:
        cfg = OrbitQuantConfig(weight_bits=wbits, activation_bits=abits, block_size=block)
        if real_quantization:
            w = torch.randn(n, k, generator=gen) * spec["w_std"]
            layer = OrbitLinear.from_weight(w, bias=torch.zeros(n), config=cfg)
        else:
            packed = torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=gen, dtype=torch.uint8)
            norms = (torch.full((n,), spec["w_std"] * np.sqrt(k)) * (1 + 0.05 * torch.randn(n, generator=gen))).to(torch.bfloat16)
            layer = OrbitLinear(in_features=k, out_features=n, config=cfg, bias=torch.zeros(n),
                                packed_weight_indices=packed, row_norms=norms)
        layer = layer.to(device)
        if layer.bias is not None:
            layer.bias.data = layer.bias.data.to(spec["dtype"])
        layers.append((layer, act))
    if activation != "separate" and spec["dtype"] in (torch.bfloat16, torch.float16):
        for (cur, act), (nxt, _) in zip(layers, layers[1:]):
            if act == "gelu":   # a table of torch's own GELU, applied by one of the two layers around it
                if activation == "output":
                    cur.fuse_output_activation(torch.nn.functional.gelu, dtype=spec["dtype"])
                else:
                    nxt.fuse_input_activation(torch.nn.functional.gelu, dtype=spec["dtype"])
    return layers


def activation_is_fused(layers, i) -> bool:
    if layers[i][0]._output_activation_table is not None:
        return True
    return i + 1 < len(layers) and layers[i + 1][0]._input_activation_table is not None


def apply_activation(h, act, fused: bool):
    if act == "gelu":
        return h if fused else torch.nn.functional.gelu(h)
    if act == "slice3072":
        return h[..., :3072].contiguous()
    return h


def run_step(layers, x):
    h = x
    for i, (layer, act) in enumerate(layers):
        h = apply_activation(layer(h), act, activation_is_fused(layers, i))
    return h


# ------------------------------------------------------------------ graph replay

def capture_step(fn, replays_checked=3):
    """Capture one step into a HIP graph and check every one of a few replays against the eager
    result (with eager work and synchronisation between replays).  Returns (replay, out) or None
    when capture is unavailable or a replay differs."""
    try:
        ref = fn()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = fn()
        for _ in range(replays_checked):
            graph.replay()
            torch.cuda.synchronize()
            again = fn()          # eager work between replays
            torch.cuda.synchronize()
            if not (torch.equal(out, ref) and torch.equal(again, ref)):
                return None
        return graph.replay, out
    except Exception as exc:  # capture not supported here: fall back to eager timing
        print(f"bench.py: graph capture unavailable ({exc}); timing eager launches", file=sys.stderr)
        return None


PREROLL_SECONDS = 0.4


def preroll(fn, seconds=PREROLL_SECONDS):
    """Run the step untimed for `seconds` before any measurement.  The device raises its clocks
    over the first tenths of a second of sustained work (the same step measures about 10 %
    slower in the first milliseconds after idle than in steady state); the W warm-up steps of
    the contract, a millisecond at this workload, do not get there."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


# ------------------------------------------------------------ kernel-only timing

def time_kernel(fn, iters):
    """Average device time of one call of `fn` (one kernel launch): events on the launch stream
    around `iters` back-to-back launches, issued eagerly and as one HIP-graph replay; the
    smaller of the two averages is returned (eager launches of a short kernel can be
    host-bound, a graph separates its nodes by more than back-to-back launches do)."""
    for _ in range(5):
        fn()
    torch.cuda.synchronize()

    def timed(run):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        run()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e-3  # seconds per launch

    def eager():
        for _ in range(iters):
            fn()

    best = timed(eager)
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(iters):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        best = min(best, timed(graph.replay))
    except Exception:
        pass
    return best


def _code_format(layer, x):
    """The activation-code format OrbitLinear's forward picks for this input (orbitquant_amd/layers.py)."""
    if layer.activation_bits <= 4:
        return "nibble"
    tokens, k = x.numel() // layer.in_features, layer.in_features
    return "u8" if (tokens > 16 and k % 64 == 0) or k % 128 == 0 else None


def chunked_step_closure(layers, x, chunks, streams=2):
    """The step in `chunks` row chunks dealt round `streams` ordinary (equal-priority) streams, each chunk its own
    chain of oq_quantized_linear calls (rows are independent): the quantizer of one chunk runs beside the matmul
    of another, on the CUs a 192-workgroup matmul leaves idle.  Host-side ordering only (events); None when
    the step has no bare-call form.  Returns (step, outputs) with outputs the list of per-chunk output tensors."""
    m = x.shape[0]
    if m % chunks != 0:
        return None
    rows = m // chunks
    chains = []
    for c in range(chunks):
        raws, h = [], x[c * rows:(c + 1) * rows]
        for i, (layer, act) in enumerate(layers):
            if _code_format(layer, h) is None or act == "slice3072" or (act == "gelu" and not activation_is_fused(layers, i)):
                return None
            raw = RawLinear(layer, h)
            raws.append(raw)
            h = raw.out
        chains.append(raws)
    side = [torch.cuda.Stream() for _ in range(streams)]

    def step():
        main = torch.cuda.current_stream()
        for st in side:
            st.wait_stream(main)
        for c, raws in enumerate(chains):
            with torch.cuda.stream(side[c % streams]):
                for raw in raws:
                    raw.linear()
        for st in side:
            main.wait_stream(st)
        return [raws[-1].out for raws in chains]
    return step


class RawLinear:
    """One OrbitLinear as bare C-ABI calls into buffers allocated once: what a native host does.

    The Python wrappers in orbitquant_amd/ops.py check every operand and allocate the outputs of every
    call; at the c2 shapes that is more host time per call than the kernels take on the device, and a
    loop of such calls measures the host.  These closures call the library the way bench.py's kernel
    timings need it: same entry points, same operands, nothing else."""

    def __init__(self, layer, x, with_output_map=True):
        from orbitquant_amd import _lib, ops

        self.lib = _lib.load()
        self.layer, self.x = layer, x
        k, n = layer.in_features, layer.out_features
        m = x.numel() // k
        self.m, self.k, self.n = m, k, n
        dev = x.device
        self.fmt = _code_format(layer, x)
        if self.fmt is None:
            raise ValueError("this layer's forward passes values, not codes")
        width = k // 2 if self.fmt == "nibble" else k
        self.codes = torch.empty((m, width), dtype=torch.uint8, device=dev)
        self.norms = torch.empty(m, dtype=torch.float32, device=dev)
        self.out = torch.empty((m, n), dtype=x.dtype, device=dev)
        dt = ops._DTYPES[x.dtype]
        fmt = {"u8": ops.OQ_CODES_U8, "nibble": ops.OQ_CODES_NIBBLE}[self.fmt]
        packed, w_bits, w_cents = layer._matmul_weight(m)   # what the layer's forward reads at this token count
        self.keep = (packed, w_cents)
        # the workspace the call may use (partial tiles of a launch that shares K between workgroups), allocated once
        self.ws_bytes = int(self.lib.oq_packed_linear_workspace_bytes(m, n, k, int(w_bits), fmt, int(layer.activation_bits)))
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev) if self.ws_bytes else None
        self.ws_ptr = None if self.ws is None else self.ws.data_ptr()
        levels = layer._activation_codebook_boundaries.numel() + 1
        imap = layer._input_activation_table
        omap = layer._output_activation_table if with_output_map else None
        plan = layer._rotation_plan
        rot = (layer._rotation_permutation.data_ptr(), layer._rotation_signs.data_ptr(),
               layer._activation_codebook_boundaries.data_ptr(), layer._activation_codebook_centroids.data_ptr())
        consts = (int(layer.rotation.block_size), float(layer.activation_eps), float(layer.rotation.normalization))
        q_tail = (self.codes.data_ptr(), fmt, None, ops.OQ_VALUES_NONE, self.norms.data_ptr())
        if imap is None:
            self._quantize = (self.lib.oq_rotate_quantize,
                              (x.data_ptr(), dt, m, k, *rot, levels, *consts, ops._ptr(plan), *q_tail))
        else:
            self._quantize = (self.lib.oq_rotate_quantize_mapped,
                              (x.data_ptr(), dt, imap.data_ptr(), m, k, *rot, levels, *consts, ops._ptr(plan), *q_tail))
        bias = layer.bias
        g_args = (self.codes.data_ptr(), fmt, self.norms.data_ptr(), layer._activation_codebook_centroids.data_ptr(),
                  int(layer.activation_bits), packed.data_ptr(), int(w_bits), layer.row_norms.data_ptr(), w_cents.data_ptr(),
                  ops._ptr(bias), ops._dt(bias) if bias is not None else ops.OQ_F32, m, n, k, self.out.data_ptr(), dt)
        self._gemm = ((self.lib.oq_packed_linear, g_args) if omap is None else
                      (self.lib.oq_packed_linear_mapped, (*g_args, omap.data_ptr())))
        self._linear = (self.lib.oq_quantized_linear,
                        (x.data_ptr(), dt, ops._ptr(imap), m, k, *rot, int(layer.activation_bits), *consts, ops._ptr(plan),
                         packed.data_ptr(), int(w_bits), layer.row_norms.data_ptr(), w_cents.data_ptr(), ops._ptr(bias),
                         ops._dt(bias) if bias is not None else ops.OQ_F32, n, self.codes.data_ptr(), self.norms.data_ptr(),
                         self.out.data_ptr(), dt, ops._ptr(omap)))

    def _call(self, what, workspace):
        fn, args = what   # (the stream is looked up per call: under graph capture it is the capturing stream)
        tail = (self.ws_ptr, self.ws_bytes) if workspace else ()
        if fn(*args, *tail, torch.cuda.current_stream().cuda_stream) != 0:
            raise RuntimeError(self.lib.oq_last_error().decode())

    def quantize(self):
        self._call(self._quantize, False)

    def gemm(self):
        self._call(self._gemm, True)

    def linear(self):
        self._call(self._linear, True)
        return self.out


def gemm_only_closure(layer, x, with_output_map=True):
    """The matmul launch of `layer` alone, on pre-computed activation codes (with the layer's
    fused output activation, as it runs in the step, unless `with_output_map` is False)."""
    from orbitquant_amd import ops

    k = layer.in_features
    if _code_format(layer, x) is not None:
        raw = RawLinear(layer, x, with_output_map)
        raw.quantize()
        return raw.gemm
    _, unit, norms = ops.rotate_quantize(
        x, layer._rotation_permutation, layer._rotation_signs, layer._activation_codebook_boundaries,
        block_size=layer.rotation.block_size, eps=layer.activation_eps,
        inv_sqrt_block=layer.rotation.normalization, centroids=layer._activation_codebook_centroids,
        code_format=None, values="unit_bf16", input_map=layer._input_activation_table)
    flat_norms = norms.reshape(-1)

    def fn():
        return ops.matmul_packed_weight_values(
            unit, layer.packed_weight_indices, layer.row_norms, layer._weight_codebook_centroids,
            bits=layer.weight_bits, out_features=layer.out_features, in_features=k, bias=layer.bias,
            token_scale=flat_norms, output_dtype=x.dtype)
    return fn


def quantize_only_closure(layer, x):
    from orbitquant_amd import ops

    fmt = _code_format(layer, x)
    if fmt is not None:
        return RawLinear(layer, x).quantize
    vals = "unit_bf16"

    def fn():
        return ops.rotate_quantize(
            x, layer._rotation_permutation, layer._rotation_signs, layer._activation_codebook_boundaries,
            block_size=layer.rotation.block_size, eps=layer.activation_eps,
            inv_sqrt_block=layer.rotation.normalization, centroids=layer._activation_codebook_centroids,
            code_format=fmt, values=vals, input_map=layer._input_activation_table, plan=layer._rotation_plan)
    return fn


def abi_step_closure(layers, x):
    """The whole step as bare C-ABI calls (one oq_quantized_linear per layer into buffers allocated once),
    or None when a layer of the step has no such form (a separate activation kernel, value activations)."""
    if any(act == "gelu" and not activation_is_fused(layers, i) for i, (_l, act) in enumerate(layers)):
        return None
    raws, h = [], x
    for layer, act in layers:
        if _code_format(layer, h) is None:
            return None
        raw = RawLinear(layer, h)
        raws.append(raw)
        h = raw.out
        if act == "slice3072":
            return None

    def step():
        for raw in raws:
            raw.linear()
        return raws[-1].out
    return step


# ----------------------------------------------------------------- CPU baseline

def _cpu_threads() -> int:
    """Thread count of the CPU leg: what the box grants (OMP_NUM_THREADS when set, else the
    affinity mask), capped at 64 like the reference's pool (cpu_threads.cpp:22-36,89-101)."""
    env = os.environ.get("ORBITQUANT_CPU_THREADS") or os.environ.get("OMP_NUM_THREADS")
    n = int(env) if env and env.isdigit() and int(env) > 0 else len(os.sched_getaffinity(0))
    return max(1, min(n, 64))


def cpu_baseline(spec, layers, x, target_seconds=15.0):
    """The CPU path on a bounded sample of the same workload, about `target_seconds` of work.

    kind "reference": the reference's own CPU kernels (quantize_activations_cpu +
    matmul_packed_weight, compiled from the reference checkout into oracle/_ref) when that
    library travelled with the tree; else kind "port": the C oracle.  Same layers, same
    packed weights, same activations as the GPU leg."""
    from oracle import oracle_c, ref_cpu

    threads = _cpu_threads()
    os.environ["ORBITQUANT_CPU_THREADS"] = str(threads)   # read by the reference's pool on first use
    use_ref = ref_cpu.available()
    prepared = []
    for layer, act in layers:
        prepared.append(dict(
            perm=layer.rotation.permutation.to(torch.int32), signs=layer.rotation.signs.to(torch.int8),
            bounds=layer.activation_codebook.boundaries.float(), cents=layer.activation_codebook.centroids.float(),
            block=layer.rotation.block_size, inv=float(np.float32(layer.rotation.normalization)),
            packed=layer.packed_weight_indices.cpu(), r=layer.row_norms.float().cpu(),
            cw=layer.weight_codebook.centroids.float(), bits=layer.weight_bits, n=layer.out_features,
            k=layer.in_features, act=act, bias=None if layer.bias is None else layer.bias.float().cpu()))

    def run(rows):
        h = x[:rows].cpu()
        for p in prepared:
            if use_ref:
                q = ref_cpu.quantize_activations_cpu(h, p["perm"], p["signs"], p["cents"], p["bounds"], eps=1e-10,
                                                     inv_sqrt_block=p["inv"], block_size=p["block"])
                y = ref_cpu.matmul_packed_weight(q, p["packed"], p["r"], p["cw"], bits=p["bits"],
                                                 out_features=p["n"], in_features=p["k"], bias=p["bias"])
            else:
                codes, s = oracle_c.rotate_quantize(h.float().numpy(), p["perm"].numpy(), p["signs"].numpy(),
                                                    p["bounds"].numpy(), p["block"], 1e-10, np.float32(p["inv"]),
                                                    threads)
                vals = p["cents"].numpy()[codes] * s[:, None]
                y = torch.from_numpy(oracle_c.matmul_packed_weight(
                    vals, p["packed"].numpy(), p["r"].numpy(), p["cw"].numpy(),
                    None if p["bias"] is None else p["bias"].numpy(), p["bits"], p["n"], threads)).to(h.dtype)
            if p["act"] == "gelu":
                y = torch.nn.functional.gelu(y)
            elif p["act"] == "slice3072":
                y = y[:, :3072].contiguous()
            h = y

    m = x.shape[0]
    rows0 = min(m, 64)
    run(rows0)                                   # warm-up: thread pool, page-in
    t0 = time.perf_counter()
    run(rows0)
    per_row = (time.perf_counter() - t0) / rows0
    rows = int(min(m, max(rows0, target_seconds / per_row)))
    reps = 1
    if rows == m:   # whole passes: a pass over all rows runs far better than the 64-row probe predicts, so time one
        t0 = time.perf_counter()
        run(rows)
        reps = max(1, int(round(target_seconds / (time.perf_counter() - t0))))
    t0 = time.perf_counter()
    for _ in range(reps):
        run(rows)
    dt = time.perf_counter() - t0
    flops = reps * sum(2.0 * rows * p["n"] * p["k"] for p in prepared)
    what = ("reference CPU kernels (quantize_activations_cpu + matmul_packed_weight) built into oracle/_ref"
            if use_ref else "oracle/oq_oracle.c with OpenMP")
    return dict(value=flops / dt / 1e12, unit="TFLOP/s", cores=threads, kind="reference" if use_ref else "port",
                sample=f"{reps} pass(es) over the first {rows} of {m} tokens through every layer of the workload, "
                       f"{dt:.1f} s, {what}, {threads} threads")


def copy_calibration(device, launches=3, mib=256):
    """A plain device copy of known size (`mib` MiB read + `mib` MiB written per launch), so that a
    profiler run of this script holds the yardstick its FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    src = torch.empty(mib << 20, dtype=torch.uint8, device=device).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(launches):
        dst.copy_(src)
    torch.cuda.synchronize()


TRAFFIC_SOURCE = ("recorded, not measured by this run: profiles/traffic.txt holds the bytes per launch that rocprofv3's "
                  "FETCH_SIZE and WRITE_SIZE counters gave for this kernel and shape")


def recorded_traffic(key: str):
    """HBM bytes per launch of the dominant kernel, measured with the profiler's FETCH_SIZE and WRITE_SIZE
    counters and written down in profiles/ (a live run cannot read those counters itself)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "traffic.txt")
    try:
        with open(path) as fh:
            for line in fh:
                parts = line.split()
                if len(parts) >= 2 and parts[0] == key:
                    return float(parts[1])
    except OSError:
        pass
    return None


# ------------------------------------------------------------------------ c5

def small_m_roofline(device, iters, m=1, copies=16):
    """The small-M half of the metric on its roofline kernel: the streaming kernel on the W4
    4096 -> 14336 matrix of the decode stack (29.4 MB of packed indices and row norms per launch),
    timed alone with events on the launch stream, over `copies` distinct matrices launched in turn
    (470 MB: more than the 256 MB of memory-side cache, so every launch streams from HBM)."""
    from orbitquant_amd import ops
    from orbitquant_amd.codebooks import get_codebook

    k, n, bits = 4096, 14336, 4
    gen = torch.Generator().manual_seed(55)
    cb = get_codebook(k, bits)
    cents = cb.centroids.to(device)
    codes = torch.randint(0, 256, (m, k // 2), generator=gen, dtype=torch.uint8).to(device)
    norms = torch.full((m,), 64.0, device=device)
    row_norms = torch.full((n,), 1.28).to(torch.bfloat16).to(device)
    mats = [torch.randint(0, 256, (n * k * bits // 8,), generator=gen, dtype=torch.uint8).to(device) for _ in range(copies)]

    # bare C-ABI calls into one output buffer (the Python wrapper's checks and allocation take longer
    # than this kernel runs)
    from orbitquant_amd import _lib
    lib = _lib.load()
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    calls = [(codes.data_ptr(), ops.OQ_CODES_NIBBLE, norms.data_ptr(), cents.data_ptr(), 4, w.data_ptr(), bits,
              row_norms.data_ptr(), cents.data_ptr(), None, ops.OQ_F32, m, n, k, out.data_ptr(), ops.OQ_BF16)
             for w in mats]
    want = ops.packed_linear(codes, norms, cents, mats[-1], row_norms, cents, code_format="nibble", activation_bits=4,
                             weight_bits=bits, out_features=n, in_features=k, output_dtype=torch.bfloat16)

    def fn():
        stream = torch.cuda.current_stream().cuda_stream   # (under graph capture: the capturing stream)
        for c in calls:
            if lib.oq_packed_linear(*c, None, 0, stream) != 0:
                raise RuntimeError(lib.oq_last_error().decode())
    fn()
    torch.cuda.synchronize()
    assert torch.equal(out, want), "bare call differs from the wrapper's"
    per_launch = time_kernel(fn, max(3, iters // 5)) / copies
    nbytes = mats[0].numel() + 2 * n
    achieved = nbytes / per_launch / 1e9
    return {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": recorded_traffic("c5_gemv_w4_4096x14336"), "traffic_source": TRAFFIC_SOURCE, "kernel": "packed_gemv_kernel<4> on 4096->14336 W4",
            "M": m, "bytes_per_launch": nbytes, "avg_launch_us": per_launch * 1e6, "distinct_matrices": copies}


def c3_gemm_lines(device, iters):
    """The packed GEMMs of the Flux-style block (c3: W3A3, M = 4608), each timed alone: the other half
    of "DiT-XL / Flux shapes" of the large-M target, reported beside the c2 headline.  The figures are
    for the layer as it is by default - the stored 3-bit index stream, fields straddling bytes; the
    `four_bit_copy_*` keys are the same launches on the opt-in copy of the indices at four bits each
    (`OrbitLinear.nibble_copy_for_many_tokens`, N*K/2 more bytes per layer)."""
    spec = workload_spec("c3", 0)
    gen = torch.Generator().manual_seed(3)
    layers = build_layers(spec, device, gen, False)
    out = {}
    for i, (layer, _act) in enumerate(layers):
        k, n = layer.in_features, layer.out_features
        x = make_input(spec, k, gen).to(device)
        layer.nibble_copy_for_many_tokens = False
        t = time_kernel(gemm_only_closure(layer, x), max(5, iters // 2))
        tflops = 2.0 * spec["M"] * n * k / t / 1e12
        line = {"gemm_us": t * 1e6, "gemm_tflops": tflops, "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "weights": "stored 3-bit stream"}
        layer.nibble_copy_for_many_tokens = True
        t4 = time_kernel(gemm_only_closure(layer, x), max(5, iters // 2))
        line["four_bit_copy_gemm_us"] = t4 * 1e6
        line["four_bit_copy_frac"] = 2.0 * spec["M"] * n * k / t4 / 1e12 / MFMA_BF16_PEAK_TFLOPS
        layer.nibble_copy_for_many_tokens = False
        layer._nibble_weight_copy = None
        out[f"{k}->{n}"] = line
    return out


def c4_gemm_lines(device, iters):
    """The two packed GEMMs of the video-DiT FFN (c4: W4A6, M = 32760, one activation code per byte), each
    timed alone: the largest configuration, on the byte-code form of the tile kernel."""
    spec = workload_spec("c4", 0)
    gen = torch.Generator().manual_seed(4)
    layers = build_layers(spec, device, gen, False, activation="separate")
    out = {}
    for layer, _act in layers:
        k, n = layer.in_features, layer.out_features
        x = make_input(spec, k, gen).to(device)
        t = time_kernel(gemm_only_closure(layer, x), max(3, iters // 10))
        tflops = 2.0 * spec["M"] * n * k / t / 1e12
        out[f"{k}->{n}"] = {"gemm_us": t * 1e6, "gemm_tflops": tflops, "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "codes": "one 6-bit code per byte"}
        del x
    torch.cuda.empty_cache()
    return out


def adaln_lines(device, iters):
    """The AdaLN INT4 group-64 linear (the other quantized linear of a DiT block) at the DiT-XL/2 modulation
    shape, 1152 -> 6912, one and sixteen tokens: microseconds per launch and GB/s of packed bytes (indices +
    bf16 scales) against HBM.  The matrix is 4.1 MB: the figure is about launch and latency, not streaming."""
    from orbitquant_amd import _lib, ops

    lib = _lib.load()
    k, n, g = 1152, 6912, 64
    gen = torch.Generator().manual_seed(7)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(device)
    packed, scales = ops.quantize_adaln_weight(w, group_size=g)
    scales = scales.to(torch.bfloat16)
    bias = torch.zeros(n, dtype=torch.bfloat16, device=device)
    nbytes = packed.numel() + 2 * scales.numel()
    out = {}
    for m in (1, 16):
        x = torch.randn(m, k, generator=gen).to(torch.bfloat16).to(device)
        y = torch.empty((m, n), dtype=torch.bfloat16, device=device)
        want = ops.adaln_int4_linear(x, packed, scales, out_features=n, in_features=k, group_size=g, bias=bias)
        args = (x.data_ptr(), packed.data_ptr(), scales.data_ptr(), bias.data_ptr(), m, n, k, g, y.data_ptr())

        def fn():
            if lib.oq_matmul_packed_adaln_int4(*args, torch.cuda.current_stream().cuda_stream) != 0:
                raise RuntimeError(lib.oq_last_error().decode())
        fn()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
        t = time_kernel(fn, max(10, iters))
        out[f"M={m}"] = {"launch_us": t * 1e6, "gbs": nbytes / t / 1e9, "frac_of_hbm": nbytes / t / 1e9 / HBM_PEAK_GBS}
    out["shape"] = [n, k]
    out["packed_bytes"] = nbytes
    return out


def float_activation_lines(device, iters):
    """`oq_matmul_packed_weight` (bf16 activation values times the packed weight, the reference's generic
    contract) on the two c2 shapes: the whole call, i.e. the pass that puts the activations into operand
    order plus the tile kernel, timed with events over back-to-back eager calls."""
    from orbitquant_amd import ops

    spec = workload_spec("c2", 0)
    gen = torch.Generator().manual_seed(9)
    layers = build_layers(spec, device, gen, False)
    out = {}
    for layer, _act in layers:
        k, n = layer.in_features, layer.out_features
        x = make_input(spec, k, gen).to(device)
        cents = layer._weight_codebook_centroids

        def fn():
            ops.matmul_packed_weight_values(x, layer.packed_weight_indices, layer.row_norms, cents, bits=layer.weight_bits,
                                            out_features=n, in_features=k)
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = max(20, iters)
        start.record()
        for _ in range(reps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        t = start.elapsed_time(stop) / reps * 1e-3
        tflops = 2.0 * spec["M"] * n * k / t / 1e12
        out[f"{k}->{n}"] = {"call_us": t * 1e6, "tflops": tflops, "frac": tflops / MFMA_BF16_PEAK_TFLOPS}
    return out


def build_c5(device, gen):
    """The 240 distinct matrices of the 40-layer decode stack: per layer q,k (4096x4096), v,o
    (4096x4096), up (14336x4096), down (4096x14336); interior layers q,k W2 and the rest W3,
    first/last 4 layers all W4."""
    from orbitquant_amd import OrbitLinear, OrbitQuantConfig

    mats = []
    for layer_idx in range(40):
        boundary = layer_idx < 4 or layer_idx >= 36
        for name, (k, n) in (("q", (4096, 4096)), ("k", (4096, 4096)), ("v", (4096, 4096)), ("o", (4096, 4096)),
                             ("up", (4096, 14336)), ("down", (14336, 4096))):
            bits = 4 if boundary else (2 if name in ("q", "k") else 3)
            cfg = OrbitQuantConfig(weight_bits=bits, activation_bits=4)
            packed = torch.randint(0, 256, ((n * k * bits + 7) // 8,), generator=gen, dtype=torch.uint8)
            norms = torch.full((n,), 0.02 * np.sqrt(k)).to(torch.bfloat16)
            mats.append(OrbitLinear(in_features=k, out_features=n, config=cfg, bias=None,
                                    packed_weight_indices=packed, row_norms=norms).to(device))
    return mats


def measure_c5(args, device, brief=False):
    """The decode stack as the step; returns the JSON line of `--workload c5` (brief: without the C-ABI
    and kernel-only legs, for the extra key of the default line)."""
    from orbitquant_amd import ops

    gen = torch.Generator().manual_seed(5)
    m = args.m or 1
    mats = build_c5(device, gen)
    # one input per role and layer, as in a transformer: q, k and v of a layer read the same tensor
    # (and share its quantization), o, up and down each their own; no tensor is read by two layers,
    # so no quantization carries over from one layer to the next
    def fresh(width):
        return torch.randn(m, width, generator=gen).to(torch.bfloat16).to(device)
    roles = ("q", "k", "v", "o", "up", "down")
    layer_input = []
    for _ in range(len(mats) // 6):
        x_attn = fresh(4096)
        layer_input.extend([x_attn, x_attn, x_attn, fresh(4096), fresh(4096), fresh(14336)])
    if not args.no_shared_quantization:
        for i, l in enumerate(mats):
            l.share_input_quantization = roles[i % 6] in ("q", "k", "v")
    # q, k and v of a block as one call (one quantization, one launch): OrbitLinearGroup
    grouped = not (args.no_shared_quantization or args.no_grouped_launch)
    if grouped:
        from orbitquant_amd import OrbitLinearGroup
        step_calls = []
        for base in range(0, len(mats), 6):
            step_calls.append((OrbitLinearGroup(*mats[base:base + 3]), layer_input[base]))
            step_calls.extend((mats[base + j], layer_input[base + j]) for j in (3, 4, 5))
    else:
        step_calls = list(zip(mats, layer_input))
    packed_bytes = sum(l.packed_weight_indices.numel() + 2 * l.out_features for l in mats)
    pre = []
    for l, x in zip(mats, layer_input):
        codes, _, norms = ops.rotate_quantize(
            x, l._rotation_permutation, l._rotation_signs, l._activation_codebook_boundaries,
            block_size=l.rotation.block_size, eps=l.activation_eps, inv_sqrt_block=l.rotation.normalization,
            code_format="nibble")
        pre.append((l, codes, norms))

    def stack_matmuls():
        for l, codes, norms in pre:
            ops.packed_linear(codes, norms, l._activation_codebook_centroids, l.packed_weight_indices, l.row_norms,
                              l._weight_codebook_centroids, code_format="nibble", activation_bits=4,
                              weight_bits=l.weight_bits, out_features=l.out_features, in_features=l.in_features,
                              output_dtype=torch.bfloat16)

    def full_step():
        for fn, x in step_calls:
            fn(x)

    def full_step_out():
        last = None
        for fn, x in step_calls:
            last = fn(x)
        return last

    preroll(full_step)
    eager_dt = time_steps(full_step, args.steps, args.warmup)
    dt, launch, graph_dt = eager_dt, "eager", None
    captured = None if args.no_graph else capture_step(full_step_out)
    if captured is not None:
        graph_dt = time_steps(captured[0], args.steps, args.warmup)
        if graph_dt < dt:
            dt, launch = graph_dt, "hipgraph"

    if brief:
        return {"ms_per_step": dt * 1e3, "gbs": packed_bytes / dt / 1e9, "frac_of_hbm": packed_bytes / dt / 1e9 / HBM_PEAK_GBS, "M": m,
                "launch": launch, "packed_bytes_per_step": packed_bytes,
                "workload": "c5 40-layer decode stack W2/W3/W4 A4: quantize + packed linear of q, k, v (one group), o, up, down per layer"}
    # The same stack driven through the C ABI alone (what a native host does: one oq_quantized_linear
    # call per linear into buffers it owns, no module, no op dispatch, no allocation), to separate
    # the library from the Python around it.  Reported beside `value`, not as `value`.
    from orbitquant_amd import _lib
    lib = _lib.load()
    stream = torch.cuda.current_stream(device).cuda_stream
    keep, calls = [], []
    for l, x in zip(mats, layer_input):
        nib = l.in_features // 2
        bufs = (torch.empty((m, nib), dtype=torch.uint8, device=device), torch.empty(m, dtype=torch.float32, device=device),
                torch.empty((m, l.out_features), dtype=torch.bfloat16, device=device))
        keep.append(bufs)
        calls.append((x.data_ptr(), 2, None, m, l.in_features, l._rotation_permutation.data_ptr(),
                      l._rotation_signs.data_ptr(), l._activation_codebook_boundaries.data_ptr(),
                      l._activation_codebook_centroids.data_ptr(), 4, l.rotation.block_size, l.activation_eps,
                      l.rotation.normalization, l._rotation_plan.data_ptr(), l.packed_weight_indices.data_ptr(), l.weight_bits,
                      l.row_norms.data_ptr(), l._weight_codebook_centroids.data_ptr(), None, 0, l.out_features,
                      bufs[0].data_ptr(), bufs[1].data_ptr(), bufs[2].data_ptr(), 2, None, None, 0, stream))

    def abi_step():
        fn = lib.oq_quantized_linear
        for c in calls:
            if fn(*c) != 0:
                raise RuntimeError(lib.oq_last_error().decode())
    abi_step()
    torch.cuda.synchronize()
    assert torch.equal(keep[-1][2], mats[-1](layer_input[-1])) and torch.equal(keep[2][2], mats[2](layer_input[2])), "C-ABI stack differs from the module stack"
    abi_dt = time_steps(abi_step, args.steps, args.warmup)

    # kernel-only: every matmul launch of the stack, events on the launch stream
    per_stack = time_kernel(stack_matmuls, max(3, args.kernel_iters // 10))
    # W4 matrices alone (the 8 boundary layers' MLP up projections), cycled so the cache cannot hold them
    w4_up = [(l, c, n) for (l, c, n) in pre if l.weight_bits == 4 and l.out_features == 14336]

    def w4_only():
        for l, codes, norms in w4_up:
            ops.packed_linear(codes, norms, l._activation_codebook_centroids, l.packed_weight_indices, l.row_norms,
                              l._weight_codebook_centroids, code_format="nibble", activation_bits=4, weight_bits=4,
                              out_features=l.out_features, in_features=l.in_features, output_dtype=torch.bfloat16)
    per_w4 = time_kernel(w4_only, max(3, args.kernel_iters // 5)) / len(w4_up)
    w4_bytes = w4_up[0][0].packed_weight_indices.numel() + 2 * 14336
    achieved = w4_bytes / per_w4 / 1e9
    out = {
        "metric": "small-M packed-weight GB/s (whole decode stack, quantize + matmul per linear)",
        "value": packed_bytes / dt / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "config": {"workload": f"c5 40-layer decode stack W2/W3/W4 A4, M={m}", "M": m,
                                        "packed_bytes_per_step": packed_bytes, "launch": launch,
                                        "shared_quantization": "none" if args.no_shared_quantization else "q, k, v of a block quantize their common input once",
                                        "grouped_launch": "q, k, v of a block in one launch" if grouped else "none",
                                        "eager_ms_per_step": eager_dt * 1e3,
                                        "graph_ms_per_step": None if graph_dt is None else graph_dt * 1e3,
                                        "c_abi_ms_per_step": abi_dt * 1e3,
                                        "c_abi_gbs": packed_bytes / abi_dt / 1e9,
                                        "preroll_s": PREROLL_SECONDS, "hip_force_dev_kernarg": os.environ.get("HIP_FORCE_DEV_KERNARG"),
                                        "hip_force_dev_kernarg": os.environ.get("HIP_FORCE_DEV_KERNARG")},
        "roofline": dict(small_m_roofline(device, args.kernel_iters, m=m), stack_matmuls_gbs=packed_bytes / per_stack / 1e9,
                         stack_w4_up_avg_launch_us=per_w4 * 1e6, stack_w4_up_gbs=achieved),
    }
    return out


def bench_c5(args, device):
    out = measure_c5(args, device)
    copy_calibration(device)
    print(json.dumps(out))


# ------------------------------------------------------- inside one GEMM launch

def gemm_phases(layers, x, launches=20):
    """Text report of one packed-GEMM launch per layer of the step, from stamps every wavefront of the tile
    kernel takes of the shader clock (s_memtime) and of the 100 MHz wall clock (s_memrealtime) as it passes:
    first instruction, lookup tables written, loop entered, loop left, barrier passed, last store issued, done.
    The stamps exist only in a library compiled with -DOQ_GEMM_STAMPS (a product build takes none)."""
    from orbitquant_amd import _lib

    lib = _lib.load()
    dev = x.device
    stamps = torch.zeros(8192 * 4 * 16, dtype=torch.int64, device=dev)

    def switch(value):
        if lib.oq_debug_override(b"OQ_GEMM_STAMPS", None if value is None else str(value).encode()) != 0:
            raise RuntimeError(lib.oq_last_error().decode())

    h = x
    for i, (layer, act) in enumerate(layers):
        raw = RawLinear(layer, h)
        raw.quantize()
        switch(None)
        per_launch = time_kernel(raw.gemm, 50)
        stamps.zero_()
        switch(stamps.data_ptr())
        for _ in range(launches):
            raw.gemm()
        torch.cuda.synchronize()
        switch(None)
        s = stamps.cpu().numpy().reshape(-1, 16)
        s = s[s[:, 0] != 0]
        if len(s) == 0:
            raise SystemExit("no stamps were written: load a library built with -DOQ_GEMM_STAMPS (see --help)")
        cycles = (s[:, 8] - s[:, 0]).astype(np.float64)
        wall = (s[:, 7] - s[:, 6]).astype(np.float64)            # 10 ns ticks
        mhz = cycles.sum() / wall.sum() * 100.0
        fused = "+gelu" if activation_is_fused(layers, i) and act == "gelu" else ""
        print(f"--- layer {i}{fused}: M={raw.m} N={raw.n} K={raw.k}, {len(s)} wavefronts stamped (the last of {launches} launches each), "
              f"{per_launch * 1e6:.2f} us per launch by events (launch to launch), "
              f"{(s[:, 7].max() - s[:, 6].min()) / 100.0:.2f} us first wavefront start to last wavefront end, shader clock {mhz:.0f} MHz")
        skew = (s[:, 6] - s[:, 6].min()) / 100.0
        print(f"    wavefront start after the first: median {np.median(skew):.2f}, max {skew.max():.2f} us; "
              f"wavefront lifetime: median {np.median(wall) / 100:.2f}, max {wall.max() / 100:.2f} us")
        rows = [("start -> kernel arguments read", 0, 10), ("-> centroids requested, tile mapped", 10, 13), ("-> operand addresses", 13, 14), ("-> first packed operands requested", 14, 15),
                ("-> output-map window requested", 15, 11), ("-> centroids arrived", 11, 12),
                ("-> lookup tables written", 12, 1), ("-> barrier, first lookups (loop entered)", 1, 2), ("main loop", 2, 3),
                ("wait at the barrier after the loop", 3, 4), ("epilogue until the last store is issued", 4, 5),  ("stores drained", 5, 8)]
        for name, a, b in rows:
            d = (s[:, b] - s[:, a]).astype(np.float64) / mhz
            print(f"    {name:42s} median {np.median(d):6.2f}   p10 {np.percentile(d, 10):6.2f}   p90 {np.percentile(d, 90):6.2f}   max {d.max():6.2f} us")
        steps = raw.k // 64
        loop = (s[:, 3] - s[:, 2]).astype(np.float64)
        print(f"    main loop: {np.median(loop) / steps:.0f} shader cycles per K-step of 64 (median over wavefronts; K-steps per wavefront when K is not shared: {steps})")
        xcc = ((s[:, 9] >> 32) & 0xf).astype(np.int64)
        print("    wavefronts per XCC:", np.bincount(xcc, minlength=8).tolist())
        h = raw.out


# ------------------------------------------------------------------------ main

def main() -> int:
    args = parse_args()
    if args.gemm_phases:
        os.environ["ORBITQUANT_DEBUG"] = "1"   # the stamp buffer's address reaches the library through oq_debug_override
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs an AMD GPU (the quantized-linear forward has no CPU fallback)", file=sys.stderr)
        return 2
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.workload == "c5":
        bench_c5(args, device)
        return 0

    spec = workload_spec(args.workload, args.m)
    gen = torch.Generator().manual_seed({"c1": 1, "c2": 2, "c3": 3, "c4": 4}[args.workload])
    real = args.workload in ("c1", "c2")        # larger workloads: synthetic indices (weight quantization is offline)
    layers = build_layers(spec, device, gen, real, activation="separate" if args.unfused_activation else args.activation)
    x = make_input(spec, spec["layers"][0][0], gen).to(device)
    flops = sum(2.0 * spec["M"] * n * k for (k, n, *_rest) in spec["layers"])

    preroll(lambda: run_step(layers, x))
    if args.gemm_phases:
        gemm_phases(layers, x)
        return 0
    eager_dt = time_steps(lambda: run_step(layers, x), args.steps, args.warmup)
    dt, launch, graph_dt = eager_dt, "eager", None
    captured = None if args.no_graph else capture_step(lambda: run_step(layers, x))
    if captured is not None:   # every way of launching is timed; `value` is the fastest, `config.launch` says which
        graph_dt = time_steps(captured[0], args.steps, args.warmup)
        if graph_dt < dt:
            dt, launch = graph_dt, "hipgraph"
    # the same step driven through the C ABI alone: one oq_quantized_linear call per layer into buffers
    # allocated once (no module, no op dispatch, no allocation per call); same kernels, same outputs
    abi_dt = None
    abi = abi_step_closure(layers, x)
    if abi is not None:
        want = run_step(layers, x)
        got = abi()
        torch.cuda.synchronize()
        if not torch.equal(got, want):
            raise AssertionError("the C-ABI step differs from the module step")
        abi_dt = time_steps(abi, args.steps, args.warmup)
        if abi_dt < dt:
            dt, launch = abi_dt, "c_abi"
    # the same calls in row chunks on two streams (quantizer of one chunk beside the matmul of another)
    chunked = {}
    if abi is not None and args.workload == "c2":
        want = run_step(layers, x)
        for chunks in (2, 4):
            step = chunked_step_closure(layers, x, chunks)
            if step is None:
                continue
            got = torch.cat(step(), dim=0)
            torch.cuda.synchronize()
            same = torch.equal(got, want)
            close = same or bool((got.float() - want.float()).abs().max() <= want.float().abs().max() * 2.0 ** -7)
            if not close:
                raise AssertionError("the chunked step differs from the module step")
            cdt = time_steps(step, args.steps, args.warmup)
            chunked[f"{chunks}_chunks_2_streams_ms"] = cdt * 1e3
            chunked[f"{chunks}_chunks_bit_identical"] = same
            if not args.no_graph:   # the same fork and join as one HIP graph (branches of a graph need no host-side events)
                try:
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        outs = step()
                    graph.replay()
                    torch.cuda.synchronize()
                    if torch.equal(torch.cat(outs, dim=0), got):
                        gdt = time_steps(graph.replay, args.steps, args.warmup)
                        chunked[f"{chunks}_chunks_2_streams_graph_ms"] = gdt * 1e3
                        if same and gdt < dt:
                            dt, launch = gdt, f"hipgraph, {chunks} row chunks on 2 streams"
                except Exception as exc:
                    chunked[f"{chunks}_chunks_graph_error"] = str(exc)[:200]
            if same and cdt < dt:
                dt, launch = cdt, f"c_abi, {chunks} row chunks on 2 streams"

    # dominant kernel alone: the packed GEMM of the first layer, and every other piece for the record
    pieces = {}
    h = x
    for i, (layer, act) in enumerate(layers):
        k, n = layer.in_features, layer.out_features
        tq = time_kernel(quantize_only_closure(layer, h), args.kernel_iters)
        tg = time_kernel(gemm_only_closure(layer, h), args.kernel_iters)
        elem = 4 if h.dtype == torch.float32 else 2
        q_bytes = spec["M"] * k * elem + spec["M"] * k * {"nibble": 0.5, "u8": 1, None: 2}[_code_format(layer, h)] + 4 * spec["M"]
        pieces[f"layer{i}"] = {
            "shape": [spec["M"], n, k], "gemm_us": tg * 1e6, "gemm_tflops": 2.0 * spec["M"] * n * k / tg / 1e12,
            "quantize_us": tq * 1e6, "quantize_gbs": q_bytes / tq / 1e9}
        if layer._output_activation_table is not None:   # the same matmul without the activation in its epilogue
            tp = time_kernel(gemm_only_closure(layer, h, with_output_map=False), args.kernel_iters)
            pieces[f"layer{i}"]["gemm_us_without_activation"] = tp * 1e6
        h = apply_activation(layer(h), act, activation_is_fused(layers, i))
    dom = max(pieces.values(), key=lambda p: p["gemm_us"])
    achieved = dom["gemm_tflops"]

    out = {
        "metric": "W4A4 packed-linear TFLOP/s (quantize + packed matmul, 2*M*N*K per linear)"
        if args.workload in ("c1", "c2") else "packed-linear TFLOP/s (quantize + packed matmul, 2*M*N*K per linear)",
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": spec["name"], "M": spec["M"], "input_dtype": str(spec["dtype"]).replace("torch.", ""),
                   "flop_per_step": flops, "launch": launch, "eager_ms_per_step": eager_dt * 1e3,
                   "graph_ms_per_step": None if graph_dt is None else graph_dt * 1e3,
                   "c_abi_ms_per_step": None if abi_dt is None else abi_dt * 1e3,
                   "row_chunks_on_two_streams": chunked,
                   "preroll_s": PREROLL_SECONDS, "hip_force_dev_kernarg": os.environ.get("HIP_FORCE_DEV_KERNARG"),
                   "activation": ("gelu as a 65536-entry table of torch's own results, looked up in the producing "
                                  "matmul's epilogue" if any(l._output_activation_table is not None for l, _ in layers)
                                  else "gelu as a 65536-entry table of torch's own results, looked up in the next "
                                  "layer's quantize kernel" if any(l._input_activation_table is not None for l, _ in layers)
                                  else "torch gelu kernel between the linears")},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": recorded_traffic(f"{args.workload}_gemm"), "traffic_source": TRAFFIC_SOURCE,
                     "kernel": "packed_gemm_kernel" + (" with the GELU table in its epilogue"
                                                       if "gemm_us_without_activation" in dom else ""),
                     "shape_mnk": dom["shape"], "avg_launch_us": dom["gemm_us"]},
        "pieces": pieces,
    }
    if "gemm_us_without_activation" in dom:
        out["roofline"]["frac_without_activation"] = (2.0 * dom["shape"][0] * dom["shape"][1] * dom["shape"][2]
                                                      / (dom["gemm_us_without_activation"] * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS)
    if args.workload == "c2":
        # the two other figures the metric names, each on its own roofline kernel (`--workload c3|c5` for the full runs)
        out["roofline_small_m"] = small_m_roofline(device, args.kernel_iters)
        out["c3_gemms"] = c3_gemm_lines(device, args.kernel_iters)
        out["float_activations"] = float_activation_lines(device, args.kernel_iters)
        out["c4_gemms"] = c4_gemm_lines(device, args.kernel_iters)
        out["adaln"] = adaln_lines(device, args.kernel_iters)
        out["decode_stack"] = measure_c5(args, device, brief=True)
    copy_calibration(device)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(spec, layers, x)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
