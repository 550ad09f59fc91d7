"""`OrbitLinear`: the quantized linear module, MI355X path.

State dict = `packed_weight_indices` (uint8, flat bit stream), `row_norms`
(bfloat16 [N]) and `bias`, exactly the reference module's persistent tensors
(src/orbitquant/layers.py:386-400); rotation / codebook constants are
non-persistent buffers rebuilt from (in_features, seed, block, bits)
(layers.py:358-385,625-649).

Forward = one opaque custom op (`orbitquant_amd::quantized_linear`) with a fake
implementation, so `torch.compile(fullgraph=True)` traces through it the way
the reference's `orbitquant::packed_linear_forward` does (layers.py:38-72,
1072-1077).  The op is stateless: every tensor it needs is an argument.

Inside the op (the reference's `_forward_impl`, layers.py:1079-1455, for AMD), one
native call (`oq_quantized_linear`):
  1. fused rotate + per-token quantize (HIP) -> activation codes + token norms
  2. packed-weight matmul (HIP): streaming kernel for <= 64 tokens, MFMA tile
     kernel otherwise.
For a single token both run in ONE launch.  Shapes the code kernels do not take
(activation widths above 4 bits with K not a multiple of 64 / 128) hand the matmul
bf16 centroid values instead of codes.
There is no dequantized-weight or CPU fallback on this path.
"""

from __future__ import annotations

import torch
from torch import nn

from . import ops
from .codebooks import get_codebook
from .config import OrbitQuantConfig
from .rotations import get_rpbh_rotation
from .weights import quantize_weight

_LIB = torch.library.Library("orbitquant_amd", "DEF")
_LIB.define(
    "quantized_linear(Tensor x, Tensor permutation, Tensor signs, Tensor act_centroids, "
    "Tensor act_boundaries, Tensor packed_weight_indices, Tensor row_norms, Tensor weight_centroids, "
    "Tensor? bias, int block_size, float eps, float inv_sqrt_block, int activation_bits, "
    "int weight_bits, int out_features, Tensor? input_map=None, Tensor? output_map=None, "
    "Tensor? rotate_plan=None) -> Tensor"
)


def quantized_linear_forward(
    x, permutation, signs, act_centroids, act_boundaries, packed_weight_indices, row_norms,
    weight_centroids, bias, block_size, eps, inv_sqrt_block, activation_bits, weight_bits, out_features,
    input_map=None, output_map=None, rotate_plan=None,
):
    in_features = x.shape[-1]
    if bias is not None and bias.dtype != x.dtype:
        bias = bias.to(x.dtype)
    tokens = x.numel() // in_features
    if (activation_bits <= 4 and in_features % 2 == 0) or (tokens > 16 and in_features % 64 == 0) or in_features % 128 == 0:
        # activation codes (two per byte up to 4 bits, else one per byte) into the tile / streaming
        # kernels; one native call: a single launch for one token, two launches otherwise
        return ops.quantized_linear(
            x, permutation, signs, act_boundaries, act_centroids, packed_weight_indices, row_norms,
            weight_centroids, block_size=block_size, eps=eps, inv_sqrt_block=inv_sqrt_block,
            activation_bits=activation_bits, weight_bits=weight_bits, out_features=out_features, bias=bias,
            input_map=input_map, output_map=output_map, plan=rotate_plan)
    _, unit, norms = ops.rotate_quantize(
        x, permutation, signs, act_boundaries, block_size=block_size, eps=eps,
        inv_sqrt_block=inv_sqrt_block, centroids=act_centroids, code_format=None, values="unit_bf16",
        input_map=input_map, plan=rotate_plan)
    out = ops.matmul_packed_weight_values(
        unit, packed_weight_indices, row_norms, weight_centroids, bits=weight_bits,
        out_features=out_features, in_features=in_features, bias=bias,
        token_scale=norms.reshape(-1), output_dtype=x.dtype)
    if output_map is not None:   # rare shapes only: plain gather through the table
        out = output_map[out.view(torch.int16).to(torch.int32) & 0xFFFF]
    return out


def _quantized_linear_fake(
    x, permutation, signs, act_centroids, act_boundaries, packed_weight_indices, row_norms,
    weight_centroids, bias, block_size, eps, inv_sqrt_block, activation_bits, weight_bits, out_features,
    input_map=None, output_map=None, rotate_plan=None,
):
    return x.new_empty((*x.shape[:-1], out_features))


_LIB.impl("quantized_linear", quantized_linear_forward, "CUDA")
torch.library.register_fake("orbitquant_amd::quantized_linear", _quantized_linear_fake, lib=_LIB)


def packed_length(value_count: int, bits: int) -> int:
    return (value_count * bits + 7) // 8


_last_quantization: dict = {}  # the one entry of OrbitLinear._forward_shared


class OrbitLinear(nn.Module):
    def __init__(
        self,
        *,
        in_features: int,
        out_features: int,
        config: OrbitQuantConfig,
        bias: torch.Tensor | None,
        packed_weight_indices: torch.Tensor,
        row_norms: torch.Tensor,
        module_name: str = "",
    ) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight_bits = config.weight_bits
        self.activation_bits = config.activation_bits
        self.activation_eps = config.activation_eps
        self.module_name = module_name
        self.rotation = get_rpbh_rotation(in_features, config.rotation_seed, config.block_size)
        self.weight_codebook = get_codebook(in_features, config.weight_bits, config.codebook_version)
        self.activation_codebook = get_codebook(in_features, config.activation_bits, config.codebook_version)
        expected = packed_length(out_features * in_features, config.weight_bits)
        if packed_weight_indices.dtype != torch.uint8 or packed_weight_indices.numel() != expected:
            raise ValueError(f"packed_weight_indices must be uint8 with {expected} bytes")
        if row_norms.dtype != torch.bfloat16 or tuple(row_norms.shape) != (out_features,):
            raise ValueError("row_norms must be bfloat16 with shape (out_features,)")
        self.packed_weight_indices = nn.Parameter(packed_weight_indices.detach().flatten(), requires_grad=False)
        self.row_norms = nn.Parameter(row_norms.detach(), requires_grad=False)
        if bias is None:
            self.register_parameter("bias", None)
        else:
            self.bias = nn.Parameter(bias.detach().clone(), requires_grad=False)
        device = packed_weight_indices.device
        for name, tensor in self._constants().items():
            self.register_buffer(name, tensor.to(device), persistent=False)
        self.register_buffer("_rotation_plan", None, persistent=False)
        self._build_rotation_plan()
        self.last_effective_runtime_mode: str | None = None
        self._input_activation = None  # (fn, dtype) once fuse_input_activation() was called
        self.register_buffer("_input_activation_table", None, persistent=False)
        self._output_activation = None
        self.register_buffer("_output_activation_table", None, persistent=False)
        # Linears that read the same tensor (q, k and v of an attention block; gate and up of an MLP) can
        # share its quantization: set this on each of them and the codes the first one computes serve the
        # others (see _shared_codes).  Off by default: the reference quantizes per layer.
        self.share_input_quantization = False
        # 2- and 3-bit weights, many tokens: the tile kernel can read a copy of the indices repacked at four
        # bits each (see _matmul_weight), 7-17 % faster there.  OFF by default, because the copy costs
        # out*in/2 bytes on top of the stored stream: a 2-bit layer then holds 0.75 instead of 0.25 byte per
        # weight (3x), a 3-bit layer 0.875 instead of 0.375 (2.3x) - most of what low-bit weights save.
        self.nibble_copy_for_many_tokens = False
        self.register_buffer("_nibble_weight_copy", None, persistent=False)
        self.register_buffer("_nibble_weight_centroids", None, persistent=False)
        self._nibble_copy_of = None   # (address, version) of the packed_weight_indices the copy was made from

    MANY_TOKENS = 65   # from here on the matmul is the tile kernel (up to 64 tokens: the streaming kernel)

    def prepare_many_token_weights(self) -> None:
        """Build the four-bit copy of a 2- or 3-bit index stream now (it is otherwise built by the first
        forward of at least `MANY_TOKENS` rows; a forward that `torch.compile` is tracing cannot build
        it and runs on the stored stream)."""
        if self.weight_bits not in (2, 3) or self.packed_weight_indices.device.type != "cuda":
            return
        with torch.no_grad():
            count = self.out_features * self.in_features
            indices = ops.unpack_lowbit(self.packed_weight_indices.detach(), self.weight_bits, count)
            self._nibble_weight_copy = ops.pack_lowbit(indices, 4)
            cents = torch.zeros(16, dtype=torch.float32, device=indices.device)
            cents[: 1 << self.weight_bits] = self._weight_codebook_centroids
            self._nibble_weight_centroids = cents
            self._nibble_copy_of = self._stored_stream_identity()

    def _stored_stream_identity(self):
        """What tells one state of the stored index stream from another: its address and torch's version
        counter (None for the counter of an inference tensor, which has none: the address alone then)."""
        w = self.packed_weight_indices
        return (w.data_ptr(), None if w.is_inference() else w._version)

    def _matmul_weight(self, tokens: int):
        """(packed indices, bits per index, centroids) the matmul of `tokens` rows reads.  The stored
        stream, except for 2- and 3-bit weights at `MANY_TOKENS` rows or more: the tile kernel is bound
        by instruction issue there, not by weight bytes, and extracting 3-bit fields that straddle bytes
        (or four 2-bit fields per byte) costs it 11-22 % against whole nibbles, so it is given the same
        indices at four bits each, with the codebook padded to sixteen entries.  Same operand values,
        same sums.  Measured from 65 tokens (7-17 % there) to several thousand.  Calls of up to 64 tokens
        take the streaming kernel, which is bound by decode work per byte, and keep reading the stored stream."""
        if (self.weight_bits in (2, 3) and self.nibble_copy_for_many_tokens and tokens >= self.MANY_TOKENS
                and self.packed_weight_indices.device.type == "cuda"):
            if not torch.compiler.is_compiling():   # (a forward being traced neither checks nor builds the copy)
                stale = self._nibble_weight_copy is not None and self._nibble_copy_of != self._stored_stream_identity()
                if self._nibble_weight_copy is None or stale:
                    self.prepare_many_token_weights()   # (also after an in-place update of the stored stream)
            if self._nibble_weight_copy is not None:
                return self._nibble_weight_copy, 4, self._nibble_weight_centroids
        return self.packed_weight_indices, self.weight_bits, self._weight_codebook_centroids

    def _load_from_state_dict(self, *args, **kwargs):
        self._nibble_weight_copy = None   # follows packed_weight_indices
        self._nibble_weight_centroids = None
        return super()._load_from_state_dict(*args, **kwargs)

    def fuse_input_activation(self, fn, *, dtype: torch.dtype = torch.bfloat16) -> "OrbitLinear":
        """Make forward(x) return what forward(fn(x)) returns, bit for bit, without a separate
        elementwise kernel and without fn(x) being written to memory: fn (elementwise, e.g. the
        GELU between the two linears of an MLP) is handed to the quantize kernel as the table of
        its values on all 65536 inputs of `dtype`, filled here by fn itself.  Inputs of another
        dtype are refused.  `fn=None` undoes it."""
        if fn is None:
            self._input_activation = None
            self._input_activation_table = None
            return self
        self._input_activation = (fn, dtype)
        self._input_activation_table = ops.activation_table(fn, dtype, self.packed_weight_indices.device)
        return self

    def fuse_output_activation(self, fn, *, dtype: torch.dtype = torch.bfloat16) -> "OrbitLinear":
        """Make forward(x) return fn(forward(x)), bit for bit, without a separate elementwise kernel:
        fn (elementwise; the activation that follows this linear) is applied as a table lookup to every
        output value right before it is stored.  This is the cheaper side to fuse an activation on
        (the matmul's epilogue waits for its stores anyway); `fuse_input_activation` on the next layer is
        for when this layer is not an OrbitLinear.  Inputs must have dtype `dtype`; `fn=None` undoes it."""
        if fn is None:
            self._output_activation = None
            self._output_activation_table = None
            return self
        self._output_activation = (fn, dtype)
        self._output_activation_table = ops.activation_table(fn, dtype, self.packed_weight_indices.device)
        return self

    def _build_rotation_plan(self) -> None:
        """What the quantize kernel can precompute from the layer's constants (`ops.rotate_plan`);
        exists only while the module sits on a GPU."""
        if self._rotation_permutation.device.type != "cuda":
            self._rotation_plan = None
            return
        self._rotation_plan = ops.rotate_plan(
            self._rotation_permutation, self._rotation_signs, self._activation_codebook_boundaries,
            block_size=self.rotation.block_size, inv_sqrt_block=self.rotation.normalization)

    def _constants(self) -> dict[str, torch.Tensor]:
        return {
            "_rotation_permutation": self.rotation.permutation.to(torch.int32),
            "_rotation_signs": self.rotation.signs.to(torch.int8),
            "_activation_codebook_centroids": self.activation_codebook.centroids.clone(),
            "_activation_codebook_boundaries": self.activation_codebook.boundaries.clone(),
            "_weight_codebook_centroids": self.weight_codebook.centroids.clone(),
        }

    @classmethod
    def from_weight(cls, weight, *, bias, config: OrbitQuantConfig, module_name: str = "") -> "OrbitLinear":
        out_features, in_features = weight.shape
        rotation = get_rpbh_rotation(in_features, config.rotation_seed, config.block_size)
        codebook = get_codebook(in_features, config.weight_bits, config.codebook_version)
        packed, row_norms = quantize_weight(
            weight, rotation=rotation, codebook=codebook, bits=config.weight_bits,
            eps=config.activation_eps, row_tile=config.weight_row_tile_size)
        device = weight.device
        return cls(
            in_features=in_features, out_features=out_features, config=config,
            bias=None if bias is None else bias.detach(),
            packed_weight_indices=packed.to(device), row_norms=row_norms.to(device),
            module_name=module_name)

    @classmethod
    def empty_from_linear(cls, layer: nn.Linear, *, config: OrbitQuantConfig, module_name: str = "") -> "OrbitLinear":
        """A skeleton with the right tensor shapes for a packed state dict to be loaded into
        (src/orbitquant/layers.py:510-561 of the reference); the constants (rotation, codebooks,
        rotate plan) are those of (in_features, config) already."""
        if not isinstance(layer, nn.Linear):
            raise TypeError(f"no OrbitQuant linear adapter registered for {type(layer).__name__}")
        n, k = layer.out_features, layer.in_features
        device = layer.weight.device
        bias = None if layer.bias is None else torch.zeros(n, dtype=layer.bias.dtype, device=device)
        return cls(
            in_features=k, out_features=n, config=config, bias=bias,
            packed_weight_indices=torch.zeros(packed_length(n * k, config.weight_bits), dtype=torch.uint8, device=device),
            row_norms=torch.zeros(n, dtype=torch.bfloat16, device=device), module_name=module_name)

    @classmethod
    def from_linear(cls, layer: nn.Linear, *, config: OrbitQuantConfig, module_name: str = "") -> "OrbitLinear":
        if not isinstance(layer, nn.Linear):
            raise TypeError(f"no OrbitQuant linear adapter registered for {type(layer).__name__}")
        return cls.from_weight(layer.weight.detach(), bias=layer.bias, config=config, module_name=module_name)

    def _apply(self, fn, recurse: bool = True):
        result = super()._apply(fn, recurse=recurse)
        # integer / fp32 constants must survive .to(dtype=...) casts unchanged
        device = self.packed_weight_indices.device
        for name, tensor in self._constants().items():
            setattr(self, name, tensor.to(device))
        self._build_rotation_plan()
        self._nibble_weight_copy = None   # rebuilt on the new device / from uncast centroids when next needed
        self._nibble_weight_centroids = None
        if self._input_activation is not None and device.type == "cuda":
            # a dtype cast must not touch the table's bits: fill it again
            self._input_activation_table = ops.activation_table(*self._input_activation, device)
        if self._output_activation is not None and device.type == "cuda":
            self._output_activation_table = ops.activation_table(*self._output_activation, device)
        return result

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape[-1] != self.in_features:
            raise ValueError(f"expected last dimension {self.in_features}, got {x.shape[-1]}")
        if x.device.type != "cuda":
            raise RuntimeError(
                "OrbitLinear runs on AMD GPUs only (torch device 'cuda'); there is no CPU fallback")
        if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            raise ValueError("x must be float32, float16 or bfloat16")
        table = self._input_activation_table
        if table is not None and table.dtype != x.dtype:
            raise ValueError(f"the fused input activation was built for {table.dtype}, got {x.dtype}")
        out_table = self._output_activation_table
        if out_table is not None and out_table.dtype != x.dtype:
            raise ValueError(f"the fused output activation was built for {out_table.dtype}, got {x.dtype}")
        self.last_effective_runtime_mode = "hip_packed"
        if self.share_input_quantization and not torch.compiler.is_compiling():
            return self._forward_shared(x, table, out_table)
        packed, weight_bits, weight_centroids = self._matmul_weight(x.numel() // self.in_features)
        return torch.ops.orbitquant_amd.quantized_linear(
            x, self._rotation_permutation, self._rotation_signs, self._activation_codebook_centroids,
            self._activation_codebook_boundaries, packed, self.row_norms,
            weight_centroids, self.bias, self.rotation.block_size,
            self.activation_eps, self.rotation.normalization, self.activation_bits, weight_bits,
            self.out_features, table, out_table, self._rotation_plan)

    def _forward_shared(self, x, table, out_table):
        """The forward as quantize + packed linear, with the codes of the most recent quantization kept
        (one entry, process-wide): a layer whose input is the same tensor, unchanged (same storage
        address, shape, dtype and version counter), quantized by the same rotation and codebook, skips
        its quantizer.  Same kernels as the fused op, so the same output bits.  The entry holds a
        reference to the input, so its address cannot be handed to another tensor meanwhile; writes
        to the input that bypass torch's version counter (a raw-pointer kernel refilling a static buffer)
        are not seen: such callers use `OrbitLinearGroup`, which shares by construction.  Inputs created
        under `torch.inference_mode()` and calls on a capturing stream are never served from the entry."""
        fmt = "nibble" if self.activation_bits <= 4 else "u8"
        # The entry is reused only when nothing can have changed unseen: an inference tensor has no version
        # counter (asking for it raises), and a stream under capture replays later on other contents, so
        # both always quantize; strides and the stream are part of the key (codes made on one stream
        # are not handed to another without an event).
        stream = torch.cuda.current_stream(x.device)
        cacheable = not x.is_inference() and not torch.cuda.is_current_stream_capturing()
        key = (x.data_ptr(), x._version if cacheable else None, tuple(x.shape), tuple(x.stride()), x.dtype, x.device,
               stream.cuda_stream, self.in_features, self.rotation.seed,
               self.rotation.block_size, self.activation_bits, self.activation_eps,
               None if table is None else table.data_ptr())
        entry = _last_quantization
        if cacheable and entry.get("key") == key:
            codes, norms = entry["codes"], entry["norms"]
        else:
            codes, _, norms = ops.rotate_quantize(
                x, self._rotation_permutation, self._rotation_signs, self._activation_codebook_boundaries,
                block_size=self.rotation.block_size, eps=self.activation_eps, inv_sqrt_block=self.rotation.normalization,
                code_format=fmt, input_map=table, plan=self._rotation_plan)
            if cacheable:
                entry.update(key=key, codes=codes, norms=norms, keep=x)
            else:
                entry.clear()
        bias = self.bias
        if bias is not None and bias.dtype != x.dtype:
            bias = bias.to(x.dtype)   # as the fused op (and the reference on accelerators) does
        packed, weight_bits, weight_centroids = self._matmul_weight(x.numel() // self.in_features)
        return ops.packed_linear(codes, norms, self._activation_codebook_centroids, packed, self.row_norms,
                                 weight_centroids, code_format=fmt, activation_bits=self.activation_bits,
                                 weight_bits=weight_bits, out_features=self.out_features, in_features=self.in_features,
                                 bias=bias, output_dtype=x.dtype, output_map=out_table)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"w{self.weight_bits}a{self.activation_bits}, block={self.rotation.block_size}")


class OrbitLinearGroup:
    """Linears that read the same input (q, k and v of an attention block; gate and up of an MLP),
    called together: `q, k, v = OrbitLinearGroup(attn.q, attn.k, attn.v)(x)`.

    The whole group is one native call (`oq_quantized_linear_group`): the input is quantized once,
    and the packed linears of at most 32 tokens are one launch.  Every output equals the module's
    own `forward(x)` bit for bit.  The group holds references to the modules, not copies, and is not
    itself a module: parameters and state dict stay where they are.  The members must share
    `in_features`, rotation, activation width and fused input activation; under `torch.compile`, or
    when a member has a fused output activation, the members are simply called one after the other.
    The reference has no counterpart: its layers each quantize and multiply on their own
    (src/orbitquant/layers.py:1079-1455)."""

    def __init__(self, *linears: OrbitLinear) -> None:
        if len(linears) < 1 or not all(isinstance(l, OrbitLinear) for l in linears):
            raise TypeError("OrbitLinearGroup takes OrbitLinear modules")
        first = linears[0]
        for l in linears[1:]:
            same = (l.in_features == first.in_features and l.rotation.seed == first.rotation.seed
                    and l.rotation.block_size == first.rotation.block_size
                    and l.activation_bits == first.activation_bits and l.activation_eps == first.activation_eps
                    and l._input_activation == first._input_activation)
            if not same:
                raise ValueError("the linears of a group must share in_features, rotation, activation width, "
                                 "eps and fused input activation")
        self.linears = tuple(linears)

    def __call__(self, x: torch.Tensor) -> tuple[torch.Tensor, ...]:
        first = self.linears[0]
        if torch.compiler.is_compiling() or any(l._output_activation_table is not None for l in self.linears):
            return tuple(l(x) for l in self.linears)
        if x.shape[-1] != first.in_features:
            raise ValueError(f"expected last dimension {first.in_features}, got {x.shape[-1]}")
        if x.device.type != "cuda":
            raise RuntimeError(
                "OrbitLinear runs on AMD GPUs only (torch device 'cuda'); there is no CPU fallback")
        if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            raise ValueError("x must be float32, float16 or bfloat16")
        table = first._input_activation_table
        if table is not None and table.dtype != x.dtype:
            raise ValueError(f"the fused input activation was built for {table.dtype}, got {x.dtype}")
        weights = []
        for l in self.linears:
            l.last_effective_runtime_mode = "hip_packed"
            bias = l.bias
            if bias is not None and bias.dtype != x.dtype:
                bias = bias.to(x.dtype)   # as the single layer's forward does
            packed, weight_bits, weight_centroids = l._matmul_weight(x.numel() // first.in_features)
            weights.append((packed, l.row_norms, weight_centroids, weight_bits, l.out_features, bias))
        return tuple(ops.quantized_linear_group(
            x, first._rotation_permutation, first._rotation_signs, first._activation_codebook_boundaries,
            first._activation_codebook_centroids, weights, block_size=first.rotation.block_size,
            eps=first.activation_eps, inv_sqrt_block=first.rotation.normalization,
            activation_bits=first.activation_bits, input_map=table, plan=first._rotation_plan))
