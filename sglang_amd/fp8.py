"""FP8 checkpoints into the gfx950 linear kernels: the quantization config, the parameters a linear layer registers, how the
tensors of an FP8-serialized checkpoint are sliced into them (merged projections, tensor-parallel shards), what happens
after loading, and the forward call.

What the reference spreads over `Fp8Config` / `Fp8LinearMethod` (python/sglang/srt/layers/quantization/fp8.py:115-195,
:198-500), the linear layers' weight loaders (python/sglang/srt/layers/linear.py:707-760 merged columns, :953-985 q/k/v,
row-parallel :1300-1330) and the parameter classes (python/sglang/srt/layers/parameter.py:100-190, :316-322) is one small
module here, because only the data format matters for this path:

  block-FP8 layer (DeepSeek-V3 style)        weight            e4m3fn [N, K]
                                             weight_scale_inv  fp32   [ceil(N / 128), ceil(K / 128)]
  per-tensor FP8 layer                       weight            e4m3fn [N, K]
                                             weight_scale      fp32   one per merged projection
                                             input_scale       fp32   one per merged projection (static activations only)

On gfx950 the checkpoint's OCP e4m3fn bytes are what the matrix instructions consume, so nothing is re-encoded after
loading (the reference's ROCm branch converts to e4m3fnuz for older parts, fp8.py:346-353).  Optionally a block-FP8 layer
is re-quantized to power-of-two scales (`requant_ue8m0=True`, fp8_utils.py:428-449), which lets the large-M GEMM apply
the scales inside the MFMA.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Sequence

import torch

ACTIVATION_SCHEMES = ["static", "dynamic"]
FP8 = torch.float8_e4m3fn


def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


@dataclass
class Fp8Config:
    """fp8.py:115-178: `quantization_config` of an FP8 checkpoint's config.json."""

    is_checkpoint_fp8_serialized: bool = False
    activation_scheme: str = "dynamic"
    ignored_layers: List[str] = field(default_factory=list)
    weight_block_size: Optional[List[int]] = None

    def __post_init__(self) -> None:
        if self.activation_scheme not in ACTIVATION_SCHEMES:
            raise ValueError(f"Unsupported activation scheme {self.activation_scheme}")
        self.ignored_layers = list(self.ignored_layers or [])
        if self.weight_block_size is not None:
            if not self.is_checkpoint_fp8_serialized:
                raise ValueError("The block-wise quantization only supports fp8-serialized checkpoint for now.")
            if len(self.weight_block_size) != 2:
                raise ValueError(
                    f"The quantization block size of weight must have 2 dimensions, but got {len(self.weight_block_size)} dimensions.")
            if self.activation_scheme != "dynamic":
                raise ValueError(
                    "The block-wise quantization only supports dynamic activation scheme for now, but got "
                    f"{self.activation_scheme} activation scheme.")
            self.weight_block_size = [int(v) for v in self.weight_block_size]

    @classmethod
    def get_name(cls) -> str:
        return "fp8"

    @classmethod
    def from_config(cls, config: Mapping[str, Any]) -> "Fp8Config":
        if "quant_method" not in config or "activation_scheme" not in config:
            raise ValueError("quantization config needs 'quant_method' and 'activation_scheme'")
        return cls(
            is_checkpoint_fp8_serialized="fp8" in config["quant_method"],
            activation_scheme=config["activation_scheme"],
            ignored_layers=config.get("ignored_layers") or [],
            weight_block_size=config.get("weight_block_size"),
        )

    @classmethod
    def from_checkpoint_dir(cls, path: str) -> "Fp8Config":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_config(json.load(f)["quantization_config"])

    def is_layer_skipped(self, prefix: str) -> bool:
        return any(prefix == name or prefix.startswith(name + ".") for name in self.ignored_layers)


def default_weight_loader(param: torch.nn.Parameter, loaded_weight: torch.Tensor, loaded_shard_id: Optional[int] = None) -> None:
    """Loader of a layer that is neither merged nor split: the checkpoint tensor is the parameter."""
    if tuple(param.shape) != tuple(loaded_weight.shape) and loaded_weight.numel() != param.numel():
        raise ValueError(f"checkpoint tensor {tuple(loaded_weight.shape)} does not fit parameter {tuple(param.shape)}")
    param.data.copy_(loaded_weight.reshape(param.shape))


class Fp8LinearMethod:
    """The reference's three-call protocol (fp8.py:198-500): `create_weights` registers `weight`, `weight_scale_inv` or
    `weight_scale`, and `input_scale` ON `layer` under those names (so `layer.named_parameters()` lists the checkpoint's
    own keys), each carrying the `weight_loader` the layer passed in plus `input_dim` / `output_dim` as the reference's
    parameter classes do (parameter.py:100-190); `process_weights_after_loading` finishes them; `apply` runs the GEMM.

    The method never guesses the tensor-parallel layout: it is given partition sizes, as in the reference, and `tp_size`
    (the reference reads a process-global, fp8.py:245) only decides which block-alignment checks apply.
    `requant_ue8m0` stands for the reference's `should_deepgemm_weight_requant_ue8m0` (fp8.py:403-408): block-FP8 weights
    are re-quantized to power-of-two scales after loading."""

    def __init__(self, quant_config: Fp8Config, *, tp_size: int = 1, requant_ue8m0: bool = False) -> None:
        self.quant_config = quant_config
        self.block_quant = quant_config.weight_block_size is not None
        self.tp_size = int(tp_size)
        self.requant_ue8m0 = bool(requant_ue8m0)

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int, output_partition_sizes: List[int],
                       input_size: int, output_size: int, params_dtype: torch.dtype, **extra_weight_attrs) -> None:
        cfg = self.quant_config
        output_size_per_partition = sum(output_partition_sizes)
        weight_loader = extra_weight_attrs.get("weight_loader") or default_weight_loader
        device = extra_weight_attrs.get("device")
        n, k = output_size_per_partition, input_size_per_partition
        if self.block_quant:  # fp8.py:246-268
            block_n, block_k = cfg.weight_block_size
            if self.tp_size > 1 and input_size // k == self.tp_size and k % block_k != 0:
                raise ValueError(f"Weight input_size_per_partition = {k} is not divisible by weight quantization block_k = {block_k}.")
            if (self.tp_size > 1 and output_size // n == self.tp_size) or len(output_partition_sizes) > 1:
                for v in output_partition_sizes:
                    if v % block_n != 0:
                        raise ValueError(f"Weight output_partition_size = {v} is not divisible by weight quantization block_n = {block_n}.")
        layer.logical_widths = list(output_partition_sizes)
        layer.input_size_per_partition = k
        layer.output_size_per_partition = n
        layer.orig_dtype = params_dtype

        def register(name: str, data: torch.Tensor, **attrs) -> None:
            param = torch.nn.Parameter(data, requires_grad=False)
            param.weight_loader = weight_loader
            for key, value in attrs.items():
                setattr(param, key, value)
            layer.register_parameter(name, param)

        serialized = cfg.is_checkpoint_fp8_serialized
        register("weight", torch.empty(n, k, dtype=FP8 if serialized else params_dtype, device=device), input_dim=1, output_dim=0)
        lowest = torch.finfo(torch.float32).min  # "not loaded yet", as the reference marks scales
        if not serialized:
            # a 16-bit checkpoint: the weight is loaded as it is and quantized in process_weights_after_loading
            # (fp8.py:293-295, :368-383); Fp8Config refuses block quantization for such a checkpoint
            layer.register_parameter("weight_scale", None)
            layer.register_parameter("input_scale", None)
            return
        if self.block_quant:
            register("weight_scale_inv", torch.full((_ceil_div(n, block_n), _ceil_div(k, block_k)), lowest, dtype=torch.float32, device=device),
                     input_dim=1, output_dim=0)
        else:
            register("weight_scale", torch.full((len(output_partition_sizes),), lowest, dtype=torch.float32, device=device))
        if cfg.activation_scheme == "static":
            register("input_scale", torch.full((len(output_partition_sizes),), lowest, dtype=torch.float32, device=device))
        else:
            layer.register_parameter("input_scale", None)

    def process_weights_after_loading(self, layer: torch.nn.Module, requant_ue8m0: Optional[bool] = None) -> None:
        """fp8.py:343-465.  A 16-bit checkpoint is quantized here, per output channel.  Block-FP8: the tensors stay as
        loaded, or are re-quantized to power-of-two scales (weight_scale_inv becomes packed int32 exponents,
        fp8_utils.py:428-449).  Per-tensor: one scale per merged projection becomes one scale per output channel (what
        fp8_scaled_mm takes), the weight is kept as its [K, N] column-major view, a static input scale is the maximum
        over the merged projections."""
        P = lambda t: torch.nn.Parameter(t, requires_grad=False)
        if not self.quant_config.is_checkpoint_fp8_serialized:
            # fp8.py:368-383, the branch of a platform with per-channel FP8 GEMMs: one quantization group per output
            # channel (per_token_group_quant_fp8 with group_size = K), scales as [1, N], no static input scale
            from .fp8_kernel import per_token_group_quant_fp8

            w = layer.weight.data.contiguous()
            qweight, weight_scale = per_token_group_quant_fp8(w, w.shape[-1])
            layer.weight = P(qweight.t())
            layer.weight_scale = P(weight_scale.t().contiguous())
            layer.input_scale = None
            return
        lowest = torch.finfo(torch.float32).min
        scale = layer.weight_scale_inv if self.block_quant else layer.weight_scale
        if bool((scale.data == lowest).any()) or (layer.input_scale is not None and bool((layer.input_scale.data == lowest).any())):
            raise RuntimeError("process_weights_after_loading: some scales were never loaded")
        if self.block_quant:
            if self.requant_ue8m0 if requant_ue8m0 is None else requant_ue8m0:
                from .fp8_utils import requant_weight_ue8m0

                if list(self.quant_config.weight_block_size) != [128, 128]:
                    raise NotImplementedError("power-of-two requantization is built for 128 x 128 blocks")
                w, s = requant_weight_ue8m0(layer.weight.data, layer.weight_scale_inv.data, [128, 128])
                layer.weight = P(w)
                layer.weight_scale_inv = P(s)
        else:
            widths = torch.tensor(layer.logical_widths, device=scale.device)
            per_channel = torch.repeat_interleave(scale.data, widths).reshape(-1, 1)  # convert_to_channelwise
            layer.weight = P(layer.weight.data.t())
            layer.weight_scale = P(per_channel)
            if layer.input_scale is not None:
                layer.input_scale = P(layer.input_scale.data.max().reshape(1))

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fp8.py:467-500."""
        from . import fp8_utils

        if self.block_quant:
            fn = (fp8_utils.deepgemm_w8a8_block_fp8_linear_with_fallback if layer.weight_scale_inv.dtype == torch.int32
                  else fp8_utils.dispatch_w8a8_block_fp8_linear())
            return fn(input=x, weight=layer.weight, block_size=self.quant_config.weight_block_size,
                      weight_scale=layer.weight_scale_inv, input_scale=None, bias=bias)
        return fp8_utils.apply_fp8_linear(input=x, weight=layer.weight, weight_scale=layer.weight_scale, input_scale=layer.input_scale,
                                          bias=bias, use_per_token_if_dynamic=False)


class Fp8Linear(torch.nn.Module):
    """One linear layer of an FP8 checkpoint on one tensor-parallel rank: the part of the reference's linear layers
    (linear.py:707-760, :953-985, :1300-1330) that slices checkpoint tensors, around an Fp8LinearMethod.

    `output_sizes` lists the merged projections (one entry for a plain layer; [gate, up] or [q, k, v] sizes for merged
    ones), all BEFORE tensor-parallel splitting.  `parallel` says how the layer is split over `tp_size` ranks: "column"
    (each projection's output channels), "row" (input features) or None (replicated).  The parameters live on this module
    under the checkpoint's names; each carries `weight_loader(param, loaded_weight, loaded_shard_id)`.
    """

    def __init__(self, input_size: int, output_sizes: Sequence[int], quant_config: Fp8Config, *, parallel: Optional[str] = None,
                 tp_rank: int = 0, tp_size: int = 1, params_dtype: torch.dtype = torch.bfloat16, bias: bool = False,
                 device: Optional[torch.device] = None, requant_ue8m0: bool = False) -> None:
        super().__init__()
        if parallel not in (None, "column", "row"):
            raise ValueError(f"parallel must be None, 'column' or 'row', got {parallel!r}")
        if not 0 <= tp_rank < tp_size:
            raise ValueError(f"tp_rank {tp_rank} outside tp_size {tp_size}")
        if parallel is None:
            tp_rank, tp_size = 0, 1
        self.quant_config = quant_config
        self.block_quant = quant_config.weight_block_size is not None
        self.serialized = quant_config.is_checkpoint_fp8_serialized
        self.parallel, self.tp_rank, self.tp_size = parallel, tp_rank, tp_size
        self.input_size, self.output_sizes = int(input_size), [int(v) for v in output_sizes]
        self.params_dtype = params_dtype
        col, row = (tp_size if parallel == "column" else 1), (tp_size if parallel == "row" else 1)
        if self.input_size % row or any(v % col for v in self.output_sizes):
            raise ValueError("layer sizes are not divisible by the tensor-parallel size")
        self.output_partition_sizes = [v // col for v in self.output_sizes]
        self.quant_method = Fp8LinearMethod(quant_config, tp_size=tp_size, requant_ue8m0=requant_ue8m0)
        self.quant_method.create_weights(self, self.input_size // row, self.output_partition_sizes, self.input_size,
                                         sum(self.output_sizes), params_dtype, weight_loader=self.weight_loader, device=device)
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(self.output_size_per_partition, dtype=params_dtype, device=device), requires_grad=False)
            self.bias.weight_loader = self.weight_loader
        else:
            self.register_parameter("bias", None)
        self._processed = False

    # ------------------------------------------------------------------ loading

    def _shard_range(self, shard: Optional[int], block: int) -> tuple:
        """(offset, size) along the output dimension of this rank's parameter for merged projection `shard` (None: the
        whole parameter), in units of `block` output channels (1 for weights and biases, block_n for block scales)."""
        if shard is None:
            return 0, _ceil_div(self.output_size_per_partition, block)
        return _ceil_div(sum(self.output_partition_sizes[:shard]), block), _ceil_div(self.output_partition_sizes[shard], block)

    def weight_loader(self, param, loaded: torch.Tensor, shard: Optional[int] = None) -> None:
        """Copy this rank's slice of checkpoint tensor `loaded` into `param`: one of this layer's parameters, as the
        reference's loaders are called (`param.weight_loader(param, loaded_weight, loaded_shard_id)`), or its name
        ("weight", "weight_scale_inv", "weight_scale", "input_scale", "bias").  `shard` selects the merged projection the
        tensor belongs to; a tensor that already holds all merged projections is loaded with shard=None on an unsplit layer."""
        if isinstance(param, str):
            name, param = param, getattr(self, param, None)
            if param is None:
                raise KeyError(f"this layer has no parameter {name!r}")
        else:
            name = next((n for n, p in self.named_parameters(recurse=False) if p is param), None)
            if name is None:
                raise KeyError("the parameter does not belong to this layer")
        if shard is not None and not 0 <= shard < len(self.output_sizes):
            raise IndexError(f"shard {shard} outside {len(self.output_sizes)} merged projections")
        if name in ("weight_scale", "input_scale"):  # one scalar per merged projection, never split
            if loaded.numel() != 1 and not (shard is None and loaded.numel() == param.numel()):
                raise ValueError(f"{name}: expected one value per merged projection")
            if shard is None:
                param.data.copy_(loaded.reshape(-1).expand(param.numel()) if loaded.numel() == 1 else loaded.reshape(-1))
            else:
                param.data[shard] = loaded.reshape(())
            return
        if shard is None and len(self.output_sizes) > 1 and self.parallel == "column" and self.tp_size > 1:
            raise ValueError("a checkpoint tensor that fuses several projections cannot be split over column-parallel ranks "
                             "without its projection index")
        block_n, block_k = (self.quant_config.weight_block_size if name == "weight_scale_inv" else (1, 1))
        off, size = self._shard_range(shard, block_n)
        dst = param.data.narrow(0, off, size)
        src = loaded
        if self.parallel == "column" and self.tp_size > 1:
            src = src.narrow(0, self.tp_rank * size, size)  # this rank's output channels (or scale block rows)
        if name != "bias" and self.parallel == "row" and self.tp_size > 1:
            cols = dst.shape[1]
            src = src.narrow(1, self.tp_rank * cols, cols)   # this rank's input features (or scale block columns)
        if name == "bias" and self.parallel == "row" and self.tp_rank != 0:
            src = torch.zeros_like(src)                      # the bias is added once, on rank 0, before the all-reduce
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"{name}: checkpoint tensor slice {tuple(src.shape)} does not fit parameter slice {tuple(dst.shape)}")
        dst.copy_(src)

    def load_from(self, tensors: Mapping[str, torch.Tensor], prefixes: Sequence[str]) -> None:
        """Load every parameter from a mapping of checkpoint names to tensors, walking `named_parameters()` as a model
        loader does.  One prefix ("model.layers.0.mlp.down_proj") for a plain layer; one per merged projection, in
        `output_sizes` order (["….gate_proj", "….up_proj"]), for a merged one.  Missing weights or scales raise KeyError."""
        if len(prefixes) not in (1, len(self.output_sizes)):
            raise ValueError("one prefix, or one per merged projection")
        for i, prefix in enumerate(prefixes):
            shard = i if len(prefixes) > 1 else (0 if len(self.output_sizes) == 1 else None)
            for name, param in self.named_parameters(recurse=False):
                param.weight_loader(param, tensors[f"{prefix}.{name}"], shard)

    # ------------------------------------------------------------------ after loading, forward

    def process_weights_after_loading(self, requant_ue8m0: Optional[bool] = None) -> None:
        self.quant_method.process_weights_after_loading(self, requant_ue8m0)
        self._processed = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Fp8LinearMethod.apply, fp8.py:467-500.  A row-parallel layer returns this rank's partial sum; the caller
        all-reduces."""
        if not self._processed:
            raise RuntimeError("call process_weights_after_loading() first")
        return self.quant_method.apply(self, x, self.bias)


def load_safetensors_dir(path: str) -> Dict[str, torch.Tensor]:
    """All tensors of the *.safetensors files in a checkpoint directory, on the CPU (small checkpoints and tests; a
    serving loader would stream tensor by tensor)."""
    from safetensors.torch import load_file

    out: Dict[str, torch.Tensor] = {}
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".safetensors"):
            out.update(load_file(os.path.join(path, fn)))
    return out
