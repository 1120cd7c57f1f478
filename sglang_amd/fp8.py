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


class Fp8Linear(torch.nn.Module):
    """One linear layer of an FP8 checkpoint on one tensor-parallel rank.

    `output_sizes` lists the merged projections (one entry for a plain layer; [gate, up] or [q, k, v] sizes for merged
    ones), all BEFORE tensor-parallel splitting.  `parallel` says how the layer is split over `tp_size` ranks: "column"
    (each projection's output channels), "row" (input features) or None (replicated).  The constructor checks what the
    reference checks in create_weights (fp8.py:244-268): a row-parallel K slice and every column-parallel or merged
    projection must be whole quantization blocks, otherwise a block of scales would straddle two shards.
    """

    def __init__(self, input_size: int, output_sizes: Sequence[int], quant_config: Fp8Config, *, parallel: Optional[str] = None,
                 tp_rank: int = 0, tp_size: int = 1, params_dtype: torch.dtype = torch.bfloat16, bias: bool = False,
                 device: Optional[torch.device] = None) -> None:
        super().__init__()
        if parallel not in (None, "column", "row"):
            raise ValueError(f"parallel must be None, 'column' or 'row', got {parallel!r}")
        if not 0 <= tp_rank < tp_size:
            raise ValueError(f"tp_rank {tp_rank} outside tp_size {tp_size}")
        if parallel is None:
            tp_rank, tp_size = 0, 1
        self.quant_config = quant_config
        self.block_quant = quant_config.weight_block_size is not None
        self.parallel, self.tp_rank, self.tp_size = parallel, tp_rank, tp_size
        self.input_size, self.output_sizes = int(input_size), [int(v) for v in output_sizes]
        self.params_dtype = params_dtype
        col, row = (tp_size if parallel == "column" else 1), (tp_size if parallel == "row" else 1)
        if self.input_size % row or any(v % col for v in self.output_sizes):
            raise ValueError("layer sizes are not divisible by the tensor-parallel size")
        self.input_size_per_partition = self.input_size // row
        self.output_partition_sizes = [v // col for v in self.output_sizes]
        self.output_size_per_partition = sum(self.output_partition_sizes)
        self.logical_widths = list(self.output_partition_sizes)
        n, k = self.output_size_per_partition, self.input_size_per_partition
        if self.block_quant:
            block_n, block_k = quant_config.weight_block_size
            if row > 1 and k % block_k != 0:
                raise ValueError(f"Weight input_size_per_partition = {k} is not divisible by weight quantization block_k = {block_k}.")
            if col > 1 or len(self.output_sizes) > 1:
                for v in self.output_partition_sizes:
                    if v % block_n != 0:
                        raise ValueError(f"Weight output_partition_size = {v} is not divisible by weight quantization block_n = {block_n}.")
        P = lambda t: torch.nn.Parameter(t, requires_grad=False)
        self.serialized = quant_config.is_checkpoint_fp8_serialized
        self.weight = P(torch.empty(n, k, dtype=FP8 if self.serialized else params_dtype, device=device))
        lowest = torch.finfo(torch.float32).min  # "not loaded yet", as the reference marks scales
        if not self.serialized:
            # a 16-bit checkpoint: the weight is loaded as it is and quantized in process_weights_after_loading
            # (fp8.py:293-295, :368-383); Fp8Config refuses block quantization for such a checkpoint
            self.weight_scale = None
            self.input_scale = None
        elif self.block_quant:
            self.weight_scale_inv = P(torch.full((_ceil_div(n, block_n), _ceil_div(k, block_k)), lowest, dtype=torch.float32, device=device))
            self.input_scale = None
        else:
            self.weight_scale = P(torch.full((len(self.output_sizes),), lowest, dtype=torch.float32, device=device))
            self.input_scale = (P(torch.full((len(self.output_sizes),), lowest, dtype=torch.float32, device=device))
                                if quant_config.activation_scheme == "static" else None)
        self.bias = P(torch.zeros(n, dtype=params_dtype, device=device)) if bias else None
        self._processed = False

    # ------------------------------------------------------------------ loading

    def _shard_range(self, shard: Optional[int], block: int) -> tuple:
        """(offset, size) along the output dimension of this rank's parameter for merged projection `shard` (None: the
        whole parameter), in units of `block` output channels (1 for weights and biases, block_n for block scales)."""
        if shard is None:
            return 0, _ceil_div(self.output_size_per_partition, block)
        return _ceil_div(sum(self.output_partition_sizes[:shard]), block), _ceil_div(self.output_partition_sizes[shard], block)

    def weight_loader(self, name: str, loaded: torch.Tensor, shard: Optional[int] = None) -> None:
        """Copy this rank's slice of checkpoint tensor `loaded` into parameter `name` ("weight", "weight_scale_inv",
        "weight_scale", "input_scale", "bias").  `shard` selects the merged projection the tensor belongs to; a tensor that
        already holds all merged projections is loaded with shard=None on an unsplit layer."""
        param = getattr(self, name, None)
        if param is None:
            raise KeyError(f"this layer has no parameter {name!r}")
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
        """Load every parameter from a mapping of checkpoint names to tensors.  One prefix ("model.layers.0.mlp.down_proj")
        for a plain layer; one per merged projection, in `output_sizes` order (["….gate_proj", "….up_proj"]), for a merged
        one.  Missing weights or scales raise KeyError."""
        if len(prefixes) not in (1, len(self.output_sizes)):
            raise ValueError("one prefix, or one per merged projection")
        names = ["weight"] + ([] if not self.serialized else ["weight_scale_inv"] if self.block_quant else ["weight_scale"])
        if self.input_scale is not None:
            names.append("input_scale")
        if self.bias is not None:
            names.append("bias")
        for i, prefix in enumerate(prefixes):
            shard = i if len(prefixes) > 1 else (0 if len(self.output_sizes) == 1 else None)
            for name in names:
                self.weight_loader(name, tensors[f"{prefix}.{name}"], shard)

    # ------------------------------------------------------------------ after loading, forward

    def process_weights_after_loading(self, requant_ue8m0: bool = False) -> None:
        """fp8.py:343-465.  A 16-bit checkpoint is quantized here, per output channel.  Block-FP8: the tensors stay as loaded (or are re-quantized to
        power-of-two scales: weight_scale_inv becomes packed int32 exponents, fp8_utils.py:428-449).  Per-tensor: one
        scale per merged projection becomes one scale per output channel (what fp8_scaled_mm takes), the weight is kept
        as its [K, N] column-major view, a static input scale is the maximum over the merged projections."""
        if not self.serialized:
            # fp8.py:368-383, the branch of a platform with per-channel FP8 GEMMs: one quantization group per output
            # channel (per_token_group_quant_fp8 with group_size = K), scales as [1, N], no static input scale
            from .fp8_kernel import per_token_group_quant_fp8

            w = self.weight.data.contiguous()
            qweight, weight_scale = per_token_group_quant_fp8(w, w.shape[-1])
            self.weight = torch.nn.Parameter(qweight.t(), requires_grad=False)
            self.weight_scale = torch.nn.Parameter(weight_scale.t().contiguous(), requires_grad=False)
            self.input_scale = None
            self._processed = True
            return
        lowest = torch.finfo(torch.float32).min
        scale = self.weight_scale_inv if self.block_quant else self.weight_scale
        if bool((scale.data == lowest).any()) or (self.input_scale is not None and bool((self.input_scale.data == lowest).any())):
            raise RuntimeError("process_weights_after_loading: some scales were never loaded")
        if self.block_quant:
            if requant_ue8m0:
                from .fp8_utils import requant_weight_ue8m0

                if list(self.quant_config.weight_block_size) != [128, 128]:
                    raise NotImplementedError("power-of-two requantization is built for 128 x 128 blocks")
                w, s = requant_weight_ue8m0(self.weight.data, self.weight_scale_inv.data, [128, 128])
                self.weight = torch.nn.Parameter(w, requires_grad=False)
                self.weight_scale_inv = torch.nn.Parameter(s, requires_grad=False)
        else:
            widths = torch.tensor(self.logical_widths, device=scale.device)
            per_channel = torch.repeat_interleave(scale.data, widths).reshape(-1, 1)  # convert_to_channelwise
            self.weight = torch.nn.Parameter(self.weight.data.t(), requires_grad=False)
            self.weight_scale = torch.nn.Parameter(per_channel, requires_grad=False)
            if self.input_scale is not None:
                self.input_scale = torch.nn.Parameter(self.input_scale.data.max().reshape(1), requires_grad=False)
        self._processed = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Fp8LinearMethod.apply, fp8.py:467-500.  A row-parallel layer returns this rank's partial sum; the caller
        all-reduces."""
        from . import fp8_utils

        if not self._processed:
            raise RuntimeError("call process_weights_after_loading() first")
        if self.block_quant:
            fn = (fp8_utils.deepgemm_w8a8_block_fp8_linear_with_fallback if self.weight_scale_inv.dtype == torch.int32
                  else fp8_utils.w8a8_block_fp8_linear)
            return fn(input=x, weight=self.weight, block_size=self.quant_config.weight_block_size,
                      weight_scale=self.weight_scale_inv, input_scale=None, bias=self.bias)
        return fp8_utils.apply_fp8_linear(input=x, weight=self.weight, weight_scale=self.weight_scale, input_scale=self.input_scale,
                                          bias=self.bias, use_per_token_if_dynamic=False)


class Fp8LinearMethod:
    """The reference's three-call protocol (fp8.py:198-500) on top of Fp8Linear, for code that is written against it:
    create_weights registers the parameters on `layer`, process_weights_after_loading finishes them, apply runs the GEMM."""

    def __init__(self, quant_config: Fp8Config) -> None:
        self.quant_config = quant_config
        self.block_quant = quant_config.weight_block_size is not None

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int, output_partition_sizes: List[int],
                       input_size: int, output_size: int, params_dtype: torch.dtype, **extra) -> None:
        tp_col = output_size // sum(output_partition_sizes)
        tp_row = input_size // input_size_per_partition
        parallel, tp = ("column", tp_col) if tp_col > 1 else (("row", tp_row) if tp_row > 1 else (None, 1))
        col = tp if parallel == "column" else 1
        layer.fp8 = Fp8Linear(input_size, [v * col for v in output_partition_sizes], self.quant_config, parallel=parallel,
                              tp_rank=int(extra.get("tp_rank", 0)), tp_size=tp, params_dtype=params_dtype,
                              device=extra.get("device"))
        layer.logical_widths = output_partition_sizes
        layer.input_size_per_partition = input_size_per_partition
        layer.output_size_per_partition = sum(output_partition_sizes)
        layer.orig_dtype = params_dtype

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        layer.fp8.process_weights_after_loading()

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        out = layer.fp8(x)
        return out if bias is None else out + bias


def load_safetensors_dir(path: str) -> Dict[str, torch.Tensor]:
    """All tensors of the *.safetensors files in a checkpoint directory, on the CPU (small checkpoints and tests; a
    serving loader would stream tensor by tensor)."""
    from safetensors.torch import load_file

    out: Dict[str, torch.Tensor] = {}
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".safetensors"):
            out.update(load_file(os.path.join(path, fn)))
    return out
