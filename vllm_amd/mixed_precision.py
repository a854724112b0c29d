"""WNA16 linear-kernel interface and its gfx950 Marlin-surface implementation.

Mirrors vllm/model_executor/layers/quantization/kernels/mixed_precision/MPLinearKernel.py:14-94
(MPLinearLayerConfig, MPLinearKernel) and .../mixed_precision/marlin.py:28-166 (MarlinLinearKernel):
same constructor, same `can_implement / process_weights_after_loading / apply_weights` contract,
same parameter names left on the layer, so a vLLM LinearMethod can hold either class.
Differences: `can_implement` accepts a ROCm gfx950 device instead of requiring CUDA, and the types offered
are uint4b8, uint8b128 and uint4 + zero points.
"""
from abc import ABC, abstractmethod
from dataclasses import dataclass

import torch

from . import _custom_ops as ops
from .marlin_utils import (MARLIN_SUPPORTED_GROUP_SIZES, apply_gptq_marlin_linear, check_marlin_supports_shape,
                           marlin_is_k_full, marlin_make_workspace_new, marlin_permute_bias, marlin_permute_scales,
                           marlin_sort_g_idx, marlin_zero_points_from_packed, query_marlin_supported_quant_types)
from .scalar_type import ScalarType


@dataclass
class MPLinearLayerConfig:
    full_weight_shape: tuple[int, int]  # [in, out]
    partition_weight_shape: tuple[int, int]
    weight_type: ScalarType
    act_type: torch.dtype
    group_size: int
    zero_points: bool
    has_g_idx: bool
    out_type: torch.dtype | None = None


def replace_parameter(layer: torch.nn.Module, name: str, new: torch.Tensor) -> None:
    if not isinstance(new, torch.nn.Parameter):
        new = torch.nn.Parameter(new, requires_grad=False)
    if name in layer._parameters:
        del layer._parameters[name]
    elif hasattr(layer, name):
        delattr(layer, name)
    layer.register_parameter(name, new)


def _to_layout(x: torch.Tensor, **dims: int) -> torch.Tensor:
    """vLLM parameters carry input_dim / output_dim / packed_dim; bring them to the layout asked
    for ({input_dim = 0, output_dim = 1[, packed_dim = 0]}).  Plain tensors are taken to be in it."""
    cur_in = getattr(x, "input_dim", None)
    cur_out = getattr(x, "output_dim", None)
    if cur_in is None or cur_out is None:
        return x.data
    if (cur_in, cur_out) == (dims["input_dim"], dims["output_dim"]):
        return x.data
    assert x.data.dim() == 2
    return x.data.t()


class MPLinearKernel(ABC):
    @classmethod
    @abstractmethod
    def get_min_capability(cls) -> int:
        raise NotImplementedError

    @classmethod
    @abstractmethod
    def can_implement(cls, c: MPLinearLayerConfig) -> tuple[bool, str | None]:
        raise NotImplementedError

    def __init__(self, c: MPLinearLayerConfig, w_q_param_name: str, w_s_param_name: str,
                 w_zp_param_name: str | None = None, w_gidx_param_name: str | None = None) -> None:
        assert self.can_implement(c)[0]
        self.config = c
        self.w_q_name = w_q_param_name
        self.w_s_name = w_s_param_name
        if c.zero_points:
            assert w_zp_param_name is not None
        if c.has_g_idx:
            assert w_gidx_param_name is not None
        self.w_zp_name = w_zp_param_name
        self.w_gidx_name = w_gidx_param_name

    @abstractmethod
    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        raise NotImplementedError

    @abstractmethod
    def apply_weights(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        raise NotImplementedError

    def _get_weight_params(self, layer: torch.nn.Module):
        return (getattr(layer, self.w_q_name), getattr(layer, self.w_s_name),
                getattr(layer, self.w_zp_name or "", None), getattr(layer, self.w_gidx_name or "", None))


@dataclass
class MarlinLayerTensors:
    """What the GEMM takes for one layer, all on the weights' device."""
    qweight: torch.Tensor        # int32 [K/16, N * bits / 2], Marlin layout
    scales: torch.Tensor         # [G, N], Marlin order
    zeros: torch.Tensor          # int32 [G, N/8] Marlin packing, or empty
    g_idx: torch.Tensor          # int32 [K] sorted group of each Marlin row, or empty
    sort_indices: torch.Tensor   # int32 [K] column gather for the activations, or empty
    workspace: torch.Tensor
    is_k_full: bool


def prepare_marlin_layer(qweight: torch.Tensor, scales: torch.Tensor, weight_type: ScalarType, size_k: int, size_n: int,
                         group_size: int, zeros_packed: torch.Tensor | None = None, g_idx: torch.Tensor | None = None,
                         row_parallel: bool = False) -> MarlinLayerTensors:
    """Checkpoint tensors of one layer -> GEMM operands, entirely on the device, in four launches at most:
    the act-order sort (torch), the weight repack, the scale permutation and the zero-point conversion (one kernel of
    the library each).  qweight: int32 [K / pack, N] packed along K; scales: [G, N]; zeros_packed: int32 [G, N/8]
    packed along N in natural nibble order; g_idx: int32 [K] group of each input row (act-order) or None."""
    dev = qweight.device
    empty = torch.empty(0, dtype=torch.int32, device=dev)
    sorted_g_idx, sort_indices = (empty, empty) if g_idx is None else marlin_sort_g_idx(g_idx)
    bits = weight_type.size_bits
    groups = 1 if group_size == -1 else size_k // group_size
    return MarlinLayerTensors(
        qweight=ops.gptq_marlin_repack(qweight.contiguous(), sort_indices, size_k, size_n, bits),
        scales=marlin_permute_scales(scales.contiguous(), size_k, size_n, group_size),
        zeros=empty if zeros_packed is None else marlin_zero_points_from_packed(zeros_packed.contiguous(), groups,
                                                                               size_n, bits),
        g_idx=sorted_g_idx, sort_indices=sort_indices, workspace=marlin_make_workspace_new(dev),
        is_k_full=marlin_is_k_full(g_idx is not None, row_parallel))


class MarlinLinearKernel(MPLinearKernel):
    """Repack at load, W4A16 GEMM at apply, both on the gfx950 HIP library.  Same contract as the reference's class
    of this name (mixed_precision/marlin.py:28-166): afterwards the layer holds the Marlin-layout weight, scales, zero
    points and sorted g_idx under the configured parameter names ("w_zp" / "g_idx" when none was given), plus
    `g_idx_sort_indices`, and a bias, if any, in Marlin order."""

    @classmethod
    def get_min_capability(cls) -> int:
        return 80  # gfx950 reports (9, 5)

    @classmethod
    def can_implement(cls, c: MPLinearLayerConfig) -> tuple[bool, str | None]:
        if not (torch.cuda.is_available() and torch.version.hip is not None):
            return False, "the gfx950 Marlin-surface kernels need a ROCm device"
        quant_types = query_marlin_supported_quant_types(c.zero_points)
        if c.weight_type not in quant_types:
            return False, (f"Quant type ({c.weight_type}) not supported by  Marlin, supported types are: "
                           f"{[str(t) for t in quant_types]}")
        if c.group_size not in MARLIN_SUPPORTED_GROUP_SIZES:
            return False, (f"Group size ({c.group_size}) not supported by Marlin, supported group sizes are: "
                           f"{MARLIN_SUPPORTED_GROUP_SIZES}")
        return check_marlin_supports_shape(c.partition_weight_shape[1], c.partition_weight_shape[0],
                                           c.full_weight_shape[0], c.group_size)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        c = self.config
        size_k, size_n = c.partition_weight_shape
        self.w_gidx_name = self.w_gidx_name or "g_idx"
        self.w_zp_name = self.w_zp_name or "w_zp"
        # checkpoint layouts: weight -> [K / pack, N] packed along K, scales -> [G, N], zero points -> [G, N / pack]
        t = prepare_marlin_layer(
            _to_layout(getattr(layer, self.w_q_name), input_dim=0, output_dim=1, packed_dim=0),
            _to_layout(getattr(layer, self.w_s_name), input_dim=0, output_dim=1),
            c.weight_type, size_k, size_n, c.group_size,
            zeros_packed=getattr(layer, self.w_zp_name).data.t() if c.zero_points else None,
            g_idx=getattr(layer, self.w_gidx_name).data if c.has_g_idx else None,
            row_parallel=size_k != c.full_weight_shape[0])
        for name, tensor in ((self.w_q_name, t.qweight), (self.w_s_name, t.scales), (self.w_zp_name, t.zeros),
                             (self.w_gidx_name, t.g_idx), ("g_idx_sort_indices", t.sort_indices)):
            replace_parameter(layer, name, tensor)
        self.workspace, self.is_k_full = t.workspace, t.is_k_full
        if getattr(layer, "bias", None) is not None:
            layer.bias.data = marlin_permute_bias(layer.bias.data)

    def apply_weights(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        size_k, size_n = self.config.partition_weight_shape
        w_q, w_s, w_zp, w_gidx = self._get_weight_params(layer)
        return apply_gptq_marlin_linear(x, w_q, w_s, w_zp, w_gidx, layer.g_idx_sort_indices, self.workspace,
                                        self.config.weight_type, size_n, size_k, self.is_k_full, bias)


_POSSIBLE_KERNELS: list[type[MPLinearKernel]] = [MarlinLinearKernel]


def choose_mp_linear_kernel(config: MPLinearLayerConfig, compute_capability: int | None = None) -> type[MPLinearKernel]:
    """Same selection loop as the reference's choose_mp_linear_kernel
    (mixed_precision/__init__.py:48-105) over the kernels this package provides."""
    import os
    if compute_capability is None and torch.cuda.is_available():
        major, minor = torch.cuda.get_device_capability()
        compute_capability = major * 10 + minor
    disabled = [k for k in os.environ.get("VLLM_DISABLED_KERNELS", "").split(",") if k]
    reasons = []
    for kernel in _POSSIBLE_KERNELS:
        if kernel.__name__ in disabled:
            reasons.append(f" {kernel.__name__} disabled by environment variable")
            continue
        if compute_capability is not None and kernel.get_min_capability() > compute_capability:
            reasons.append(f"{kernel.__name__} requires capability {kernel.get_min_capability()}, current compute "
                           f" capability is {compute_capability}")
            continue
        ok, why = kernel.can_implement(config)
        if ok:
            return kernel
        reasons.append(f" {kernel.__name__} cannot implement due to: {why}")
    raise ValueError("Failed to find a kernel that can implement the WNA16 linear layer. Reasons: \n" + "\n".join(reasons))
