"""WNA16 linear-kernel interface and its gfx950 Marlin-surface implementation.

Mirrors vllm/model_executor/layers/quantization/kernels/mixed_precision/MPLinearKernel.py:14-94
(MPLinearLayerConfig, MPLinearKernel) and .../mixed_precision/marlin.py:28-166 (MarlinLinearKernel):
same constructor, same `can_implement / process_weights_after_loading / apply_weights` contract,
same parameter names left on the layer, so a vLLM LinearMethod can hold either class.
Differences: `can_implement` accepts a ROCm gfx950 device instead of requiring CUDA, and the types offered
are uint4b8, uint8b128 and uint4 + zero points.
"""
from abc import ABC, abstractmethod
from collections.abc import Callable
from dataclasses import dataclass

import torch

from . import _custom_ops as ops
from .marlin_utils import (MARLIN_SUPPORTED_GROUP_SIZES, apply_gptq_marlin_linear, check_marlin_supports_shape,
                           marlin_is_k_full, marlin_make_empty_g_idx, marlin_make_workspace_new,
                           marlin_permute_bias, marlin_permute_scales, marlin_sort_g_idx, marlin_zero_points,
                           query_marlin_supported_quant_types)
from .quant_utils import unpack_cols
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

    def _transform_param(self, layer: torch.nn.Module, name: str | None, fn: Callable) -> None:
        if name is not None and getattr(layer, name, None) is not None:
            new_param = fn(getattr(layer, name))
            replace_parameter(layer, name, torch.nn.Parameter(new_param.data, requires_grad=False))

    def _get_weight_params(self, layer: torch.nn.Module):
        return (getattr(layer, self.w_q_name), getattr(layer, self.w_s_name),
                getattr(layer, self.w_zp_name or "", None), getattr(layer, self.w_gidx_name or "", None))


class MarlinLinearKernel(MPLinearKernel):
    """Repack at load, W4A16 GEMM at apply — both on the gfx950 HIP library."""

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

    # `weight_packed` is brought to {input_dim = 0, output_dim = 1, packed_dim = 0},
    # `weight_scale` to {input_dim = 0, output_dim = 1}
    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        device = getattr(layer, self.w_q_name).device
        c = self.config
        size_k, size_n = c.partition_weight_shape

        row_parallel = c.partition_weight_shape[0] != c.full_weight_shape[0]
        self.is_k_full = marlin_is_k_full(c.has_g_idx, row_parallel)
        self.workspace = marlin_make_workspace_new(device)

        if self.w_gidx_name is None:
            self.w_gidx_name = "g_idx"
        if self.w_zp_name is None:
            self.w_zp_name = "w_zp"

        if c.has_g_idx:
            g_idx, g_idx_sort_indices = marlin_sort_g_idx(getattr(layer, self.w_gidx_name))
            self._transform_param(layer, self.w_gidx_name, lambda _: g_idx)
            layer.g_idx_sort_indices = g_idx_sort_indices
        else:
            setattr(layer, self.w_gidx_name, marlin_make_empty_g_idx(device))
            layer.g_idx_sort_indices = marlin_make_empty_g_idx(device)

        def transform_w_q(x):
            w = _to_layout(x, input_dim=0, output_dim=1, packed_dim=0)
            x.data = ops.gptq_marlin_repack(w.contiguous(), perm=layer.g_idx_sort_indices, size_k=size_k,
                                            size_n=size_n, num_bits=c.weight_type.size_bits)
            return x

        def transform_w_s(x):
            s = _to_layout(x, input_dim=0, output_dim=1)
            x.data = marlin_permute_scales(s.contiguous(), size_k=size_k, size_n=size_n, group_size=c.group_size)
            return x

        if c.zero_points:
            grouped_k = size_k // c.group_size if c.group_size != -1 else 1
            self._transform_param(
                layer, self.w_zp_name,
                lambda x: marlin_zero_points(unpack_cols(x.t(), c.weight_type.size_bits, grouped_k, size_n),
                                             size_k=grouped_k, size_n=size_n, num_bits=c.weight_type.size_bits))
        else:
            setattr(layer, self.w_zp_name, marlin_make_empty_g_idx(device))
        self._transform_param(layer, self.w_q_name, transform_w_q)
        self._transform_param(layer, self.w_s_name, transform_w_s)

        if hasattr(layer, "bias") and layer.bias is not None:
            layer.bias.data = marlin_permute_bias(layer.bias)

    def apply_weights(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        c = self.config
        w_q, w_s, w_zp, w_gidx = self._get_weight_params(layer)
        return apply_gptq_marlin_linear(
            input=x, weight=w_q, weight_scale=w_s, weight_zp=w_zp, g_idx=w_gidx,
            g_idx_sort_indices=layer.g_idx_sort_indices, workspace=self.workspace, wtype=c.weight_type,
            input_size_per_partition=c.partition_weight_shape[0],
            output_size_per_partition=c.partition_weight_shape[1], is_k_full=self.is_k_full, bias=bias)


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
