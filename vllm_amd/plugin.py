"""vLLM general-plugin entry point: makes the gfx950 Marlin-surface operators and kernel class visible to an
unmodified vLLM on ROCm.

Declare it in the installing package's metadata as

    [project.entry-points."vllm.general_plugins"]
    w4a16_gfx950 = "vllm_amd.plugin:register"

vLLM calls every entry point of that group once per process before it builds a model
(vllm/plugins/__init__.py:65-78).  `register()` is idempotent and never raises on a vLLM whose layout differs from
the one this was written against: a gate it cannot find is reported and skipped.

What it does, in order:
  1. imports `vllm_amd.ops`, which defines torch.ops._C.{gptq_marlin_repack, awq_marlin_repack, gptq_marlin_gemm,
     permute_cols, silu_and_mul} and torch.ops._moe_C.{moe_wna16_marlin_gemm, moe_align_block_size, moe_sum,
     topk_softmax} when they do not exist (ROCm builds of vLLM compile their definitions out,
     csrc/torch_bindings.cpp:240, csrc/moe/torch_bindings.cpp:52);
  2. puts `Gfx950MarlinLinearKernel` in front of `_POSSIBLE_KERNELS`
     (vllm/model_executor/layers/quantization/kernels/mixed_precision/__init__.py:36-45), so `choose_mp_linear_kernel`
     finds a kernel for uint4b8 / uint8b128 / uint4 + zero points on this platform; the class is vLLM's own
     MarlinLinearKernel with `can_implement` replaced (see `register_kernel_class`);
  3. lifts the CUDA-only gates in front of the Marlin quantization configs: `is_gptq_marlin_compatible`
     (gptq_marlin.py:254-279), `is_awq_marlin_compatible` (awq_marlin.py:216-241) and the ROCm platform's
     `supported_quantization` list (platforms/rocm.py:175-187).
"""
import importlib
import logging

logger = logging.getLogger("vllm_amd.plugin")

_MP_KERNELS = "vllm.model_executor.layers.quantization.kernels.mixed_precision"
_GPTQ_MARLIN = "vllm.model_executor.layers.quantization.gptq_marlin"
_AWQ_MARLIN = "vllm.model_executor.layers.quantization.awq_marlin"
_ROCM_PLATFORM = "vllm.platforms.rocm"

_registered = False


def _try_import(name: str):
    try:
        return importlib.import_module(name)
    except Exception as exc:  # vLLM absent, or a layout this shim does not know
        logger.info("vllm_amd.plugin: %s not importable (%s); step skipped", name, exc)
        return None


def register_kernel_class(own_load_path: bool = False) -> bool:
    """Step 2.  The class put in front of `_POSSIBLE_KERNELS` is named Gfx950MarlinLinearKernel, so that vLLM's
    VLLM_DISABLED_KERNELS=MarlinLinearKernel still only addresses vLLM's CUDA kernel.

    With vLLM's own `MarlinLinearKernel` importable (kernels/mixed_precision/marlin.py:27) the class derives from
    THAT one and overrides `can_implement` alone (marlin.py:33-59, whose first test is "CUDA only"): weight
    preparation and `apply_weights` stay vLLM's code, which reaches this library through the `_C` operators of
    step 1, so parameter handling follows the installed vLLM version.  `own_load_path=True`, or a vLLM without that
    module, registers this library's class instead, which prepares a layer with its device-side kernels
    (`vllm_amd.mixed_precision.prepare_marlin_layer`)."""
    mp = _try_import(_MP_KERNELS)
    if mp is None or not hasattr(mp, "_POSSIBLE_KERNELS"):
        return False
    from .mixed_precision import MarlinLinearKernel as OwnKernel

    if any(k.__name__ == "Gfx950MarlinLinearKernel" for k in mp._POSSIBLE_KERNELS):
        return True

    theirs = None if own_load_path else getattr(_try_import(_MP_KERNELS + ".marlin"), "MarlinLinearKernel", None)
    if theirs is not None:
        class Gfx950MarlinLinearKernel(theirs):
            @classmethod
            def can_implement(cls, c):
                return OwnKernel.can_implement(c)   # the reference's rule without its platform test
    else:
        class Gfx950MarlinLinearKernel(OwnKernel):
            pass

    mp._POSSIBLE_KERNELS.insert(0, Gfx950MarlinLinearKernel)
    return True


def _compatible(quant_config: dict, method: str, has_zp_key: str | None) -> bool:
    """The reference's compatibility rule without its platform test, on this library's supported types."""
    from .marlin_utils import MARLIN_SUPPORTED_GROUP_SIZES, query_marlin_supported_quant_types
    from .scalar_type import scalar_types
    if str(quant_config.get("quant_method", "")).lower() != method:
        return False
    bits, group = quant_config.get("bits"), quant_config.get("group_size")
    if bits is None or group is None or group not in MARLIN_SUPPORTED_GROUP_SIZES:
        return False
    if method == "gptq":
        sym, desc_act = quant_config.get("sym"), quant_config.get("desc_act")
        if sym is None or desc_act is None or not sym:
            return False
        wtype = {4: scalar_types.uint4b8, 8: scalar_types.uint8b128}.get(bits)
        return wtype in query_marlin_supported_quant_types(False)
    zero_point = quant_config.get(has_zp_key)
    if zero_point is None:
        return False
    wtype = {4: scalar_types.uint4}.get(bits)
    return bool(zero_point) and wtype in query_marlin_supported_quant_types(True)


def lift_platform_gates() -> list[str]:
    """Step 3; returns the names of the gates that were lifted."""
    lifted = []
    gm = _try_import(_GPTQ_MARLIN)
    if gm is not None and hasattr(gm, "GPTQMarlinConfig"):
        gm.GPTQMarlinConfig.is_gptq_marlin_compatible = classmethod(
            lambda cls, quant_config: _compatible(quant_config, "gptq", None))
        lifted.append("GPTQMarlinConfig.is_gptq_marlin_compatible")
    am = _try_import(_AWQ_MARLIN)
    if am is not None and hasattr(am, "AWQMarlinConfig"):
        am.AWQMarlinConfig.is_awq_marlin_compatible = classmethod(
            lambda cls, quant_config: _compatible(quant_config, "awq", "zero_point"))
        lifted.append("AWQMarlinConfig.is_awq_marlin_compatible")
    rp = _try_import(_ROCM_PLATFORM)
    if rp is not None and hasattr(rp, "RocmPlatform"):
        names = list(getattr(rp.RocmPlatform, "supported_quantization", []))
        for q in ("gptq_marlin", "awq_marlin"):
            if q not in names:
                names.append(q)
        rp.RocmPlatform.supported_quantization = names
        lifted.append("RocmPlatform.supported_quantization")
    return lifted


def register() -> None:
    global _registered
    if _registered:
        return
    _registered = True
    from . import ops  # noqa: F401  (step 1: operator definitions and implementations)
    have_kernel = register_kernel_class()
    lifted = lift_platform_gates()
    logger.info("vllm_amd.plugin: operators %s; kernel class %s; gates lifted: %s", sorted(ops.REGISTERED),
                "registered" if have_kernel else "not registered", lifted or "none")
