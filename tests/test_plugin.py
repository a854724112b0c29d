"""The vLLM plugin shim against a stand-in `vllm` package tree (CPU only: no vLLM, no GPU)."""
import importlib
import sys
import types

import pytest


def _fake_vllm(monkeypatch):
    def mod(name, **attrs):
        m = types.ModuleType(name)
        for k, v in attrs.items():
            setattr(m, k, v)
        monkeypatch.setitem(sys.modules, name, m)
        return m

    class GPTQMarlinConfig:
        @classmethod
        def is_gptq_marlin_compatible(cls, quant_config):
            return False            # "not CUDA"

    class AWQMarlinConfig:
        @classmethod
        def is_awq_marlin_compatible(cls, quant_config):
            return False

    class RocmPlatform:
        supported_quantization = ["awq", "gptq", "fp8"]

    class OtherKernel:
        pass

    for pkg in ("vllm", "vllm.model_executor", "vllm.model_executor.layers", "vllm.model_executor.layers.quantization",
                "vllm.model_executor.layers.quantization.kernels", "vllm.platforms"):
        mod(pkg).__path__ = []
    mp = mod("vllm.model_executor.layers.quantization.kernels.mixed_precision", _POSSIBLE_KERNELS=[OtherKernel])
    gm = mod("vllm.model_executor.layers.quantization.gptq_marlin", GPTQMarlinConfig=GPTQMarlinConfig)
    am = mod("vllm.model_executor.layers.quantization.awq_marlin", AWQMarlinConfig=AWQMarlinConfig)
    rp = mod("vllm.platforms.rocm", RocmPlatform=RocmPlatform)
    return mp, gm, am, rp


def test_kernel_class_and_gates(monkeypatch):
    mp, gm, am, rp = _fake_vllm(monkeypatch)
    plugin = importlib.import_module("vllm_amd.plugin")
    assert plugin.register_kernel_class()
    assert mp._POSSIBLE_KERNELS[0].__name__ == "Gfx950MarlinLinearKernel" and len(mp._POSSIBLE_KERNELS) == 2
    assert plugin.register_kernel_class() and len(mp._POSSIBLE_KERNELS) == 2          # idempotent
    from vllm_amd.mixed_precision import MarlinLinearKernel
    assert issubclass(mp._POSSIBLE_KERNELS[0], MarlinLinearKernel)

    lifted = plugin.lift_platform_gates()
    assert len(lifted) == 3
    ok = gm.GPTQMarlinConfig.is_gptq_marlin_compatible
    assert ok({"quant_method": "gptq", "bits": 4, "group_size": 128, "sym": True, "desc_act": False})
    assert ok({"quant_method": "GPTQ", "bits": 8, "group_size": -1, "sym": True, "desc_act": True})
    assert not ok({"quant_method": "gptq", "bits": 4, "group_size": 128, "sym": False, "desc_act": False})
    assert not ok({"quant_method": "gptq", "bits": 3, "group_size": 128, "sym": True, "desc_act": False})
    assert not ok({"quant_method": "gptq", "bits": 4, "group_size": 100, "sym": True, "desc_act": False})
    assert not ok({"quant_method": "gptq", "bits": 4, "group_size": 128, "sym": True})      # desc_act missing
    assert not ok({"quant_method": "awq", "bits": 4, "group_size": 128, "sym": True, "desc_act": False})
    ok = am.AWQMarlinConfig.is_awq_marlin_compatible
    assert ok({"quant_method": "awq", "bits": 4, "group_size": 128, "zero_point": True})
    assert not ok({"quant_method": "awq", "bits": 4, "group_size": 128, "zero_point": False})
    assert not ok({"quant_method": "awq", "bits": 8, "group_size": 128, "zero_point": True})
    assert not ok({"quant_method": "awq", "bits": 4, "group_size": 128})
    assert rp.RocmPlatform.supported_quantization == ["awq", "gptq", "fp8", "gptq_marlin", "awq_marlin"]
    plugin.lift_platform_gates()
    assert rp.RocmPlatform.supported_quantization.count("gptq_marlin") == 1


def test_without_vllm_nothing_is_registered_and_nothing_raises(monkeypatch):
    for name in list(sys.modules):
        if name == "vllm" or name.startswith("vllm."):
            monkeypatch.delitem(sys.modules, name)
    plugin = importlib.import_module("vllm_amd.plugin")
    assert plugin.register_kernel_class() is False
    assert plugin.lift_platform_gates() == []
