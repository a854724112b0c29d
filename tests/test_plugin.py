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
    assert issubclass(mp._POSSIBLE_KERNELS[0], MarlinLinearKernel)    # this stand-in vLLM has no marlin module

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


def test_kernel_class_derives_from_the_installed_marlin_kernel(monkeypatch):
    """With vLLM's MarlinLinearKernel importable the registered class is a subclass of it that replaces
    can_implement only: weight preparation and apply_weights stay the installed vLLM's."""
    mp, *_ = _fake_vllm(monkeypatch)

    class TheirMarlin:
        @classmethod
        def can_implement(cls, c):
            return False, "Marlin only supported on CUDA"

        def process_weights_after_loading(self, layer):
            return "theirs"

        def apply_weights(self, layer, x, bias=None):
            return "theirs"

    m = types.ModuleType(mp.__name__ + ".marlin")
    m.MarlinLinearKernel = TheirMarlin
    monkeypatch.setitem(sys.modules, m.__name__, m)
    mp.__path__ = []
    plugin = importlib.import_module("vllm_amd.plugin")
    assert plugin.register_kernel_class()
    k = mp._POSSIBLE_KERNELS[0]
    assert k.__name__ == "Gfx950MarlinLinearKernel" and issubclass(k, TheirMarlin)
    assert set(vars(k)) & {"can_implement", "process_weights_after_loading", "apply_weights"} == {"can_implement"}
    from vllm_amd.scalar_type import scalar_types
    cfg = types.SimpleNamespace(full_weight_shape=(4096, 4096), partition_weight_shape=(4096, 4096),
                                weight_type=scalar_types.uint4b8, act_type=None, group_size=128, zero_points=False,
                                has_g_idx=False)
    import torch
    assert k.can_implement(cfg) == (False, "the gfx950 Marlin-surface kernels need a ROCm device") \
        or torch.cuda.is_available()
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.version, "hip", "7.0")
    assert k.can_implement(cfg)[0]
    cfg.group_size = 100
    assert not k.can_implement(cfg)[0]
    # the library's own class on request
    mp._POSSIBLE_KERNELS.pop(0)
    assert plugin.register_kernel_class(own_load_path=True)
    from vllm_amd.mixed_precision import MarlinLinearKernel
    assert issubclass(mp._POSSIBLE_KERNELS[0], MarlinLinearKernel)


def test_without_vllm_nothing_is_registered_and_nothing_raises(monkeypatch):
    for name in list(sys.modules):
        if name == "vllm" or name.startswith("vllm."):
            monkeypatch.delitem(sys.modules, name)
    plugin = importlib.import_module("vllm_amd.plugin")
    assert plugin.register_kernel_class() is False
    assert plugin.lift_platform_gates() == []
