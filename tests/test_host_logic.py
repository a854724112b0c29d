"""Host-side mirror of the reference interface, checked on the CPU against the oracle:
type ids, scale / bias / zero-point conversions, column packers, shape gates, operator registration."""
import pytest
import torch

from oracle import marlin_layout as ml
from oracle import quant_utils as qu
from oracle import scalar_types as ost


def test_scalar_type_ids_and_roundtrip():
    from vllm_amd.scalar_type import ScalarType, scalar_types
    assert scalar_types.uint4.id == ost.uint4.id == 1125899906843648
    assert scalar_types.uint4b8.id == ost.uint4b8.id == 1125899907892224
    assert scalar_types.uint8b128.id == ost.uint8b128.id == 1125899923621888
    for t in (scalar_types.uint4, scalar_types.uint4b8, scalar_types.uint8b128, scalar_types.int4, scalar_types.int8):
        assert ScalarType.from_id(t.id) == t
    assert str(scalar_types.uint4b8) == "uint4b8" and scalar_types.uint4b8.size_bits == 4
    assert (scalar_types.uint4b8.min(), scalar_types.uint4b8.max()) == (-8, 7)
    assert (scalar_types.int4.min(), scalar_types.int4.max()) == (-8, 7)
    assert scalar_types.uint4b8.has_bias() and not scalar_types.uint4.has_bias()


def test_pack_unpack_cols_match_oracle():
    from vllm_amd.quant_utils import get_pack_factor, pack_cols, unpack_cols
    assert get_pack_factor(4) == 8 and get_pack_factor(8) == 4
    q = torch.randint(0, 16, (6, 128), generator=torch.Generator().manual_seed(0), dtype=torch.int32)
    p = pack_cols(q, 4, 6, 128)
    assert p.dtype == torch.int32 and torch.equal(p, qu.pack_cols(q, 4))
    assert torch.equal(unpack_cols(p, 4, 6, 128), q)
    top = torch.full((1, 8), 15, dtype=torch.int32)
    assert int(pack_cols(top, 4, 1, 8)[0, 0]) == -1


@pytest.mark.parametrize("group", [-1, 128])
def test_scale_bias_zero_point_conversions_match_oracle(group):
    from vllm_amd import marlin_utils as mu
    k, n = 256, 192
    g = k // group if group != -1 else 1
    s = torch.randn(g, n, generator=torch.Generator().manual_seed(1)).half()
    assert torch.equal(mu.marlin_permute_scales(s, k, n, group), ml.marlin_permute_scales(s, k, n, group))
    b = torch.randn(n, generator=torch.Generator().manual_seed(2)).half()
    assert torch.equal(mu.marlin_permute_bias(b), ml.marlin_permute_bias(b))
    zp = torch.randint(0, 16, (g, n), generator=torch.Generator().manual_seed(3), dtype=torch.int32)
    assert torch.equal(mu.marlin_zero_points(zp, g, n, 4), ml.marlin_zero_points_closed_form(zp))
    assert torch.equal(mu.awq_to_marlin_zero_points(qu.awq_pack(zp), g, n, 4), ml.marlin_zero_points_closed_form(zp))
    se = torch.stack([s, s * 2])
    out = mu.marlin_moe_permute_scales(se, k, n, group)
    assert torch.equal(out[1], ml.marlin_permute_scales(s * 2, k, n, group))
    ze = torch.stack([qu.awq_pack(zp), qu.awq_pack(15 - zp)])
    assert torch.equal(mu.moe_awq_to_marlin_zero_points(ze, g, n, 4)[1], ml.marlin_zero_points_closed_form(15 - zp))


def test_sort_g_idx_and_k_full_rules():
    from vllm_amd import marlin_utils as mu
    g_idx = torch.tensor([3, 0, 2, 1, 0, 3, 1, 2], dtype=torch.int32)
    sorted_g, order = mu.marlin_sort_g_idx(g_idx)
    assert sorted_g.tolist() == [0, 0, 1, 1, 2, 2, 3, 3] and order.dtype == torch.int32
    assert torch.equal(g_idx[order.long()], sorted_g)
    assert mu.marlin_is_k_full(False, True) and mu.marlin_is_k_full(True, False) and not mu.marlin_is_k_full(True, True)
    assert mu.marlin_repeat_scales_on_all_ranks(True, 128, True)
    assert mu.marlin_repeat_scales_on_all_ranks(False, -1, True)
    assert not mu.marlin_repeat_scales_on_all_ranks(False, 128, True)


def test_shape_gates():
    from vllm_amd import marlin_utils as mu
    assert mu.check_marlin_supports_shape(4096, 4096, 4096, 128) == (True, None)
    ok, why = mu.check_marlin_supports_shape(4096 + 32, 4096, 4096, 128)
    assert not ok and "min_thread_n" in why
    ok, why = mu.check_marlin_supports_shape(4096, 4096 + 64, 8192, 128)
    assert not ok and "min_thread_k" in why
    ok, why = mu.check_marlin_supports_shape(4096, 384, 768, 256)
    assert not ok and "group_size" in why
    from vllm_amd.scalar_type import scalar_types
    assert mu.query_marlin_supported_quant_types(False) == [scalar_types.uint4b8, scalar_types.uint8b128,
                                                            scalar_types.float8_e4m3fn, scalar_types.float4_e2m1f]
    assert mu.query_marlin_supported_quant_types(False, include_fp_type=False) == [scalar_types.uint4b8,
                                                                                   scalar_types.uint8b128]
    assert mu.query_marlin_supported_quant_types(True) == [scalar_types.uint4]


def test_operators_registered_with_reference_schemas():
    import vllm_amd.ops as ops
    for name in ("gptq_marlin_repack", "awq_marlin_repack", "gptq_marlin_gemm", "permute_cols"):
        assert hasattr(torch.ops._C, name)
    for name in ("moe_wna16_marlin_gemm", "moe_align_block_size", "moe_sum"):
        assert hasattr(torch.ops._moe_C, name)
    schema = str(torch.ops._C.gptq_marlin_gemm.default._schema)
    for arg in ("c_or_none", "b_q_weight", "b_bias_or_none", "global_scale", "perm_or_none", "workspace",
                "b_q_type", "is_k_full", "use_atomic_add", "use_fp32_reduce", "is_zp_float"):
        assert arg in schema
    assert len(ops.REGISTERED) >= 8


def test_fake_impls_give_reference_shapes():
    """Meta tensors: output shapes as the reference's fake ops (vllm/_custom_ops.py:553-576, 1179-1218)."""
    from vllm_amd.scalar_type import scalar_types
    meta = torch.device("meta")
    out = torch.ops._C.gptq_marlin_repack(torch.empty(512 // 8, 256, dtype=torch.int32, device=meta),
                                          torch.empty(0, dtype=torch.int32, device=meta), 512, 256, 4)
    assert out.shape == (32, 512) and out.dtype == torch.int32
    out = torch.ops._C.awq_marlin_repack(torch.empty(512, 256 // 8, dtype=torch.int32, device=meta), 512, 256, 4)
    assert out.shape == (32, 512)
    e = torch.empty(0, dtype=torch.int32, device=meta)
    out = torch.ops._C.gptq_marlin_gemm(
        torch.empty(5, 512, dtype=torch.float16, device=meta), None, torch.empty(32, 512, dtype=torch.int32, device=meta),
        None, torch.empty(4, 256, dtype=torch.float16, device=meta), None, e, e, e,
        torch.empty(256, dtype=torch.int32, device=meta), scalar_types.uint4b8.id, 5, 256, 512, True, False, True, False)
    assert out.shape == (5, 256) and out.dtype == torch.float16


def test_cpu_tensors_are_rejected_not_silently_computed():
    """There is no CPU implementation behind the operators."""
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops._C.gptq_marlin_repack(torch.zeros(2, 64, dtype=torch.int32), torch.empty(0, dtype=torch.int32),
                                        16, 64, 4)


def test_kernel_selection_rejects_unsupported_configs():
    from vllm_amd.mixed_precision import MarlinLinearKernel, MPLinearLayerConfig
    from vllm_amd.scalar_type import scalar_types
    c = MPLinearLayerConfig(full_weight_shape=(4096, 4096), partition_weight_shape=(4096, 4096),
                            weight_type=scalar_types.uint4b8, act_type=torch.float16, group_size=128,
                            zero_points=False, has_g_idx=False)
    ok, why = MarlinLinearKernel.can_implement(c)
    if not torch.cuda.is_available():
        assert not ok and "ROCm device" in why


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more exits with a message instead of a JSON line."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_support_queries_and_layer_checks():
    import types
    from vllm_amd import marlin_utils as mu
    from vllm_amd.scalar_type import scalar_types
    assert mu.check_marlin_supported(scalar_types.uint4b8, 128) and mu.check_marlin_supported(scalar_types.uint4, 64, True)
    assert not mu.check_marlin_supported(scalar_types.uint4, 128)              # uint4 needs zero points
    assert not mu.check_marlin_supported(scalar_types.uint4b8, 100)
    with pytest.raises(ValueError, match="does not support group_size = 100"):
        mu.verify_marlin_supported(scalar_types.uint4b8, 100)
    with pytest.raises(ValueError, match="does not support weight_bits = uint4"):
        mu.verify_marlin_supported(scalar_types.uint4, 128)
    layer = types.SimpleNamespace(output_size_per_partition=6144, input_size_per_partition=4096, input_size=4096,
                                  output_size=6144)
    assert mu.check_marlin_supports_layer(layer, 128)
    layer.input_size_per_partition = 4000
    assert not mu.check_marlin_supports_layer(layer, 128)
    moe = types.SimpleNamespace(hidden_size=4096, intermediate_size_per_partition=14336,
                                apply_router_weight_on_input=False, activation="silu")
    assert mu.check_moe_marlin_supports_layer(moe, 128)
    moe.activation = "gelu"
    assert not mu.check_moe_marlin_supports_layer(moe, 128)
    moe.activation, moe.intermediate_size_per_partition = "silu", 14336 + 32
    assert not mu.check_moe_marlin_supports_layer(moe, 128)
    import torch
    assert mu.marlin_moe_intermediate_size(torch.empty(8, 256, 57344), torch.empty(8, 896, 8192)) == 14336
    assert mu.marlin_make_workspace(4096, torch.device("cpu")).shape == (1024,)


def test_moe_block_size_rule():
    """Blocks of 16 slots while an expert's share of the slots stays below ~1.25 blocks (sooner for experts of a few MB),
    blocks of 64 from there on; never 8, 32 or 48.  The quantity is the reference's (tokens * topk / experts,
    fused_marlin_moe.py:279-282); the thresholds are this library's."""
    from vllm_amd.fused_marlin_moe import pick_block_size
    big, small = 88 << 20, 5 << 20
    assert pick_block_size(1, 2, 8, big) == 16
    assert pick_block_size(16, 2, 8, big) == 16           # 4 slots per expert
    assert pick_block_size(64, 2, 8, big) == 16           # 16
    assert pick_block_size(79, 2, 8, big) == 16           # 19.75
    assert pick_block_size(80, 2, 8, big) == 64           # 20
    assert pick_block_size(4096, 2, 8, big) == 64
    assert pick_block_size(128, 8, 128, small) == 16      # 8 slots per expert
    assert pick_block_size(223, 8, 128, small) == 16      # 13.9
    assert pick_block_size(224, 8, 128, small) == 64      # 14
    assert pick_block_size(224, 8, 128, big) == 16        # the same share with large experts
    assert pick_block_size(100, 2, 8) == 64               # default: large experts
    assert all(pick_block_size(t, k, e, b) in (16, 64) for t in (1, 7, 300, 5000) for k in (1, 2, 8) for e in (4, 64, 256)
               for b in (small, big))
