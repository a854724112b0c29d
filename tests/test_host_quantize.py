"""The in-package synthetic-layer helpers (vllm_amd/marlin_utils_test.py, vllm_amd/quant_utils.py), run on CPU
tensors, against the oracle: same integers, scales, zero points, dequantised weights and packed words."""
import pytest
import torch

from oracle import quant_utils as qu
from oracle import scalar_types as ost


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group", [-1, 32, 128])
def test_quantize_weights_matches_oracle(dtype, group):
    from vllm_amd.marlin_utils_test import quantize_weights
    from vllm_amd.scalar_type import scalar_types as st
    w = (torch.randn(256, 192, generator=torch.Generator().manual_seed(1)) * 0.02).to(dtype)
    for rule in ("reference", "absmax"):
        got = quantize_weights(w, st.uint4b8, group, rule=rule)
        if rule == "reference":
            want = qu.quantize_weights(w, ost.uint4b8, group)[:3]
        else:
            want = qu.quantize_absmax7(w, group)
        for g, x in zip(got[:3], want):
            assert torch.equal(g, x)
        got = quantize_weights(w, st.uint4, group, zero_points=True, rule=rule)
        want = qu.quantize_weights(w, ost.uint4, group, zero_points=True) if rule == "reference" else \
            qu.quantize_minmax_zp(w, group)
        for g, x in zip(got, want):
            assert torch.equal(g, x)
    got8 = quantize_weights(w, st.uint8b128, group)
    want8 = qu.quantize_weights(w, ost.uint8b128, group)[:3]
    for g, x in zip(got8[:3], want8):
        assert torch.equal(g, x)


@pytest.mark.parametrize("bits", [4, 8])
def test_checkpoint_packers_match_oracle(bits):
    from vllm_amd.quant_utils import awq_pack, gptq_pack, pack_rows, unpack_rows
    k, n = 64, 96
    q = torch.randint(0, 1 << bits, (k, n), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    assert torch.equal(gptq_pack(q, bits, k, n), qu.gptq_pack(q, bits))
    assert torch.equal(awq_pack(q, bits, k, n), qu.awq_pack(q, bits))
    assert torch.equal(unpack_rows(pack_rows(q, bits, k, n), bits, k, n), q)
    # literal word: rows 0..7 of column 0 holding 0..7 pack to 0x76543210
    lit = torch.arange(8, dtype=torch.int32).view(8, 1)
    assert int(pack_rows(lit, 4, 8, 1)[0, 0]) == 0x76543210
