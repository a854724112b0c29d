"""GPU parity of the W4A16 GEMM against the CPU oracle (dequantize, fp32 matmul), through the torch
op -> C ABI -> HIP kernels.  Tolerances: max|out-ref|/max|ref| <= 2e-2 (fp16) / 4e-2 (bf16) and the
reference test's mean|out-ref|/mean|ref| < 0.04 (tests/kernels/quantization/test_marlin_gemm.py:78-81,
359-361); one-hot activations must reproduce the dequantised weight rows bit-for-bit."""
import pytest
import torch

from helpers import check_close, make_layer, run_gemm
from oracle import gemm_ref as gr

pytestmark = pytest.mark.gpu

MNK_FACTORS = [(1, 1, 1), (1, 4, 8), (26, 37, 13), (257, 13, 11)]


@pytest.fixture(scope="module")
def ops(dev):
    import vllm_amd.ops as o
    return o


@pytest.fixture(scope="module")
def workspace(dev):
    from vllm_amd.marlin_utils import marlin_make_workspace_new
    return marlin_make_workspace_new(dev)


def _a(m, k, dtype, dev, seed=11):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(m, k, generator=g).to(dtype).to(dev)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("has_zp", [False, True])
@pytest.mark.parametrize("group_size", [-1, 32, 64, 128])
def test_one_hot_rows_are_exact(ops, dev, workspace, dtype, has_zp, group_size):
    """A = unit vectors: every output row is a single product 1 * w, so it must equal w_ref exactly.
    Pins layout decode, nibble order, the -8 bias / zero points and scale indexing with zero tolerance."""
    size_k, size_n = 512, 320
    print(f"one_hot dtype={dtype} zp={has_zp} g={group_size}", flush=True)
    layer = make_layer(size_k, size_n, group_size, dtype, has_zp=has_zp, seed=5)
    ks = torch.tensor([0, 1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 100, 127, 128, 300, 511])
    a = torch.zeros(16, size_k, dtype=dtype)
    a[torch.arange(16), ks] = 1.0
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_one_hot_every_k(ops, dev, workspace, dtype):
    """All K positions of a 256-deep layer, 64 rows at a time (also exercises the 4-m-block tile)."""
    size_k, size_n = 256, 128
    layer = make_layer(size_k, size_n, 64, dtype, seed=6)
    a = torch.eye(size_k, dtype=dtype)
    for m0 in range(0, size_k, 64):
        print(f"one_hot_all dtype={dtype} rows={m0}", flush=True)
        out = run_gemm(ops, layer, a[m0:m0 + 64].contiguous().to(dev), dev, workspace)
        assert torch.equal(out.cpu(), layer.w_ref[m0:m0 + 64])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("is_k_full", [True, False])
def test_one_hot_act_order(ops, dev, workspace, dtype, is_k_full):
    size_k, size_n = 512, 192
    print(f"one_hot_act_order dtype={dtype} k_full={is_k_full}", flush=True)
    layer = make_layer(size_k, size_n, 64, dtype, act_order=True, seed=8)
    ks = torch.randperm(size_k, generator=torch.Generator().manual_seed(2))[:32]
    a = torch.zeros(32, size_k, dtype=dtype)
    a[torch.arange(32), ks] = 1.0
    out = run_gemm(ops, layer, a.to(dev), dev, workspace, is_k_full=is_k_full)
    assert torch.equal(out.cpu(), layer.w_ref[ks])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n_chunk", [64, 256])
@pytest.mark.parametrize("mnk", MNK_FACTORS)
@pytest.mark.parametrize("group_size", [-1, 32, 64, 128])
@pytest.mark.parametrize("mode", ["gptq", "gptq_act_order", "gptq_act_order_partial_k", "awq"])
def test_gemm_reference_grid(ops, dev, workspace, dtype, n_chunk, mnk, group_size, mode):
    """The reference's test_gptq_marlin_gemm grid restricted to the 4-bit types."""
    mf, nf, kf = mnk
    size_m, size_k, size_n = mf, 128 * kf, n_chunk * nf
    act_order = mode.startswith("gptq_act_order")
    if act_order and (group_size == -1 or group_size == size_k):
        pytest.skip("act-order needs more than one group")
    if size_k % (group_size if group_size > 0 else size_k) != 0:
        pytest.skip("group does not divide K")
    print(f"grid {mode} dtype={dtype} m={size_m} n={size_n} k={size_k} g={group_size}", flush=True)
    layer = make_layer(size_k, size_n, group_size, dtype, has_zp=(mode == "awq"), act_order=act_order,
                       seed=size_n + size_k)
    a = _a(size_m, size_k, dtype, dev)
    out = run_gemm(ops, layer, a, dev, workspace, is_k_full=(mode != "gptq_act_order_partial_k"))
    assert out.shape == (size_m, size_n) and out.dtype == dtype
    check_close(out, a, layer)
    assert int(workspace.abs().sum()) == 0


def test_integer_exact(ops, dev, workspace):
    """Unit scales and small-integer activations: every partial sum is an exact integer below 2^24,
    so the GEMM must equal the integer matmul exactly whatever the summation order."""
    size_m, size_k, size_n = 48, 1024, 256
    g = torch.Generator().manual_seed(4)
    layer = make_layer(size_k, size_n, 128, torch.float16, seed=9)
    layer.marlin_s = torch.ones_like(layer.marlin_s)
    a = torch.randint(-4, 5, (size_m, size_k), generator=g).half()
    want = a.float() @ (layer.q.float() - 8)
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    assert torch.equal(out.float().cpu(), want.half().float())


def test_rows_independent_of_m_and_deterministic(ops, dev, workspace):
    """Row m of the result does not depend on M, on the other rows, or on the run (ordered split-K)."""
    size_k, size_n = 4096, 1024
    layer = make_layer(size_k, size_n, 128, torch.float16, seed=10, w_std=0.02)
    a = _a(200, size_k, torch.float16, dev)
    full = run_gemm(ops, layer, a, dev, workspace)
    again = run_gemm(ops, layer, a, dev, workspace)
    assert torch.equal(full, again)
    for m in (1, 4, 16, 17, 64, 65):
        part = run_gemm(ops, layer, a[:m].contiguous(), dev, workspace)
        d = (part.float() - full[:m].float()).abs().max() / full.float().abs().max()
        assert float(d) < 2e-3, (m, float(d))   # same operands, only the split-K partition may differ
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_strided_a_and_bias_and_given_c(ops, dev, workspace, dtype):
    """Sub-view activations (test_marlin_gemm.py:537-581), bias (:584-629), caller-provided output."""
    from vllm_amd.marlin_utils import marlin_permute_bias
    size_m, size_k, size_n = 37, 512, 384
    layer = make_layer(size_k, size_n, 128, dtype, seed=12)
    g = torch.Generator().manual_seed(13)
    big = torch.randn(size_m, size_k + 64, generator=g).to(dtype).to(dev)
    a = big[:, 32:32 + size_k]
    assert not a.is_contiguous()
    bias = torch.randn(size_n, generator=g).to(dtype).to(dev)
    c = torch.empty(size_m, size_n, dtype=dtype, device=dev)
    out = run_gemm(ops, layer, a, dev, workspace, bias=marlin_permute_bias(bias), c=c)
    assert out.data_ptr() == c.data_ptr()
    check_close(out, a, layer, bias=bias)


def test_empty_m(ops, dev, workspace):
    layer = make_layer(128, 64, 128, torch.float16)
    out = run_gemm(ops, layer, torch.empty(0, 128, dtype=torch.float16, device=dev), dev, workspace)
    assert out.shape == (0, 64)


def test_argument_errors(ops, dev, workspace):
    layer = make_layer(128, 64, 128, torch.float16)
    a = torch.zeros(4, 128, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError):
        run_gemm(ops, layer, torch.zeros(4, 64, dtype=torch.float16, device=dev), dev, workspace)   # K mismatch
    with pytest.raises(RuntimeError):
        run_gemm(ops, layer, a.float(), dev, workspace)                                              # dtype
    import vllm_amd.scalar_type as vst
    with pytest.raises((RuntimeError, NotImplementedError)):
        ops.gptq_marlin_gemm(a, None, layer.marlin_q.to(dev), None, layer.marlin_s.to(dev), None, None, None, None,
                             workspace, vst.scalar_types.uint8b128, 4, 64, 128)


@pytest.mark.parametrize("shape", [(4096, 4096), (4096, 6144), (14336, 4096)])
@pytest.mark.parametrize("m", [1, 16, 64, 256])
def test_llama_shapes_fp16(ops, dev, workspace, shape, m):
    """Configuration 1 / 2 shapes: N(0,1) activations, N(0, 0.02) weights, absmax/7 RTN, group 128."""
    size_k, size_n = shape
    print(f"llama k={size_k} n={size_n} m={m}", flush=True)
    layer = make_layer(size_k, size_n, 128, torch.float16, seed=1, w_std=0.02, rule="benchmark")
    a = _a(m, size_k, torch.float16, dev, seed=2)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)
    assert int(workspace.abs().sum()) == 0


# ------------------------------------------------------------------------- prefill (128-row tile) kernel
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("has_zp", [False, True])
@pytest.mark.parametrize("group_size", [-1, 32, 128])
def test_prefill_one_hot(ops, dev, workspace, dtype, has_zp, group_size):
    """Identity activations through the large-M path: every dequantised weight row comes back bit-exact."""
    size_k, size_n = 256, 576   # N = 4.5 column pairs: a partly filled 512-column tile and an odd n-tile
    print(f"prefill one_hot dtype={dtype} zp={has_zp} g={group_size}", flush=True)
    layer = make_layer(size_k, size_n, group_size, dtype, has_zp=has_zp, seed=21)
    a = torch.eye(size_k, dtype=dtype)
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["gptq", "awq", "gptq_act_order", "channel"])
@pytest.mark.parametrize("mnk", [(128, 512, 128), (129, 1088, 384), (300, 64, 1024), (1000, 2048, 2048)])
def test_prefill_shapes(ops, dev, workspace, dtype, mode, mnk):
    size_m, size_n, size_k = mnk
    group = -1 if mode == "channel" else 128
    if mode == "gptq_act_order" and size_k == group:
        pytest.skip("act-order needs more than one group")
    print(f"prefill {mode} dtype={dtype} m={size_m} n={size_n} k={size_k}", flush=True)
    layer = make_layer(size_k, size_n, group, dtype, has_zp=(mode == "awq"), act_order=(mode == "gptq_act_order"),
                       seed=size_m)
    a = _a(size_m, size_k, dtype, dev, seed=3)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)


def test_prefill_bias_and_strided_a(ops, dev, workspace):
    from vllm_amd.marlin_utils import marlin_permute_bias
    size_m, size_k, size_n = 200, 512, 640
    layer = make_layer(size_k, size_n, 128, torch.float16, seed=31)
    g = torch.Generator().manual_seed(32)
    a = torch.randn(size_m, size_k + 128, generator=g).half().to(dev)[:, 64:64 + size_k]
    bias = torch.randn(size_n, generator=g).half().to(dev)
    out = run_gemm(ops, layer, a, dev, workspace, bias=marlin_permute_bias(bias))
    check_close(out, a, layer, bias=bias)


def test_prefill_llama_o_proj_bf16_awq(ops, dev, workspace):
    """Configuration 3, o_proj: M = 4096, bf16, uint4 + zero points, group 128."""
    size_m, size_k, size_n = 4096, 4096, 4096
    print("prefill llama o_proj M=4096 bf16 awq", flush=True)
    layer = make_layer(size_k, size_n, 128, torch.bfloat16, has_zp=True, seed=41, w_std=0.02, rule="benchmark")
    a = _a(size_m, size_k, torch.bfloat16, dev, seed=42)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)


@pytest.mark.parametrize("dtype,mode", [(torch.float16, "gptq"), (torch.bfloat16, "awq")])
def test_mid_kernel_split_k(ops, dev, workspace, dtype, mode):
    """1024 x 4096 output = 128 tiles of 64 x 512: the 64-row kernel runs with K split in two and the reduction pass."""
    size_m, size_k, size_n = 1024, 2048, 4096
    layer = make_layer(size_k, size_n, 128, dtype, has_zp=(mode == "awq"), seed=21, rule="absmax7" if mode == "gptq" else "minmax")
    a = _a(size_m, size_k, dtype, dev)
    bias = torch.randn(size_n, generator=torch.Generator().manual_seed(3)).to(dtype)
    from vllm_amd.marlin_utils import marlin_permute_bias
    out = run_gemm(ops, layer, a, dev, workspace, bias=marlin_permute_bias(bias.to(dev)))
    check_close(out, a, layer, bias=bias)
    out2 = run_gemm(ops, layer, a, dev, workspace, bias=marlin_permute_bias(bias.to(dev)))
    assert torch.equal(out, out2)
    # one-hot rows stay exact through the split (one split holds the product, the others add zero)
    ks = torch.randperm(size_k, generator=torch.Generator().manual_seed(1))[:size_m // 2]
    oh = torch.zeros(size_m, size_k, dtype=dtype)
    oh[torch.arange(size_m // 2), ks] = 1.0
    out = run_gemm(ops, layer, oh.to(dev), dev, workspace)
    assert torch.equal(out[:size_m // 2].cpu(), layer.w_ref[ks])
    assert int(out[size_m // 2:].abs().sum()) == 0


def test_reduce_flags_do_not_change_results(ops, dev, workspace):
    """use_atomic_add / use_fp32_reduce are accepted for interface parity (test_marlin_gemm.py:62-63); partial sums are
    always fp32 and added in a fixed order, so every combination gives the same bits."""
    import vllm_amd.scalar_type as vst
    layer = make_layer(4096, 512, 128, torch.float16, seed=31, rule="absmax7", w_std=0.05)
    a = _a(16, 4096, torch.float16, dev)
    outs = []
    for atomic in (False, True):
        for fp32 in (False, True):
            outs.append(ops.gptq_marlin_gemm(a, None, layer.marlin_q.to(dev), None, layer.marlin_s.to(dev), None,
                                             layer.marlin_zp.to(dev), layer.g_idx_sorted.to(dev), layer.sort_indices.to(dev),
                                             workspace, vst.scalar_types.uint4b8, 16, 512, 4096, is_k_full=True,
                                             use_atomic_add=atomic, use_fp32_reduce=fp32, is_zp_float=False))
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    check_close(outs[0], a, layer)


@pytest.mark.parametrize("size_m,handed", [(4096, 4), (3072, 2), (2100, 1)])
def test_prefill_tail_strips_go_to_the_64_row_kernel(ops, dev, workspace, size_m, handed):
    """N = 6144 in 128 x 512 tiles on 256 compute units: 4096 rows give one full round plus half a round (four whole
    strips), 3072 rows one round plus 32 tiles (one strip and a third), 2100 rows 204 tiles (no second round: `handed`
    strips only if a second round exists).  The handed-over strips are computed by the 64-row kernel; both parts must
    meet the same bar."""
    size_k, size_n = 256, 6144
    layer = make_layer(size_k, size_n, 128, torch.bfloat16, has_zp=True, seed=41, rule="minmax", w_std=0.05)
    a = _a(size_m, size_k, torch.bfloat16, dev)
    bias = torch.randn(size_n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    from vllm_amd.marlin_utils import marlin_permute_bias
    out = run_gemm(ops, layer, a, dev, workspace, bias=marlin_permute_bias(bias.to(dev)))
    ref = gr.gemm_ref(a.cpu(), layer.w_ref, bias)
    split = size_n - 512 * handed
    for lo, hi in ((0, split), (split, size_n)):      # prefill-kernel strips, strips that may be handed over
        m = gr.error_metrics(out[:, lo:hi], ref[:, lo:hi])
        assert m["max_rel"] <= 4e-2 and m["mean_rel"] < 0.04, (lo, hi, m)


# ------------------------------------------------------------ 33..128 rows
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode", ["gptq", "awq", "gptq_act_order", "channel", "gptq_g32"])
@pytest.mark.parametrize("mnk", [(33, 192, 128), (64, 320, 512), (67, 832, 384), (100, 128, 2048), (128, 4096, 256)])
def test_rows_33_to_128(ops, dev, workspace, dtype, mode, mnk):
    """Between the decode and prefill regimes: N/64 odd and even, shallow and deep K (K split or not)."""
    size_m, size_n, size_k = mnk
    group = -1 if mode == "channel" else 32 if mode == "gptq_g32" else 128
    if mode == "gptq_act_order" and size_k == group:
        pytest.skip("act-order needs more than one group")
    print(f"rows33-128 {mode} dtype={dtype} m={size_m} n={size_n} k={size_k}", flush=True)
    layer = make_layer(size_k, size_n, group, dtype, has_zp=(mode == "awq"), act_order=(mode == "gptq_act_order"),
                       seed=size_m + 1)
    a = _a(size_m, size_k, dtype, dev, seed=4)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)
    assert int(workspace.abs().sum()) == 0
    assert torch.equal(out, run_gemm(ops, layer, a, dev, workspace))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("has_zp", [False, True])
@pytest.mark.parametrize("group_size", [-1, 64, 128])
def test_rows_33_to_128_one_hot(ops, dev, workspace, dtype, has_zp, group_size):
    """Unit-vector rows for 100 rows: wide N with shallow K, narrow N with deep K."""
    for size_k, size_n in ((256, 1536), (2048, 192)):
        layer = make_layer(size_k, size_n, group_size, dtype, has_zp=has_zp, seed=9)
        ks = torch.randperm(size_k, generator=torch.Generator().manual_seed(3))[:100]
        a = torch.zeros(100, size_k, dtype=dtype)
        a[torch.arange(100), ks] = 1.0
        out = run_gemm(ops, layer, a.to(dev), dev, workspace)
        assert torch.equal(out.cpu(), layer.w_ref[ks])


def test_rows_33_to_128_bias_strided_a_given_c(ops, dev, workspace):
    from vllm_amd.marlin_utils import marlin_permute_bias
    size_m, size_k, size_n = 90, 1024, 448
    layer = make_layer(size_k, size_n, 128, torch.bfloat16, has_zp=True, seed=33)
    g = torch.Generator().manual_seed(34)
    a = torch.randn(size_m, size_k + 64, generator=g).bfloat16().to(dev)[:, 32:32 + size_k]
    bias = torch.randn(size_n, generator=g).bfloat16().to(dev)
    c = torch.full((size_m, size_n), 7.0, dtype=torch.bfloat16, device=dev)
    out = run_gemm(ops, layer, a, dev, workspace, bias=marlin_permute_bias(bias), c=c)
    assert out.data_ptr() == c.data_ptr()
    check_close(out, a, layer, bias=bias)


@pytest.mark.parametrize("ws_len", [64, 128, 256, 1024])
def test_split_k_with_short_workspaces(ops, dev, ws_len):
    """K-split launches place the tile counters 1, 2 or 4 ints apart depending on the workspace length (the reference's
    marlin_make_workspace_new gives one int per compute unit); results do not depend on it and the counters end at zero."""
    size_m, size_k, size_n = 16, 4096, 4096          # 64 tiles of 64 columns, K split in four
    layer = make_layer(size_k, size_n, 128, torch.float16, seed=51, rule="absmax7", w_std=0.02)
    a = _a(size_m, size_k, torch.float16, dev, seed=52)
    ws = torch.zeros(ws_len, dtype=torch.int32, device=dev)
    out = run_gemm(ops, layer, a, dev, ws)
    check_close(out, a, layer)
    assert int(ws.abs().sum()) == 0
    big = torch.zeros(4096, dtype=torch.int32, device=dev)
    assert torch.equal(out, run_gemm(ops, layer, a, dev, big))
    assert torch.equal(out, run_gemm(ops, layer, a, dev, ws))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mode,group", [("gptq", 128), ("gptq", -1), ("awq", 64), ("gptq_act_order", 128)])
@pytest.mark.parametrize("size_m", [65, 100, 128])
def test_two_row_tiles_of_256_columns(ops, dev, workspace, dtype, mode, group, size_m):
    """65..128 rows and N wide enough that two row tiles of 64 x 256 give most compute units a workgroup: the kernel with
    the in-workgroup K split.  N = 25664 leaves a partial 256-column tile; one-hot rows must be bit-exact."""
    size_k, size_n = 1024, 25664
    print(f"kq dtype={dtype} {mode} g={group} m={size_m}", flush=True)
    layer = make_layer(size_k, size_n, group, dtype, has_zp=(mode == "awq"), act_order=(mode == "gptq_act_order"),
                       seed=size_m)
    a = _a(size_m, size_k, dtype, dev)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)
    ks = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(3))
    hot = torch.zeros(size_m, size_k, dtype=dtype)
    hot[torch.arange(size_m), ks] = 1.0
    out = run_gemm(ops, layer, hot.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    assert int(workspace.abs().sum()) == 0


@pytest.mark.parametrize("dtype,mode,group", [(torch.float16, "gptq", 128), (torch.bfloat16, "awq", 128)])
def test_one_row_tile_of_256_columns(ops, dev, workspace, dtype, mode, group):
    """33..64 rows with N so wide (193 tiles of 256 columns) that one row tile fills the chip: same kernel as above."""
    size_m, size_k, size_n = 40, 512, 49216
    layer = make_layer(size_k, size_n, group, dtype, has_zp=(mode == "awq"), seed=77)
    a = _a(size_m, size_k, dtype, dev)
    out = run_gemm(ops, layer, a, dev, workspace)
    check_close(out, a, layer)
    ks = torch.randint(0, size_k, (size_m,), generator=torch.Generator().manual_seed(3))
    hot = torch.zeros(size_m, size_k, dtype=dtype)
    hot[torch.arange(size_m), ks] = 1.0
    out = run_gemm(ops, layer, hot.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    assert int(workspace.abs().sum()) == 0


# ------------------------------------------------- decode kernel with more column tiles than compute units
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("has_zp,group_size", [(False, 128), (True, 128), (False, -1), (True, 64)])
def test_decode_more_tiles_than_compute_units(ops, dev, workspace, dtype, has_zp, group_size):
    """N / 128 = 320 column tiles: the launch runs as 4-wavefront workgroups, two to a compute unit, whose final phase
    walks the tile's 16 rows in two passes.  One-hot rows bit for bit, random rows within the GEMM tolerance."""
    size_k, size_n = 256, 128 * 320
    print(f"wide decode dtype={dtype} zp={has_zp} g={group_size}", flush=True)
    layer = make_layer(size_k, size_n, group_size, dtype, has_zp=has_zp, seed=21)
    ks = torch.tensor([0, 1, 9, 15, 16, 31, 32, 63, 64, 100, 127, 128, 200, 254, 255, 77])
    a = torch.zeros(16, size_k, dtype=dtype)
    a[torch.arange(16), ks] = 1.0
    out = run_gemm(ops, layer, a.to(dev), dev, workspace)
    assert torch.equal(out.cpu(), layer.w_ref[ks])
    for m in (3, 13):  # rows 8..15 absent / present
        a = _a(m, size_k, dtype, dev, seed=22 + m)
        check_close(run_gemm(ops, layer, a, dev, workspace), a, layer)
    assert int(workspace.abs().sum()) == 0
