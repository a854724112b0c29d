"""w4a16_marlin_gemm_static (the GEMM entry point that allocates nothing: split-K partials, the act-order copy of A and
the arrival counters live in the library's own device memory) against w4a16_marlin_gemm, through the C ABI.  Results
must be bit-identical (same plan, same ordered split-K sums).  Each case makes two calls in a row, the second with a
smaller input, so that stale scratch contents of the first call would show."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _args(lib_mod, a, c, layer_dev, m, n, k, groups, ws, c_tmp, zp, g_idx, perm, dtype):
    args = lib_mod.GemmArgs()
    args.struct_size = ctypes.sizeof(lib_mod.GemmArgs)
    args.dtype = lib_mod.DTYPE_F16 if dtype == torch.float16 else lib_mod.DTYPE_BF16
    args.wtype = lib_mod.WTYPE_U4 if zp is not None else lib_mod.WTYPE_U4B8
    args.flags = lib_mod.F_IS_K_FULL | lib_mod.F_USE_FP32_REDUCE
    args.a, args.lda, args.c = a.data_ptr(), a.stride(0), c.data_ptr()
    args.b_q_weight, args.b_scales = layer_dev["q"].data_ptr(), layer_dev["s"].data_ptr()
    args.b_zeros = None if zp is None else zp.data_ptr()
    args.g_idx = None if g_idx is None else g_idx.data_ptr()
    args.perm = None if perm is None else perm.data_ptr()
    args.c_tmp = None if c_tmp is None else c_tmp.data_ptr()
    args.workspace = None if ws is None else ws.data_ptr()
    args.workspace_len = 0 if ws is None else ws.numel()
    args.size_m, args.size_n, args.size_k, args.num_groups = m, n, k, groups
    return args


CASES = [
    # (k, n, group, dtype, zp, act_order, (m_first, m_second))
    (14336, 4096, 128, torch.float16, False, False, (16, 3)),     # decode kernel, K split across workgroups
    (4096, 4096, 128, torch.float16, False, False, (16, 1)),      # decode kernel, small layer
    (2048, 512, 128, torch.bfloat16, True, False, (48, 16)),      # general kernel with a K split, zero points
    (1024, 4096, 128, torch.float16, False, False, (200, 64)),    # 17..128 and more rows on few tiles
    (2048, 16384, 128, torch.float16, False, False, (256, 200)),  # 64-row kernel, two-pass K split (32 MiB of partials)
    (2048, 1024, 128, torch.float16, False, True, (40, 5)),       # act-order: A gathered into the scratch
    (4096, 6144, 128, torch.bfloat16, True, False, (300, 130)),   # prefill kernel (no scratch needed)
    (1024, 4096, 128, torch.bfloat16, True, False, (2048, 1600)), # 128 x 256 tiles, K halves inside the workgroup
    (512, 6144, 128, torch.float16, False, False, (4096, 4000)),  # prefill kernel + 128 x 256 tiles on the last strips
]


@pytest.mark.parametrize("k,n,group,dtype,zp,act_order,ms", CASES)
def test_static_scratch_gemm_matches(dev, k, n, group, dtype, zp, act_order, ms):
    from helpers import make_layer
    from vllm_amd import _lib
    lib = _lib.load()
    layer = make_layer(k, n, group, dtype, has_zp=zp, act_order=act_order, seed=11, w_std=0.05)
    ld = {"q": layer.marlin_q.to(dev), "s": layer.marlin_s.to(dev)}
    zpt = layer.marlin_zp.to(dev) if zp else None
    g_idx = layer.g_idx_sorted.to(dev) if act_order else None
    perm = layer.sort_indices.to(dev) if act_order else None
    ws = torch.zeros(4096, dtype=torch.int32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    for m in ms:
        print(f"static scratch case k={k} n={n} dtype={dtype} zp={zp} act_order={act_order} m={m}", flush=True)
        a = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).to(dtype).to(dev)
        want = torch.zeros(m, n, dtype=dtype, device=dev)
        got = torch.zeros(m, n, dtype=dtype, device=dev)
        args = _args(_lib, a, want, ld, m, n, k, layer.marlin_s.shape[0], ws, None, zpt, g_idx, perm, dtype)
        need = lib.w4a16_gemm_scratch_bytes(ctypes.byref(args))
        assert 0 <= need <= _lib.STATIC_SCRATCH_BYTES
        c_tmp = torch.empty(max(need // 4, 1), dtype=torch.float32, device=dev)
        args.c_tmp = c_tmp.data_ptr()
        _lib.check(lib.w4a16_marlin_gemm(ctypes.byref(args), stream))
        sargs = _args(_lib, a, got, ld, m, n, k, layer.marlin_s.shape[0], None, None, zpt, g_idx, perm, dtype)
        _lib.check(lib.w4a16_marlin_gemm_static(ctypes.byref(sargs), stream))
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert float(want.float().abs().max()) > 0
        assert int(ws.abs().sum()) == 0


def test_static_scratch_gemm_rejects_oversized(dev):
    """A problem whose scratch exceeds the static buffer fails with a message and launches nothing."""
    from vllm_amd import _lib
    lib = _lib.load()
    k, n, m = 14336, 4096, 4096   # act-order copy of A alone: 4096 x 14336 x 2 bytes = 112 MiB
    q = torch.zeros(k // 16, 2 * n, dtype=torch.int32, device=dev)
    s = torch.ones(k // 128, n, dtype=torch.float16, device=dev)
    idx = torch.arange(k, dtype=torch.int32, device=dev)
    g_idx = (idx // 128).contiguous()
    a = torch.zeros(m, k, dtype=torch.float16, device=dev)
    c = torch.full((m, n), 7.0, dtype=torch.float16, device=dev)
    args = _args(_lib, a, c, {"q": q, "s": s}, m, n, k, k // 128, None, None, None, g_idx, idx, torch.float16)
    rc = lib.w4a16_marlin_gemm_static(ctypes.byref(args), ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == -1
    assert b"static buffer" in lib.w4a16_last_error()
    torch.cuda.synchronize()
    assert float(c.min()) == 7.0 and float(c.max()) == 7.0


def _moe_args(lib_mod, a, c, q, s, g_idx, perm, ws, align, tw, bs, topk, m, n, k, e):
    sorted_ids, expert_ids, post = align
    args = _args(lib_mod, a, c, {"q": q, "s": s}, m, n, k, s.shape[1], ws, None, None, g_idx, perm, torch.float16)
    args.flags |= lib_mod.F_MOE | lib_mod.F_MUL_TOPK_WEIGHTS
    args.sorted_token_ids, args.expert_ids = sorted_ids.data_ptr(), expert_ids.data_ptr()
    args.num_tokens_past_padded, args.topk_weights = post.data_ptr(), tw.data_ptr()
    args.n_sorted = min(sorted_ids.numel(), expert_ids.numel() * bs)
    args.moe_block_size, args.top_k, args.num_experts = bs, topk, e
    return args


@pytest.mark.parametrize("bs,ms", [(16, (24, 5)), (64, (600, 200))])
def test_static_scratch_moe_gemm_matches(dev, bs, ms):
    """The MoE mode through the entry point that allocates nothing: blocks of 16 (16-row kernel) and blocks of 64 (64-row
    kernel, whose K split of the tail tiles is decided on the device and keeps its partial tiles in the scratch)."""
    from test_gpu_moe import make_experts, rand_topk
    from vllm_amd import _lib
    from vllm_amd.moe_align_block_size import moe_align_block_size
    lib = _lib.load()
    e, topk, k, n = 4, 2, 4096, 512
    layers, mq, ms_, _, _, _ = make_experts(e, k, n, 128, torch.float16, False, False, seed=70)
    q, s = mq.to(dev), ms_.to(dev)
    ws = torch.zeros(4096, dtype=torch.int32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    for m in ms:
        print(f"static scratch MoE case bs={bs} m={m}", flush=True)
        a = (torch.randn(m, k, generator=torch.Generator().manual_seed(m)) / 4).half().to(dev)
        ids = rand_topk(m, topk, e, seed=m).to(dev)
        tw = torch.rand(m, topk, generator=torch.Generator().manual_seed(7)).to(dev)
        align = moe_align_block_size(ids, bs, e)
        want = torch.zeros(m * topk, n, dtype=torch.float16, device=dev)
        got = torch.zeros(m * topk, n, dtype=torch.float16, device=dev)
        args = _moe_args(_lib, a, want, q, s, None, None, ws, align, tw, bs, topk, m, n, k, e)
        need = lib.w4a16_gemm_scratch_bytes(ctypes.byref(args))
        assert 0 <= need <= _lib.STATIC_SCRATCH_BYTES
        c_tmp = torch.empty(max(need // 4, 1), dtype=torch.float32, device=dev)
        args.c_tmp = c_tmp.data_ptr()
        _lib.check(lib.w4a16_marlin_gemm(ctypes.byref(args), stream))
        sargs = _moe_args(_lib, a, got, q, s, None, None, None, align, tw, bs, topk, m, n, k, e)
        _lib.check(lib.w4a16_marlin_gemm_static(ctypes.byref(sargs), stream))
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert float(want.float().abs().max()) > 0 and int(ws.abs().sum()) == 0


def test_static_scratch_moe_act_order_is_refused_when_it_does_not_fit(dev):
    """MoE with act-order needs one gathered row of A per sorted slot on top of the partial tiles: a call whose total
    exceeds the static buffer is refused with the message, and nothing is launched."""
    from vllm_amd import _lib
    from vllm_amd.moe_align_block_size import moe_align_block_size
    lib = _lib.load()
    e, topk, k, n, m, bs = 8, 2, 14336, 4096, 2048, 64
    q = torch.zeros(e, k // 16, 2 * n, dtype=torch.int32, device=dev)
    s = torch.ones(e, k // 128, n, dtype=torch.float16, device=dev)
    idx = torch.arange(k, dtype=torch.int32, device=dev).repeat(e, 1).contiguous()
    g_idx = (idx // 128).contiguous()
    a = torch.zeros(m, k, dtype=torch.float16, device=dev)
    ids = (torch.arange(m * topk, device=dev, dtype=torch.int32) % e).view(m, topk).contiguous()
    tw = torch.ones(m, topk, device=dev)
    align = moe_align_block_size(ids, bs, e)
    c = torch.full((m * topk, n), 7.0, dtype=torch.float16, device=dev)
    args = _moe_args(_lib, a, c, q, s, g_idx, idx, None, align, tw, bs, topk, m, n, k, e)
    rc = lib.w4a16_marlin_gemm_static(ctypes.byref(args), ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == -1 and b"static buffer" in lib.w4a16_last_error()
    torch.cuda.synchronize()
    assert float(c.min()) == 7.0 and float(c.max()) == 7.0
