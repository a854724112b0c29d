"""Pins the oracle's Marlin layouts (weights, scales, bias, zero points) without the GPU.

Checks are independent of the formulas under test: hand-derived words, a second formulation,
brute-force scalar loops on the smallest tile, conservation laws and inverses.
"""
import numpy as np
import pytest
import torch

from oracle import marlin_layout as ml
from oracle import quant_utils as qu


def u32(t):
    return t.numpy().view(np.uint32)


def rand_q(k, n, seed=0):
    return torch.randint(0, 16, (k, n), generator=torch.Generator().manual_seed(seed), dtype=torch.int32)


# ------------------------------------------------------------------------------------ weights
def test_weights_known_words_q_equals_row():
    """q[k,n] = k on one 16x64 tile: thread th holds rows r=2(th%4) -> nibbles (r, r+8, r, r+8, r+1, r+9, r+1, r+9)."""
    q = torch.arange(16, dtype=torch.int32).view(16, 1).expand(16, 64).contiguous()
    w = u32(ml.marlin_weights_closed_form(q))[0]
    assert [hex(int(w[4 * th])) for th in range(4)] == ["0x91918080", "0xb3b3a2a2", "0xd5d5c4c4", "0xf7f7e6e6"]
    # all four sub-tile words of a thread are equal (rows only), and threads th, th+4 share rows
    for th in range(32):
        assert len({int(w[4 * th + i]) for i in range(4)}) == 1
        assert w[4 * th] == w[4 * (th % 4)]


def test_weights_known_words_q_equals_col():
    """q[k,n] = n % 16: word (th, w) has columns c = th//4 (+8 for nibbles 2,3,6,7) of sub-tile w."""
    q = (torch.arange(64, dtype=torch.int32) % 16).view(1, 64).expand(16, 64).contiguous()
    w = u32(ml.marlin_weights_closed_form(q))[0]
    assert hex(int(w[0 * 4 + 0])) == "0x88008800"
    assert hex(int(w[4 * 4 + 1])) == "0x99119911"
    assert hex(int(w[31 * 4 + 3])) == "0xff77ff77"


@pytest.mark.parametrize("k,n", [(16, 64), (64, 192), (128, 256)])
def test_two_formulations_agree(k, n):
    q = rand_q(k, n, seed=k + n)
    a = ml.marlin_weights_closed_form(q)
    b = ml.marlin_weights_perm_table(q)
    assert a.shape == (k // 16, 2 * n) and a.dtype == torch.int32
    assert torch.equal(a, b)


def test_brute_force_min_tile():
    """Scalar loop straight from the per-thread description, on the 16x64 tile."""
    q = rand_q(16, 64, seed=5)
    want = np.zeros(128, dtype=np.uint32)
    for th in range(32):
        for w in range(4):
            col = 16 * w + th // 4
            row = 2 * (th % 4)
            vals = [q[row, col], q[row + 8, col], q[row, col + 8], q[row + 8, col + 8],
                    q[row + 1, col], q[row + 9, col], q[row + 1, col + 8], q[row + 9, col + 8]]
            word = 0
            for j, v in enumerate(vals):
                word |= int(v) << (4 * j)
            want[th * 4 + w] = word
    assert np.array_equal(u32(ml.marlin_weights_closed_form(q))[0], want)


def test_nibble_multiset_and_inverse():
    q = rand_q(96, 128, seed=9)
    m = ml.marlin_weights_closed_form(q)
    nib = np.stack([(u32(m) >> np.uint32(4 * j)) & 0xF for j in range(8)])
    assert np.array_equal(np.bincount(nib.ravel(), minlength=16), np.bincount(q.numpy().ravel(), minlength=16))
    # every 16-row k-tile keeps its own nibbles
    for kt in range(96 // 16):
        assert np.array_equal(np.bincount(nib[:, kt].ravel(), minlength=16),
                              np.bincount(q[16 * kt:16 * kt + 16].numpy().ravel(), minlength=16))
    assert torch.equal(ml.marlin_unpack_weights(m), q)


def test_gptq_and_awq_checkpoints_repack_to_same_words():
    q = rand_q(64, 128, seed=3)
    a = ml.gptq_marlin_repack(qu.gptq_pack(q), None, 64, 128, 4)
    b = ml.awq_marlin_repack(qu.awq_pack(q), 64, 128, 4)
    assert torch.equal(a, b)
    assert torch.equal(a, ml.marlin_weights_closed_form(q))


def test_act_order_repack_is_repack_of_gathered_rows():
    q = rand_q(64, 64, seed=4)
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(1)).to(torch.int32)
    a = ml.gptq_marlin_repack(qu.gptq_pack(q), perm, 64, 64, 4)
    b = ml.gptq_marlin_repack(qu.gptq_pack(q[perm.long()]), None, 64, 64, 4)
    assert torch.equal(a, b)
    assert torch.equal(ml.marlin_weights_perm_table(q, perm), a)


# ------------------------------------------------------------------------------ scales / bias
def test_grouped_scale_perm_is_8x8_transpose():
    p = ml.scale_perm_grouped()
    assert sorted(p) == list(range(64))
    assert all(p[8 * c + j] == c + 8 * j for c in range(8) for j in range(8))
    assert [p[p[i]] for i in range(64)] == list(range(64))          # involution
    s = torch.arange(2 * 128, dtype=torch.float32).view(2, 128)
    out = ml.marlin_permute_scales(s, 256, 128, 128)
    for g in range(2):
        for chunk in range(2):
            blk = s[g, 64 * chunk:64 * chunk + 64].view(8, 8).t().reshape(-1)
            assert torch.equal(out[g, 64 * chunk:64 * chunk + 64], blk)
    assert torch.equal(ml.marlin_unpermute_scales(out, True), s)


def test_single_scale_perm_closed_form():
    """Channelwise scales and bias: 32-column chunks, position 8*i + t holds column 2*i + (0,1,8,9,16,17,24,25)[t]."""
    p = ml.scale_perm_single()
    assert sorted(p) == list(range(32))
    for cl in range(32):
        pos = 8 * ((cl & 7) >> 1) + 2 * (cl >> 3) + (cl & 1)
        assert p[pos] == cl
    s = torch.arange(64, dtype=torch.float32).view(1, 64)
    out = ml.marlin_permute_scales(s, 128, 64, -1)
    assert out[0, :8].tolist() == [0, 1, 8, 9, 16, 17, 24, 25]
    assert out[0, 32:40].tolist() == [32, 33, 40, 41, 48, 49, 56, 57]
    assert torch.equal(ml.marlin_permute_scales(s, 128, 64, 128), out)     # group == K is channelwise
    assert torch.equal(ml.marlin_unpermute_scales(out, False), s)
    b = torch.arange(64, dtype=torch.float32)
    assert torch.equal(ml.marlin_permute_bias(b), out[0])


# -------------------------------------------------------------------------------- zero points
def test_zero_points_closed_form_and_known_word():
    zp = (torch.arange(64, dtype=torch.int32) % 16).view(1, 64)
    m = ml.marlin_zero_points(zp, 1, 64)
    # word i, nibble t <- column i + 8*(0,2,4,6,1,3,5,7)[t];  column value = col % 16
    w0 = 0
    for t, o in enumerate((0, 2, 4, 6, 1, 3, 5, 7)):
        w0 |= ((0 + 8 * o) % 16) << (4 * t)
    assert int(u32(m)[0, 0]) == w0 == 0x88880000
    z = torch.randint(0, 16, (3, 192), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    a = ml.marlin_zero_points(z, 3, 192)
    assert torch.equal(a, ml.marlin_zero_points_closed_form(z))
    assert torch.equal(ml.marlin_unpack_zero_points(a), z)
    assert torch.equal(ml.awq_to_marlin_zero_points(qu.awq_pack(z), 3, 192), a)


# ------------------------------------------------------------------------------ 8-bit weights
def rand_q8(k, n, seed=0):
    return torch.randint(0, 256, (k, n), generator=torch.Generator().manual_seed(seed), dtype=torch.int32)


def test_weights8_known_words():
    """q[k,n] = k: word th*8 + 2w + half holds rows r, r+8, r+1, r+9 (r = 2(th%4)) in bytes 0..3."""
    q = torch.arange(16, dtype=torch.int32).view(16, 1).expand(16, 64).contiguous()
    w = u32(ml.marlin_weights_closed_form8(q))[0]
    assert [hex(int(w[8 * th])) for th in range(4)] == ["0x9010800", "0xb030a02", "0xd050c04", "0xf070e06"]
    # q[k,n] = n: every byte of word (th, w, half) is the column 16w + th//4 + 8*half
    q = torch.arange(64, dtype=torch.int32).view(1, 64).expand(16, 64).contiguous()
    w = u32(ml.marlin_weights_closed_form8(q))[0]
    for th, sub, half in ((0, 0, 0), (5, 1, 1), (31, 3, 1)):
        col = 16 * sub + th // 4 + 8 * half
        assert int(w[th * 8 + 2 * sub + half]) == col * 0x01010101


@pytest.mark.parametrize("k,n", [(16, 64), (64, 192)])
def test_weights8_two_formulations_inverse_and_checkpoints(k, n):
    q = rand_q8(k, n, seed=k * n)
    a = ml.marlin_weights_closed_form8(q)
    assert a.shape == (k // 16, 4 * n)
    assert torch.equal(a, ml.marlin_weights_perm_table(q, num_bits=8))
    assert torch.equal(ml.marlin_unpack_weights8(a), q)
    assert torch.equal(ml.gptq_marlin_repack(qu.pack_rows(q, 8), None, k, n, 8), a)
    assert torch.equal(ml.awq_marlin_repack(qu.awq_pack(q, 8), k, n, 8), a)
    perm = torch.randperm(k, generator=torch.Generator().manual_seed(2)).to(torch.int32)
    assert torch.equal(ml.gptq_marlin_repack(qu.pack_rows(q, 8), perm, k, n, 8), ml.marlin_weights_closed_form8(q[perm.long()]))


def test_pack8_literals():
    q = torch.tensor([[1], [2], [3], [4]], dtype=torch.int32)
    assert int(u32(qu.pack_rows(q, 8))[0, 0]) == 0x04030201
    q = torch.tensor([[1, 2, 3, 4]], dtype=torch.int32)
    assert int(u32(qu.awq_pack(q, 8))[0, 0]) == 0x04020301      # byte t holds column (0, 2, 1, 3)[t]
    assert torch.equal(qu.awq_unpack(qu.awq_pack(q, 8), 8), q)
