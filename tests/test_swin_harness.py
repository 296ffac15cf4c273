"""The Swin-MoE-shaped harness's own pieces on the CPU (the FFN depths need the GPU and are covered by
tests/test_gpu_swin_shape.py): window partitioning round trip, patch-merging channel order, and the
windowed attention against the explicit softmax formulation with the shift mask."""
import torch

import swin_moe_harness as S


def test_window_round_trip_and_merge_order():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 24, 24, 8, generator=g)
    w = S._windows(x, 12)
    assert w.shape == (2, 4, 144, 8)
    assert torch.equal(w[1, 3].reshape(12, 12, 8), x[1, 12:, 12:])
    assert torch.equal(S._unwindows(w, 12, 24, 24), x)
    pm = S.PatchMerging((24, 24), 8)
    pm.norm = torch.nn.Identity(); pm.reduction = torch.nn.Identity()
    t = x.reshape(2, 576, 8)
    want = torch.cat([x[:, 0::2, 0::2], x[:, 1::2, 0::2], x[:, 0::2, 1::2], x[:, 1::2, 1::2]], -1).reshape(2, 144, 32)
    assert torch.equal(pm(t), want)


def test_shifted_window_attention_matches_explicit_softmax():
    torch.manual_seed(1)
    dim, heads, w, res = 32, 4, 4, (8, 8)
    blk = S.AttentionHalf(dim, res, heads, w, shift=2, drop_path=0.0).eval()
    a = blk.attn
    x = torch.randn(3, 4, 16, dim)                       # [B, nW, N, C]
    got = a(x, blk.shift_mask)
    qkv = a.qkv(x).reshape(3, 4, 16, 3, heads, dim // heads)
    q, k, v = (qkv[:, :, :, i].permute(0, 1, 3, 2, 4) for i in range(3))      # [B,nW,h,N,hd]
    table = a.cpb_mlp(a.offset_table)                    # [(2w-1)^2, heads]
    bias = torch.empty(heads, 16, 16)
    for i in range(16):
        for j in range(16):
            dy, dx = i // w - j // w, i % w - j % w
            bias[:, i, j] = table[(dy + w - 1) * (2 * w - 1) + (dx + w - 1)]
    logits = q @ k.transpose(-1, -2) / (dim // heads) ** 0.5 + bias[None, None] + blk.shift_mask[None, :, None]
    want = a.proj((logits.softmax(-1) @ v).permute(0, 1, 3, 2, 4).reshape(3, 4, 16, dim))
    assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
    # the mask separates exactly the wrapped-around regions: the last window holds 4 of them
    assert blk.shift_mask.shape == (4, 16, 16) and (blk.shift_mask[0] == 0).all()
    assert int((blk.shift_mask[3] == 0).sum()) == 4 * (2 * 2) ** 2


def test_model_layout_follows_the_swin_moe_small_config():
    m = S.SwinMoE(num_experts=4, num_classes=10)
    assert m.moe_depths == [5, 7, 9, 11, 13, 15, 17, 19, 21, 23]
    c = m.cascaded_moe
    assert [tuple(w.shape) for w in c.batched_fc1_w] == [(4, 1536, 384)] * 9 + [(4, 3072, 768)]
    assert len(c.mlp_fc1_w) == 14 and [b.shift for b in m.blocks[:4]] == [0, 6, 0, 6]
    assert m.blocks[-1].w == 6 and m.blocks[-1].shift == 0 and m.blocks[5].w == 12 and m.blocks[5].shift == 0
