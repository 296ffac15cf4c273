"""A Swin-MoE-shaped model around hexa_moe.moe.MoE_Cascaded: the caller side of the operators.

It restates the model the reference trains (Swin-Transformer-MoE/models/swin_transformer_moe_cascaded.py:
650-879) with stock PyTorch only -- no timm, no window_process extension: patch embedding, four stages of
shifted-window attention blocks (continuous relative position bias from a small MLP, as in :160-201,
evaluated through scaled_dot_product_attention), patch merging between stages, and ONE MoE_Cascaded object
that owns every depth's FFN, dense or MoE, and is called once per block with the depth index (:859-866).
Only the FFN depths run this build's kernels; everything else here is ordinary torch and exists so that the
operators can be exercised at the shapes, call order and autocast setting of their real caller.

Differences from the reference model that a user can see:
  * no process group is needed (the reference multiplies the expert count by the world size, :709-711);
    `num_experts` is the global number;
  * the activation handed to MoE_Cascaded is plain GELU when `moe_drop == 0` (which lets the layer fuse it
    into the fc1 kernel) and GELU followed by dropout otherwise (the reference always wraps, :826);
  * weights are drawn with torch.nn.init.trunc_normal_ (same distribution as timm's).
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from hexa_moe import moe as hmoe


def _windows(x, w):
    """[B,H,W,C] -> [B, nW, w*w, C], windows in row-major order."""
    B, H, W, C = x.shape
    x = x.reshape(B, H // w, w, W // w, w, C).permute(0, 1, 3, 2, 4, 5)
    return x.reshape(B, (H // w) * (W // w), w * w, C)


def _unwindows(x, w, H, W):
    """Inverse of _windows."""
    B, _, _, C = x.shape
    x = x.reshape(B, H // w, W // w, w, w, C).permute(0, 1, 3, 2, 4, 5)
    return x.reshape(B, H, W, C)


class StochasticDepth(nn.Module):
    """Drops the whole residual branch of a sample with probability p (training only)."""

    def __init__(self, p):
        super().__init__()
        self.p = float(p)

    def forward(self, x):
        if self.p == 0.0 or not self.training:
            return x
        keep = 1.0 - self.p
        mask = x.new_empty((x.shape[0],) + (1,) * (x.dim() - 1)).bernoulli_(keep)
        return x * mask / keep


class WindowAttention(nn.Module):
    """Multi-head attention inside w x w windows with a learned continuous position bias."""

    def __init__(self, dim, w, heads):
        super().__init__()
        self.w, self.heads = w, heads
        self.qkv = nn.Linear(dim, 3 * dim)
        self.proj = nn.Linear(dim, dim)
        self.cpb_mlp = nn.Sequential(nn.Linear(2, 512), nn.ReLU(inplace=True), nn.Linear(512, heads, bias=False))
        # log-spaced relative offsets in [-1,1] for every (dy,dx) in (-(w-1) .. w-1)^2
        r = torch.arange(-(w - 1), w, dtype=torch.float32)
        table = torch.stack(torch.meshgrid(r, r, indexing="ij"), dim=-1) / max(w - 1, 1) * 8
        table = torch.sign(table) * torch.log2(table.abs() + 1.0) / math.log2(8)
        self.register_buffer("offset_table", table.reshape(-1, 2))
        pos = torch.stack(torch.meshgrid(torch.arange(w), torch.arange(w), indexing="ij")).flatten(1)   # [2, w*w]
        rel = pos[:, :, None] - pos[:, None, :] + (w - 1)
        self.register_buffer("offset_index", (rel[0] * (2 * w - 1) + rel[1]).reshape(-1))

    def forward(self, x, shift_mask):
        """x [B, nW, N, C]; shift_mask [nW, N, N] (0 / -100) or None."""
        B, nW, N, C = x.shape
        qkv = self.qkv(x).reshape(B, nW, N, 3, self.heads, C // self.heads).permute(3, 0, 1, 4, 2, 5)
        bias = self.cpb_mlp(self.offset_table)[self.offset_index].reshape(N, N, self.heads).permute(2, 0, 1)
        bias = bias[None, None] if shift_mask is None else bias[None, None] + shift_mask[None, :, None]
        out = F.scaled_dot_product_attention(qkv[0], qkv[1], qkv[2], attn_mask=bias.to(qkv.dtype))
        return self.proj(out.transpose(2, 3).reshape(B, nW, N, C))


class AttentionHalf(nn.Module):
    """The attention half of a Swin block; returns the normalised FFN input and the residual, the
    FFN itself being the model-wide MoE_Cascaded's (reference :369-406)."""

    def __init__(self, dim, res, heads, w, shift, drop_path):
        super().__init__()
        if min(res) <= w:          # a window as large as the map: one window, no shift
            w, shift = min(res), 0
        self.res, self.w, self.shift = res, w, shift
        self.norm1, self.norm2 = nn.LayerNorm(dim), nn.LayerNorm(dim)
        self.attn = WindowAttention(dim, w, heads)
        self.drop_path = StochasticDepth(drop_path)
        mask = None
        if shift > 0:              # tokens that wrapped around must not attend across the seam
            H, W = res
            region = torch.zeros(1, H, W, 1)
            cuts = (slice(0, -w), slice(-w, -shift), slice(-shift, None))
            for i, hs in enumerate(cuts):
                for j, ws in enumerate(cuts):
                    region[:, hs, ws, :] = i * 3 + j
            ids = _windows(region, w)[0, :, :, 0]                      # [nW, N]
            mask = (ids[:, None, :] != ids[:, :, None]).float() * -100.0
        self.register_buffer("shift_mask", mask)

    def forward(self, x):
        H, W = self.res
        B, L, C = x.shape
        y = self.norm1(x).reshape(B, H, W, C)
        if self.shift:
            y = torch.roll(y, (-self.shift, -self.shift), dims=(1, 2))
        y = _unwindows(self.attn(_windows(y, self.w), self.shift_mask), self.w, H, W)
        if self.shift:
            y = torch.roll(y, (self.shift, self.shift), dims=(1, 2))
        x = x + self.drop_path(y.reshape(B, L, C))
        return self.norm2(x), x


class PatchMerging(nn.Module):
    """2x2 neighbourhoods concatenated (4C), normalised, projected to 2C (reference :455-476)."""

    def __init__(self, res, dim):
        super().__init__()
        self.res = res
        self.norm = nn.LayerNorm(4 * dim)
        self.reduction = nn.Linear(4 * dim, 2 * dim, bias=False)

    def forward(self, x):
        H, W = self.res
        B, _, C = x.shape
        x = x.reshape(B, H // 2, 2, W // 2, 2, C).permute(0, 1, 3, 4, 2, 5)   # (.., col parity, row parity, C)
        return self.reduction(self.norm(x.reshape(B, (H // 2) * (W // 2), 4 * C)))


class SwinMoE(nn.Module):
    """Swin Transformer whose FFNs all live in one MoE_Cascaded.  Defaults: the Swin-MoE-S model of
    configs/swinmoe/swin_moe_small_patch4_window12_192_4gpu_1k.yaml:12-24 with 32 experts."""

    def __init__(self, img_size=192, patch_size=4, in_chans=3, num_classes=1000, embed_dim=96, depths=(2, 2, 18, 2),
                 num_heads=(3, 6, 12, 24), window_size=12, mlp_ratio=4.0,
                 moe_blocks=((-1,), (-1,), (1, 3, 5, 7, 9, 11, 13, 15, 17), (1,)), num_experts=32, top_value=1,
                 gate_noise=1.0, is_gshard_loss=False, moe_drop=0.0, drop_path_rate=0.2, mlp_fc2_bias=False,
                 init_std=0.005, aux_loss_weight=0.01):
        super().__init__()
        self.aux_loss_weight = aux_loss_weight
        self.init_std = init_std
        grid = img_size // patch_size
        self.patch_proj = nn.Conv2d(in_chans, embed_dim, kernel_size=patch_size, stride=patch_size)
        self.patch_norm = nn.LayerNorm(embed_dim)
        rates = torch.linspace(0, drop_path_rate, sum(depths)).tolist()
        self.blocks = nn.ModuleList()
        self.ffn_drop_path = nn.ModuleList()
        self.merges = nn.ModuleDict()          # keyed by the depth after which the merge happens
        dims, moe_depths, depth = [], [], 0
        for stage, n in enumerate(depths):
            dim, res = embed_dim * 2 ** stage, (grid // 2 ** stage, grid // 2 ** stage)
            for j in range(n):
                self.blocks.append(AttentionHalf(dim, res, num_heads[stage], window_size,
                                                 0 if j % 2 == 0 else window_size // 2, rates[depth]))
                self.ffn_drop_path.append(StochasticDepth(rates[depth]))
                dims.append(dim)
                if j in moe_blocks[stage]:
                    moe_depths.append(depth)
                depth += 1
            if stage < len(depths) - 1:
                self.merges[str(depth - 1)] = PatchMerging(res, dim)
        self.moe_depths = moe_depths
        self.moe_dropout = nn.Dropout(moe_drop)
        act = F.gelu if moe_drop == 0 else (lambda t: self.moe_dropout(F.gelu(t)))
        self.cascaded_moe = hmoe.MoE_Cascaded(
            gate_type={'type': 'top', 'k': top_value, 'gate_noise': gate_noise, 'fp32_gate': True},
            model_dim_list=dims, moe_idx_list=moe_depths, mlp_ratio=mlp_ratio, mlp_proportion=None,
            num_global_experts=num_experts, total_depth=sum(depths), data_centric=True, mlp_fc1_bias=False,
            mlp_fc2_bias=mlp_fc2_bias, activation_fn=act, is_gshard_loss=is_gshard_loss)
        self.norm = nn.LayerNorm(dims[-1])
        self.head = nn.Linear(dims[-1], num_classes)
        self.apply(self._init)

    def _init(self, m):
        if isinstance(m, nn.Linear):
            nn.init.trunc_normal_(m.weight, std=self.init_std)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.LayerNorm):
            nn.init.ones_(m.weight)
            nn.init.zeros_(m.bias)

    def forward(self, images, ffn_hook=None):
        """images [B,3,S,S] -> (logits [B,classes], weighted auxiliary loss).  ffn_hook(depth, ffn_in,
        ffn_out), if given, sees every FFN call (used by tests and per-layer timing)."""
        x = self.patch_norm(self.patch_proj(images).flatten(2).transpose(1, 2))
        l_aux = 0.0
        for depth, block in enumerate(self.blocks):
            ffn_in, shortcut = block(x)
            ffn_out, aux = self.cascaded_moe(depth, ffn_in)
            if ffn_hook is not None:
                ffn_hook(depth, ffn_in, ffn_out)
            x = shortcut + self.ffn_drop_path[depth](ffn_out)
            l_aux = l_aux + aux
            if str(depth) in self.merges:
                x = self.merges[str(depth)](x)
        x = self.norm(x).mean(dim=1)
        return self.head(x), l_aux * self.aux_loss_weight
