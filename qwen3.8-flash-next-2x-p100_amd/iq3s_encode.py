"""An IQ3_S encoder in torch (runs on the GPU or the CPU), for making synthetic expert weights from float matrices.

This is this build's own encoder, not ggml's quantize_row_iq3_s (which is not in the reference tree): per 32-weight
sub-block it tries the scales amax / c for c in (15, 13.5, 12, 10.5, 9), codes every group of four magnitudes with the
nearest codebook entry and keeps the scale with the least squared error; the block scale is the largest sub-block scale
/ 31 as a half, sub-block codes s = round((scale / d - 1) / 2) in 0..15, and the groups are coded again against
d (1 + 2 s). Signs are the weights' own. The block layout is ggml's block_iq3_s (tensor_convert.hpp:295-322 reads it):
d (f16), qs[64], qh[8], signs[32], scales[4] = 110 bytes per 256 weights."""
import os
import re

import torch

IQ3S_BLOCK = 110
_CANDIDATES = (15.0, 13.5, 12.0, 10.5, 9.0)
_grid_cache = {}


def grid(device):
    """the codebook as [512][4] float magnitudes (the build's table in csrc/iq3s_grid.h: low byte first)"""
    key = str(device)
    if key not in _grid_cache:
        text = open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "iq3s_grid.h")).read()
        body = text[text.index("fnx_iq3s_grid_host[512]"):]
        words = [int(h, 16) for h in re.findall(r"0x([0-9a-fA-F]{8})", body)][:512]
        assert len(words) == 512
        g = torch.tensor([[(v >> (8 * j)) & 255 for j in range(4)] for v in words], dtype=torch.float32)
        _grid_cache[key] = g.to(device)
    return _grid_cache[key]


def _nearest(a, g, chunk=1 << 18):
    """a: [M][4] magnitudes in codebook units -> the index of the nearest entry (squared error) and that error"""
    idx = torch.empty(a.shape[0], dtype=torch.int64, device=a.device)
    g2 = (g * g).sum(dim=1)
    for i in range(0, a.shape[0], chunk):
        c = a[i:i + chunk]
        idx[i:i + chunk] = (g2[None, :] - 2.0 * (c @ g.T)).argmin(dim=1)
    err = ((a - g[idx]) ** 2).sum(dim=1)
    return idx, err


def encode_iq3s(w):
    """w: float tensor with a multiple of 256 values (rows of ncols % 256 == 0, row-major) -> uint8 tensor of blocks"""
    x = w.reshape(-1).to(torch.float32)
    assert x.numel() % 256 == 0
    B = x.numel() // 256
    dev = x.device
    g = grid(dev)
    x = x.view(B, 8, 8, 4)                     # [block][sub-block][group][weight]
    ax = x.abs()
    amax = ax.amax(dim=(2, 3))                 # [B][8]
    best = torch.full((B, 8), float("inf"), device=dev)
    sc = torch.zeros((B, 8), device=dev)
    for c in _CANDIDATES:
        s = torch.where(amax > 0, amax / c, torch.ones_like(amax))
        a = (ax / s[:, :, None, None]).reshape(-1, 4)
        _, e = _nearest(a, g)
        err = e.view(B, 8, 8).sum(dim=2) * s * s
        take = (err < best) & (amax > 0)
        best = torch.where(take, err, best)
        sc = torch.where(take, s, sc)
    dh = (sc.amax(dim=1) / 31.0).to(torch.float16)
    d = dh.to(torch.float32)
    s4 = torch.where(d[:, None] > 0, torch.round((sc / d[:, None].clamp_min(1e-30) - 1.0) * 0.5), torch.zeros_like(sc)).clamp(0, 15)
    db = d[:, None] * (1.0 + 2.0 * s4)
    a = torch.where(db[:, :, None, None] > 0, ax / db[:, :, None, None].clamp_min(1e-30), torch.zeros_like(ax)).reshape(-1, 4)
    gi, _ = _nearest(a, g)
    gi = gi.view(B, 8, 8)
    out = torch.zeros((B, IQ3S_BLOCK), dtype=torch.uint8, device=dev)
    out[:, 0:2] = dh.view(torch.uint8).view(B, 2)
    out[:, 2:66] = (gi & 255).to(torch.uint8).view(B, 64)
    sh = torch.arange(8, device=dev)
    out[:, 66:74] = (((gi >> 8) & 1) << sh[None, None, :]).sum(dim=2).to(torch.uint8)
    neg = (x < 0).to(torch.int64)                                           # [B][8][8][4]
    nib = (neg << torch.arange(4, device=dev)[None, None, None, :]).sum(dim=3)   # a group's four sign bits
    out[:, 74:106] = (nib[:, :, 0::2] | (nib[:, :, 1::2] << 4)).to(torch.uint8).view(B, 32)
    s4i = s4.to(torch.int64)
    out[:, 106:110] = (s4i[:, 0::2] | (s4i[:, 1::2] << 4)).to(torch.uint8)
    return out.reshape(-1)
