"""Eager PyTorch deformable multi-view SDPA (any device, autograd by PyTorch).

The counterpart of the reference's ``deform_sdpa_torch`` (``ops/torch.py:5-28``):
a separate, unfused operator that materialises the sampled keys and values. It
is never used by ``ops.triton.deform_sdpa_triton``; it exists so that callers
written against ``from ops.torch import deform_sdpa_torch`` (``benchmark.py:7``)
keep working. K and V are stacked along the channel axis so that each key view
costs one ``grid_sample`` call, and the softmax is taken in base 2 exactly as
the reference does (``ops/torch.py:20-25``).
"""
import torch
import torch.nn.functional as F

_LOG2E = 1.4426950408889634


def deform_sdpa_torch(q, k, v, coords, WIDTH, HEIGHT, sm_scale):
    B, V, H, L, D = q.shape
    P = coords.shape[-2]
    f32 = torch.float32
    # (B, V, H, L, 2D) -> one 2D-channel image per (b, h) and key view
    kv = torch.cat([k, v], dim=-1).to(f32)
    kv = kv.permute(0, 2, 1, 4, 3).reshape(B * H, V, 2 * D, HEIGHT, WIDTH)
    # grid for key view s2: all (s1, l) queries x P samples, shared by heads
    grid = coords.to(f32).mul(2.0).sub(1.0)                         # (B, s1, L, s2, P, 2)
    grid = grid.permute(0, 3, 1, 2, 4, 5).reshape(B, V, V * L, P, 2)
    sampled = []
    for s2 in range(V):
        g = grid[:, s2].unsqueeze(1).expand(B, H, V * L, P, 2).reshape(B * H, V * L, P, 2)
        sampled.append(F.grid_sample(kv[:, s2], g, mode="bilinear", padding_mode="zeros", align_corners=True))
    sampled = torch.stack(sampled, dim=3)                           # (B*H, 2D, V*L, s2, P)
    sampled = sampled.reshape(B, H, 2 * D, V, L, V * P).permute(0, 3, 1, 4, 5, 2)   # (B, s1, H, L, N, 2D)
    ks, vs = sampled[..., :D], sampled[..., D:]
    logits = torch.einsum("bshld,bshlnd->bshln", q.to(f32) * (sm_scale * _LOG2E), ks)
    w = torch.exp2(logits - logits.amax(dim=-1, keepdim=True))
    w = w / w.sum(dim=-1, keepdim=True)
    out = torch.einsum("bshln,bshlnd->bshld", w, vs)
    return out.to(q.dtype)
