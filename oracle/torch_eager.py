"""The op through ATen library routines -- TEST INFRASTRUCTURE ONLY.

``grid_sample`` (bilinear, zeros padding, ``align_corners=True``) followed by
``softmax`` and a weighted sum: the semantics of ``ops/torch.py:5-28`` said
with library calls, used (a) to pin the C oracle against a library routine,
(b) through PyTorch autograd to pin the C oracle's backward, and (c) as the
"host-CPU torch" baseline timed by ``bench.py``. Written independently of the
reference: views are folded into the batch so each of K and V takes a single
``grid_sample`` call, and the softmax is the library's natural-base one
(mathematically identical to the reference's base-2 form,
``ops/torch.py:20-25``).
"""
import torch
import torch.nn.functional as F


def deform_sdpa_eager(q, k, v, coords, WIDTH, HEIGHT, sm_scale, dtype=torch.float32):
    """q,k,v (B,V,H,L,D); coords (B,V,L,V,P,2) in [0,1]. Returns (B,V,H,L,D) in q.dtype."""
    B, V, H, L, D = q.shape
    P = coords.shape[-2]
    # feature maps: one image per (b, s2, h): (B*V*H, D, Himg, Wimg)   [ops/torch.py:8-9]
    def as_maps(t):
        return t.to(dtype).permute(0, 1, 2, 4, 3).reshape(B * V * H, D, HEIGHT, WIDTH)
    # sampling grid per (b, s2, h): all (s1, l) queries x P samples      [ops/torch.py:10-11]
    g = coords.to(dtype).permute(0, 3, 1, 2, 4, 5)             # (B, s2, s1, L, P, 2)
    g = g.reshape(B, V, 1, V * L, P, 2).expand(B, V, H, V * L, P, 2)
    g = g.reshape(B * V * H, V * L, P, 2) * 2.0 - 1.0          # [0,1] -> [-1,1]  [ops/torch.py:14]
    ks = F.grid_sample(as_maps(k), g, mode="bilinear", padding_mode="zeros", align_corners=True)
    vs = F.grid_sample(as_maps(v), g, mode="bilinear", padding_mode="zeros", align_corners=True)
    # (B*V*H, D, V*L, P) -> (B, s1, H, L, s2*P, D): samples ordered view-major [ops/torch.py:16-17]
    def as_samples(t):
        t = t.reshape(B, V, H, D, V, L, P)                      # b s2 h d s1 l p
        return t.permute(0, 4, 2, 5, 1, 6, 3).reshape(B, V, H, L, V * P, D)
    ks, vs = as_samples(ks), as_samples(vs)
    logits = torch.matmul(ks, q.to(dtype).unsqueeze(-1)).squeeze(-1) * sm_scale   # (B,V,H,L,N)
    p = torch.softmax(logits, dim=-1)
    out = torch.matmul(p.unsqueeze(-2), vs).squeeze(-2)
    return out.to(q.dtype)


def deform_sdpa_eager_chunked(q, k, v, coords, WIDTH, HEIGHT, sm_scale):
    """Same result, one (batch, head) at a time to bound host memory.

    Exact: batches and heads are independent and coords are shared by heads.
    """
    B, V, H, L, D = q.shape
    out = torch.empty_like(q)
    for b in range(B):
        for h in range(H):
            out[b:b + 1, :, h:h + 1] = deform_sdpa_eager(
                q[b:b + 1, :, h:h + 1], k[b:b + 1, :, h:h + 1], v[b:b + 1, :, h:h + 1],
                coords[b:b + 1], WIDTH, HEIGHT, sm_scale)
    return out


def eager_fwd_bwd(q, k, v, coords, dout, WIDTH, HEIGHT, sm_scale, dtype=torch.float32, chunked=False,
                  with_coords=False):
    """out, dq, dk, dv [, dcoords] through PyTorch autograd (used to pin the C oracle's backward)."""
    qd = q.detach().to(dtype).requires_grad_(True)
    kd = k.detach().to(dtype).requires_grad_(True)
    vd = v.detach().to(dtype).requires_grad_(True)
    cd = coords.detach().to(dtype)
    if with_coords:
        cd.requires_grad_(True)
    if chunked:
        B, V, H, L, D = q.shape
        outs = torch.empty_like(qd)
        for b in range(B):
            for h in range(H):
                o = deform_sdpa_eager(qd[b:b + 1, :, h:h + 1], kd[b:b + 1, :, h:h + 1],
                                      vd[b:b + 1, :, h:h + 1], cd[b:b + 1], WIDTH, HEIGHT, sm_scale, dtype)
                o.backward(dout[b:b + 1, :, h:h + 1].to(dtype))
                outs.data[b:b + 1, :, h:h + 1] = o.detach()
        out = outs.detach()
    else:
        out = deform_sdpa_eager(qd, kd, vd, cd, WIDTH, HEIGHT, sm_scale, dtype)
        out.backward(dout.to(dtype))
        out = out.detach()
    if with_coords:
        return out, qd.grad, kd.grad, vd.grad, cd.grad
    return out, qd.grad, kd.grad, vd.grad
