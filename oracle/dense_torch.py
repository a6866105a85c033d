"""Dense PyTorch restatement of the reference's pure-PyTorch pooling path.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product package never imports it.

This is the parity target: it follows the *formulation* of the reference's dense branch
  voxel centres      flashbev/flashbevpool/sampling_vt.py:364-378
  projection         flashbev/flashbevpool/sampling_vt.py:449-466  (einsum, signed clamp)
  pooling            flashbev/flashbevpool/sampling_vt.py:36-123   (two grid_sample calls,
                     likelihood, mask by multiplication, sum over cameras and height,
                     division by the clamped valid count)
  projection matrix  flashbev/flashbevpool/sampling_vt.py:21-33
i.e. it materialises the frustum volume per camera and uses the library routine
``torch.nn.functional.grid_sample(bilinear, border, align_corners=True)`` where the
fused kernel does explicit corner arithmetic.  Cameras are processed one at a time so the
larger configurations fit in host memory; autograd through it gives the true gradients.

The interface is channels-last like the fused operator: feats [B,N,H,W,C],
depth [B,N,H,W,D], result [B,gy,gx,C].

Depth model 2 (categorical bins, linear interpolation along depth) is an extension with no
counterpart in the reference: parity unpinned by the reference.
"""
from __future__ import annotations

from typing import Sequence

import torch
import torch.nn.functional as F


def projection_matrix(sensor2ego, camera2imgs, post_rots, post_trans):
    """[B,N,3,4] = ([post_rots @ K, post_trans added to column 2] embedded in I4) @ inv(sensor2ego)."""
    B, N = camera2imgs.shape[:2]
    K4 = torch.eye(4, dtype=camera2imgs.dtype, device=camera2imgs.device).repeat(B, N, 1, 1)
    K4[..., :3, :3] = post_rots @ camera2imgs
    K4[..., :3, 2] = K4[..., :3, 2] + post_trans
    return (K4 @ torch.linalg.inv(sensor2ego))[:, :, :3, :]


def voxel_centres(roi_range: Sequence[float], grid_size: Sequence[int], dtype=torch.float32):
    """[gx,gy,gz,3] centres: linspace(lo,hi,n+1)[:-1] + step/2 per axis, 'ij' meshgrid."""
    axes = []
    for a in range(3):
        lo, hi, n = float(roi_range[2 * a]), float(roi_range[2 * a + 1]), int(grid_size[a])
        step = (hi - lo) / n
        axes.append(torch.linspace(lo, hi, n + 1, dtype=dtype)[:-1] + step / 2.0)
    return torch.stack(torch.meshgrid(*axes, indexing="ij"), dim=-1)


def project(coords_xyz, P):
    """coords [..., 3], P [3,4] -> (u_img, v_img, d) with sign-preserving clamp of the divisor."""
    ones = torch.ones_like(coords_xyz[..., :1])
    uvd = torch.einsum("ij,...j->...i", P, torch.cat([coords_xyz, ones], dim=-1))
    d = uvd[..., 2]
    eps = 1e-6
    dc = torch.where(d >= 0, d.clamp(min=eps), d.clamp(max=-eps))
    return uvd[..., 0] / dc, uvd[..., 1] / dc, d


def depth_weight(d, sampled, depth_distribution: int, epsilon: float, depth_range):
    """sampled [D, ...] bilinearly interpolated depth tensor at each sample -> (weight, extra_valid)."""
    if depth_distribution in (0, 1):
        mu, s = sampled[0], sampled[1] + epsilon
        z = (d - mu) / s
        if depth_distribution == 1:
            return 0.5 * torch.exp(-z.abs()) / s, None
        return torch.exp(-0.5 * z * z) / s, None
    if depth_distribution == 2:
        D = sampled.shape[0]
        t = (d - float(depth_range[0])) / float(depth_range[1])
        ok = (t >= 0) & (t <= D - 1)
        tf = torch.floor(t)
        k0 = tf.clamp(0, D - 1).long()
        k1 = (k0 + 1).clamp(max=D - 1)
        r = (t - tf).detach()
        p0 = torch.gather(sampled, 0, k0.unsqueeze(0))[0]
        p1 = torch.gather(sampled, 0, k1.unsqueeze(0))[0]
        return (1 - r) * p0 + r * p1, ok
    raise ValueError(f"depth_distribution must be 0, 1 or 2, got {depth_distribution}")


def dense_pool(feats, depth, proj, image_size, roi_range, grid_size, depth_distribution=0,
               epsilon=1e-6, depth_weight_threshold=1e-6, depth_range=(1.0, 1.0), reduction="mean",
               return_aux=False):
    """Frustum-materialising pooling; differentiable w.r.t. feats and depth.

    feats [B,N,H,W,C], depth [B,N,H,W,D], proj [B,N,3|4,4]  ->  [B,gy,gx,C]
    With return_aux also (counts [B,gy,gx], fov mask bool [B,gy,gx,N,gz]).
    """
    B, N, H, W, C = feats.shape
    dt = feats.dtype
    Hi, Wi = int(image_size[0]), int(image_size[1])
    gx, gy, gz = (int(v) for v in grid_size)
    coords = voxel_centres(roi_range, grid_size, dt).to(feats.device)
    outs, cnts, fovs = [], [], []
    for b in range(B):
        acc = torch.zeros(C, gx, gy, dtype=dt, device=feats.device)
        cnt = torch.zeros(gx, gy, dtype=dt, device=feats.device)
        fov_b = []
        for n in range(N):
            iu, iv, d = project(coords, proj[b, n, :3, :].to(dt))
            fu = iu / Wi * W
            fv = iv / Hi * H
            fov = (fu >= 0) & (fu < W) & (fv >= 0) & (fv < H) & (d > 0)
            grid = torch.stack([fu / (W - 1.0) * 2.0 - 1.0, fv / (H - 1.0) * 2.0 - 1.0], dim=-1)
            grid = grid.reshape(1, gx * gy, gz, 2)
            kw = dict(mode="bilinear", padding_mode="border", align_corners=True)
            f3 = F.grid_sample(feats[b, n].permute(2, 0, 1).unsqueeze(0), grid, **kw)
            d3 = F.grid_sample(depth[b, n].permute(2, 0, 1).unsqueeze(0), grid, **kw)
            f3 = f3.reshape(C, gx, gy, gz)
            d3 = d3.reshape(-1, gx, gy, gz)
            wgt, ok = depth_weight(d, d3, depth_distribution, epsilon, depth_range)
            valid = (wgt >= depth_weight_threshold) & fov
            if ok is not None:
                valid = valid & ok
            f3 = f3 * wgt.unsqueeze(0)
            f3 = f3 * valid.unsqueeze(0)
            acc = acc + f3.sum(dim=-1)
            cnt = cnt + valid.sum(dim=-1)
            fov_b.append(fov)
        if reduction == "mean":
            acc = acc / cnt.clamp(min=1.0).unsqueeze(0)
        outs.append(acc.permute(2, 1, 0))          # [gy, gx, C]
        cnts.append(cnt.transpose(0, 1))
        fovs.append(torch.stack(fov_b, dim=0).permute(2, 1, 0, 3))  # [gy, gx, N, gz]
    out = torch.stack(outs, dim=0)
    if return_aux:
        return out, torch.stack(cnts, dim=0), torch.stack(fovs, dim=0)
    return out


def dense_pool_grads(feats, depth, proj, grad_out, **kw):
    """(out, d_depth, d_feats) via autograd on leaf copies of the inputs."""
    f = feats.detach().clone().requires_grad_(True)
    d = depth.detach().clone().requires_grad_(True)
    out = dense_pool(f, d, proj, **kw)
    out.backward(grad_out)
    return out.detach(), d.grad, f.grad
