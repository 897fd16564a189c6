"""An independent float64 statement of what the rasterizer computes, in dense
torch tensor algebra, used ONLY to pin the CPU oracle (tolerance level).

It shares no code and no formulas-as-typed with oracle/trigrad_oracle.cpp:
barycentrics come from signed areas (not from a precomputed matrix), the
compositing is a cumulative product over per-pixel sorted fragments, and every
gradient comes from torch autograd instead of hand-derived formulas.

Model (reference src/trigrad/wrapper.py:131-141 for the data layout):
  vertices are (x, y, z, w) with w = 1/w_clip; a pixel centre p is inside a
  triangle when its three barycentrics are positive; attributes are
  interpolated perspective-correctly, a = sum(b_i w_i a_i) / sum(b_i w_i);
  the sorting depth is the perspective-correct interpolation of z; the depth
  written to the depth map is sum(b_i / w_i) / sum(b_i) composited with the
  blend weights; opacity is clamped to [0, 0.9999]; fragments are composited
  front to back, C = sum T_k o_k c_k with T_k = prod_{i<k} (1 - o_i); channel 3
  of the image is the final transmittance.
"""
import torch


def pixel_centres(W, H, dtype=torch.float64):
    xs = (torch.arange(W, dtype=dtype) + 0.5) / W * 2 - 1
    ys = (torch.arange(H, dtype=dtype) + 0.5) / H * 2 - 1
    return xs, ys


def fragments(vertices, indices, W, H):
    """Dense per (pixel, triangle) quantities: inside mask and barycentrics, shapes (H, W, M[, 3])."""
    tri = vertices[indices.long()]  # (M, 3, 4)
    xs, ys = pixel_centres(W, H, vertices.dtype)
    px = xs[None, :, None]
    py = ys[:, None, None]
    ax, ay = tri[:, 0, 0], tri[:, 0, 1]
    bx, by = tri[:, 1, 0], tri[:, 1, 1]
    cx, cy = tri[:, 2, 0], tri[:, 2, 1]

    def area(ux, uy, vx, vy, qx, qy):  # twice the signed area of (u, v, q)
        return (vx - ux) * (qy - uy) - (vy - uy) * (qx - ux)

    total = area(ax, ay, bx, by, cx, cy)
    b0 = area(bx, by, cx, cy, px, py) / total
    b1 = area(cx, cy, ax, ay, px, py) / total
    b2 = area(ax, ay, bx, by, px, py) / total
    bary = torch.stack([b0, b1, b2], dim=-1)  # (H, W, M, 3)
    inside = (bary > 0).all(dim=-1) & (total.abs() > 0)
    return tri, bary, inside


def render(vertices, indices, colors, opacities, W, H, order_rank=None, max_layers=None, threshold=None):
    """-> image (H, W, 4), depthmap (H, W).

    order_rank: None -> per-pixel depth order (per_pixel_sort=True);
                (H, W, M) tensor of ranks -> composite in that order (the tile
                list order for per_pixel_sort=False), smaller first.
    max_layers: composite at most this many fragments per pixel.
    threshold : with order_rank given, stop a pixel once its transmittance is
                <= threshold (tested before each fragment).
    """
    tri, bary, inside = fragments(vertices, indices, W, H)
    idx = indices.long()
    w = tri[:, :, 3]                                   # (M, 3)
    bw = bary * w                                      # (H, W, M, 3)
    denom = bw.sum(-1)
    z_sort = (bw * tri[:, :, 2]).sum(-1) / denom
    opac = ((bw * opacities[idx]).sum(-1) / denom).clamp(0.0, 0.9999)
    col = (bw[..., None] * colors[idx]).sum(-2) / denom[..., None]   # (H, W, M, 3)
    z_view = (bary / w).sum(-1) / bary.sum(-1)

    big = torch.finfo(vertices.dtype).max
    if order_rank is None:
        sort_key = torch.where(inside, z_sort.detach(), torch.full_like(z_sort, big))
    else:
        sort_key = torch.where(inside, order_rank.to(vertices.dtype), torch.full_like(z_sort, big))
    perm = torch.argsort(sort_key, dim=-1, stable=True)
    ins = torch.gather(inside, -1, perm)
    o = torch.where(ins, torch.gather(opac, -1, perm), torch.zeros_like(opac))
    c = torch.gather(col, -2, perm[..., None].expand(-1, -1, -1, 3))
    zv = torch.gather(z_view, -1, perm)
    c = torch.where(ins[..., None], c, torch.zeros_like(c))
    zv = torch.where(ins, zv, torch.zeros_like(zv))
    keep = ins.clone()
    if max_layers is not None:
        keep &= torch.cumsum(ins.long(), dim=-1) <= max_layers
    o = torch.where(keep, o, torch.zeros_like(o))
    trans = torch.cumprod(1 - o, dim=-1)
    before = torch.cat([torch.ones_like(trans[..., :1]), trans[..., :-1]], dim=-1)
    if threshold is not None:
        alive = before > threshold
        o = torch.where(alive, o, torch.zeros_like(o))
        trans = torch.cumprod(1 - o, dim=-1)
        before = torch.cat([torch.ones_like(trans[..., :1]), trans[..., :-1]], dim=-1)
    wgt = before * o
    rgb = (wgt[..., None] * c).sum(-2)
    alpha = trans[..., -1] if trans.shape[-1] else torch.ones((H, W), dtype=vertices.dtype)
    wsum = wgt.sum(-1)
    depth = torch.where(wsum > 0, (wgt * zv).sum(-1) / torch.where(wsum > 0, wsum, torch.ones_like(wsum)),
                        torch.full_like(wsum, float("inf")))
    return torch.cat([rgb, alpha[..., None]], dim=-1), depth


def tile_order_rank(sorted_ids, offsets, M, W, H, tw, th):
    """(H, W, M) rank of each triangle in the list of the pixel's tile (M where absent)."""
    import numpy as np
    tiles_x = (W + tw - 1) // tw
    rank = np.full((H, W, M), M, dtype=np.int64)
    for iy in range(H):
        for ix in range(W):
            t = (iy // th) * tiles_x + ix // tw
            ids = sorted_ids[offsets[t]:offsets[t + 1]]
            rank[iy, ix, ids] = np.arange(len(ids))
    return torch.from_numpy(rank)
