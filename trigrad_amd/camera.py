"""The step in front of `render`: camera projection and near-plane splitting.

`render` takes vertices as (x/w, y/w, z/w, 1/w) in NDC (reference
wrapper.py:131-141).  The reference produces them in its viewer
(viewer.py:96-111 projection matrix, viewer.py:271-279 projection of a mesh)
and, for triangles that cross the near plane, in its notebook
(notebooks/renderer.ipynb cell 15, `split_clipped`).  These are the same
operations as differentiable torch functions that run on whatever device the
tensors live on; `split_clipped` is vectorised over triangles instead of the
notebook's Python loop and returns the triangles in the same order with the
same vertex order.
"""
import math

import torch


def perspective(fov_degrees, width, height, near=0.1, far=100.0, dtype=torch.float32, device=None):
    """OpenGL-style projection matrix of the reference camera (viewer.py:96-111): looks down -z, w_clip = -z_eye."""
    t = math.tan(math.radians(fov_degrees) / 2.0) * near
    r = t * width / height
    f, n = far, near
    return torch.tensor([[n / r, 0.0, 0.0, 0.0],
                         [0.0, n / t, 0.0, 0.0],
                         [0.0, 0.0, -(f + n) / (f - n), -(2.0 * f * n) / (f - n)],
                         [0.0, 0.0, -1.0, 0.0]], dtype=dtype, device=device)


def to_clip(positions, matrix):
    """(V,3) positions (or (V,>=3): the first three columns) -> (V,4) clip coordinates matrix @ (x, y, z, 1)."""
    xyz = positions[:, :3]
    ones = torch.ones((xyz.shape[0], 1), dtype=xyz.dtype, device=xyz.device)
    return torch.cat([xyz, ones], dim=-1) @ matrix.to(xyz.dtype).to(xyz.device).T


def clip_to_render(clip_vertices):
    """(V,4) clip coordinates -> (V,4) render input (x/w, y/w, z/w, 1/w) (viewer.py:276-278)."""
    w = clip_vertices[:, 3:4]
    return torch.cat([clip_vertices[:, :3] / w, 1.0 / w], dim=-1)


def project(positions, matrix):
    """Positions through a projection-view matrix to `render`'s vertex layout (viewer.py:271-279)."""
    return clip_to_render(to_clip(positions, matrix))


def split_clipped(clip_vertices, indices, vertex_colors, vertex_opacities):
    """Clips triangles against the plane z + w >= 0 in clip space (notebook cell 15).

    A triangle with all vertices inside is kept, one with none is dropped, one
    with a single vertex inside shrinks to (inside, cut towards the next vertex,
    cut towards the one after), one with two inside becomes the two triangles
    (in1, in2, cut1) and (cut1, in2, cut2), where in1, in2 follow the outside
    vertex in winding order and cut_k lies on the edge from in_k to the outside
    vertex.  Colours and opacities are interpolated with the same parameter
    t = d_in / (d_in - d_out).

    Returns (vertices (3N,4), indices (N,3) int32 = arange, colors (3N,C),
    opacities (3N,...)) as a triangle soup in input order.
    """
    idx = indices.long()
    dev = clip_vertices.device
    d_all = clip_vertices[:, 2] + clip_vertices[:, 3]
    d = d_all[idx]                                   # (M,3)
    inside = d >= 0
    count = inside.sum(dim=1)

    def attributes(vertex_ids):
        return clip_vertices[vertex_ids], vertex_colors[vertex_ids], vertex_opacities[vertex_ids]

    def cut(tri, i_in, i_out):
        """Attributes of the point where edge (corner i_in -> corner i_out) of triangles `tri` meets the plane."""
        rows = torch.arange(tri.shape[0], device=dev)
        a, b = idx[tri][rows, i_in], idx[tri][rows, i_out]
        da, db = d[tri][rows, i_in], d[tri][rows, i_out]
        t = da / (da - db)
        out = []
        for x in (clip_vertices, vertex_colors, vertex_opacities):
            xa, xb = x[a], x[b]
            tt = t.reshape((-1,) + (1,) * (xa.dim() - 1))
            out.append(xa + tt * (xb - xa))
        return out

    pieces = []  # (sort key, corner attribute triples)

    # all inside
    t3 = torch.nonzero(count == 3).flatten()
    if t3.numel():
        corners = [attributes(idx[t3, k]) for k in range(3)]
        pieces.append((t3 * 2, corners))

    # one inside: rotate so that corner `s` is the inside one
    t1 = torch.nonzero(count == 1).flatten()
    if t1.numel():
        s = inside[t1].to(torch.int64).argmax(dim=1)
        o1, o2 = (s + 1) % 3, (s + 2) % 3
        rows = torch.arange(t1.numel(), device=dev)
        corners = [attributes(idx[t1][rows, s]), cut(t1, s, o1), cut(t1, s, o2)]
        pieces.append((t1 * 2, corners))

    # two inside: rotate so that corner `s` is the outside one
    t2 = torch.nonzero(count == 2).flatten()
    if t2.numel():
        s = (~inside[t2]).to(torch.int64).argmax(dim=1)
        i1, i2 = (s + 1) % 3, (s + 2) % 3
        rows = torch.arange(t2.numel(), device=dev)
        in1, in2 = attributes(idx[t2][rows, i1]), attributes(idx[t2][rows, i2])
        c1, c2 = cut(t2, i1, s), cut(t2, i2, s)
        pieces.append((t2 * 2, [in1, in2, c1]))
        pieces.append((t2 * 2 + 1, [c1, in2, c2]))

    if not pieces:
        return (clip_vertices.new_empty((0, 4)), torch.empty((0, 3), dtype=torch.int32, device=dev),
                vertex_colors.new_empty((0,) + tuple(vertex_colors.shape[1:])),
                vertex_opacities.new_empty((0,) + tuple(vertex_opacities.shape[1:])))

    order = torch.argsort(torch.cat([k for k, _ in pieces]), stable=True)
    out = []
    for a in range(3):  # attribute: position, colour, opacity
        per_corner = [torch.cat([corners[c][a] for _, corners in pieces], dim=0)[order] for c in range(3)]
        stacked = torch.stack(per_corner, dim=1)            # (N,3,...)
        out.append(stacked.reshape((-1,) + tuple(stacked.shape[2:])))
    n = out[0].shape[0] // 3
    new_indices = torch.arange(3 * n, dtype=torch.int32, device=dev).reshape(n, 3)
    return out[0], new_indices, out[1], out[2]
