"""Camera projection and near-plane splitting (trigrad_amd.camera) against the
reference's Python statements of the same steps: viewer.py:96-111 (matrix),
viewer.py:271-279 (projection), notebooks/renderer.ipynb cell 15 (split_clipped).

The splitting is checked against a per-triangle loop written from the notebook's
description, and against what geometry fixes: every output vertex is on the
kept side, cut points lie on the plane, the kept area is the similar-triangle
fraction of the original, the winding is preserved.
"""
import math

import numpy as np
import pytest
import torch

from trigrad_amd import camera


def test_perspective_matrix_maps_the_frustum_to_the_cube():
    W, H, near, far, fov = 640, 480, 0.5, 20.0, 40.0
    P = camera.perspective(fov, W, H, near, far, dtype=torch.float64)
    t = math.tan(math.radians(fov) / 2) * near
    r = t * W / H
    corners = torch.tensor([[r, t, -near], [-r, -t, -near], [0.0, 0.0, -far], [r * far / near, t * far / near, -far]], dtype=torch.float64)
    out = camera.project(corners, P)
    np.testing.assert_allclose(out[0, :3].numpy(), [1, 1, -1], atol=1e-12)
    np.testing.assert_allclose(out[1, :3].numpy(), [-1, -1, -1], atol=1e-12)
    np.testing.assert_allclose(out[2, :3].numpy(), [0, 0, 1], atol=1e-12)
    np.testing.assert_allclose(out[3, :3].numpy(), [1, 1, 1], atol=1e-12)
    # fourth component is 1 / w_clip = 1 / distance along the view axis
    np.testing.assert_allclose(out[:, 3].numpy(), [1 / near, 1 / near, 1 / far, 1 / far], atol=1e-12)


def test_project_is_matrix_product_then_division():
    g = torch.Generator().manual_seed(0)
    pos = torch.randn((50, 3), generator=g, dtype=torch.float64)
    pos[:, 2] -= 5.0
    M = torch.randn((4, 4), generator=g, dtype=torch.float64)
    got = camera.project(pos, M)
    h = np.concatenate([pos.numpy(), np.ones((50, 1))], axis=1) @ M.numpy().T
    want = np.concatenate([h[:, :3] / h[:, 3:4], 1.0 / h[:, 3:4]], axis=1)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-12, atol=1e-12)
    # extra vertex columns are ignored, as the viewer passes (V,>=3) meshes
    got2 = camera.project(torch.cat([pos, torch.zeros((50, 2), dtype=torch.float64)], dim=1), M)
    np.testing.assert_array_equal(got.numpy(), got2.numpy())


def _split_loop(cv, idx, col, op):
    """Triangle-by-triangle statement of the notebook's rule."""
    V, C, O = [], [], []

    def mix(a, b, t):
        return cv[a] + t * (cv[b] - cv[a]), col[a] + t * (col[b] - col[a]), op[a] + t * (op[b] - op[a])

    for tri in idx:
        ids = [int(x) for x in tri]
        d = [float(cv[i, 2] + cv[i, 3]) for i in ids]
        ins = [x >= 0 for x in d]
        k = sum(ins)
        if k == 3:
            tris = [[(cv[i], col[i], op[i]) for i in ids]]
        elif k == 0:
            tris = []
        elif k == 1:
            s = ins.index(True)
            a, b, c = ids[s], ids[(s + 1) % 3], ids[(s + 2) % 3]
            da, db, dc = d[s], d[(s + 1) % 3], d[(s + 2) % 3]
            tris = [[(cv[a], col[a], op[a]), mix(a, b, da / (da - db)), mix(a, c, da / (da - dc))]]
        else:
            s = ins.index(False)
            o, a, b = ids[s], ids[(s + 1) % 3], ids[(s + 2) % 3]
            do, da, db = d[s], d[(s + 1) % 3], d[(s + 2) % 3]
            n1, n2 = mix(a, o, da / (da - do)), mix(b, o, db / (db - do))
            A, B = (cv[a], col[a], op[a]), (cv[b], col[b], op[b])
            tris = [[A, B, n1], [n1, B, n2]]
        for t3 in tris:
            for v, c, o_ in t3:
                V.append(v); C.append(c); O.append(o_)
    return np.array(V).reshape(-1, 4), np.array(C).reshape(-1, col.shape[1]), np.array(O).reshape(-1)


def _mesh(seed, n_vertices=60, n_triangles=150):
    rng = np.random.default_rng(seed)
    cv = rng.normal(size=(n_vertices, 4))
    cv[:, 3] = np.abs(cv[:, 3]) + 0.2
    cv[:, 2] = rng.normal(scale=1.5, size=n_vertices)     # z + w changes sign for many vertices
    idx = rng.integers(0, n_vertices, size=(n_triangles, 3)).astype(np.int32)
    col = rng.uniform(size=(n_vertices, 3))
    op = rng.uniform(size=n_vertices)
    return cv, idx, col, op


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_split_clipped_matches_triangle_loop(seed):
    cv, idx, col, op = _mesh(seed)
    d = cv[idx][:, :, 2] + cv[idx][:, :, 3]
    counts = (d >= 0).sum(axis=1)
    assert set(counts.tolist()) == {0, 1, 2, 3}            # the mesh exercises every case
    v, i, c, o = camera.split_clipped(torch.from_numpy(cv), torch.from_numpy(idx), torch.from_numpy(col), torch.from_numpy(op))
    wv, wc, wo = _split_loop(cv, idx, col, op)
    n = int((counts == 3).sum() + (counts == 1).sum() + 2 * (counts == 2).sum())
    assert v.shape == (3 * n, 4) and i.dtype == torch.int32
    np.testing.assert_array_equal(i.numpy(), np.arange(3 * n).reshape(n, 3))
    np.testing.assert_allclose(v.numpy(), wv, rtol=0, atol=1e-14)
    np.testing.assert_allclose(c.numpy(), wc, rtol=0, atol=1e-14)
    np.testing.assert_allclose(o.numpy(), wo, rtol=0, atol=1e-14)


def test_split_clipped_geometry():
    cv, idx, col, op = _mesh(5, 40, 200)
    v, i, c, o = camera.split_clipped(torch.from_numpy(cv), torch.from_numpy(idx), torch.from_numpy(col), torch.from_numpy(op))
    v = v.numpy()
    dist = v[:, 2] + v[:, 3]
    assert (dist >= -1e-12).all()                          # nothing left behind the plane
    # area and winding in the (x, y, z+w) chart of the triangle's plane
    def normals(p):
        q = np.stack([p[:, :, 0], p[:, :, 1], p[:, :, 2] + p[:, :, 3]], axis=-1)
        return np.cross(q[:, 1] - q[:, 0], q[:, 2] - q[:, 0])
    src = cv[idx]
    d = src[:, :, 2] + src[:, :, 3]
    inside = d >= 0
    count = inside.sum(axis=1)
    n_src = normals(src)
    # expected kept fraction of each triangle's area from similar triangles
    frac = np.zeros(len(idx))
    for t in range(len(idx)):
        if count[t] == 3:
            frac[t] = 1.0
        elif count[t] == 1:
            s = int(np.argmax(inside[t])); a, b = (s + 1) % 3, (s + 2) % 3
            frac[t] = d[t, s] / (d[t, s] - d[t, a]) * d[t, s] / (d[t, s] - d[t, b])
        elif count[t] == 2:
            s = int(np.argmin(inside[t])); a, b = (s + 1) % 3, (s + 2) % 3
            frac[t] = 1.0 - d[t, s] / (d[t, s] - d[t, a]) * d[t, s] / (d[t, s] - d[t, b])
    out_per_tri = np.where(count == 2, 2, np.where(count == 0, 0, 1))
    owner = np.repeat(np.arange(len(idx)), out_per_tri)
    n_out = normals(v.reshape(-1, 3, 4))
    # same orientation as the source triangle, and the areas add up to the kept fraction
    assert (np.einsum("ij,ij->i", n_out, n_src[owner]) >= -1e-12).all()
    area_out = np.zeros(len(idx))
    np.add.at(area_out, owner, np.linalg.norm(n_out, axis=1))
    np.testing.assert_allclose(area_out, frac * np.linalg.norm(n_src, axis=1), rtol=1e-9, atol=1e-12)


def test_split_clipped_empty_and_gradients():
    cv = torch.tensor([[0.0, 0, -2, 1], [1, 0, -2, 1], [0, 1, -2, 1]])
    out = camera.split_clipped(cv, torch.tensor([[0, 1, 2]], dtype=torch.int32), torch.rand(3, 3), torch.rand(3))
    assert out[0].shape == (0, 4) and out[1].shape == (0, 3) and out[2].shape == (0, 3) and out[3].shape == (0,)
    cv, idx, col, op = _mesh(7, 20, 30)
    colors = torch.from_numpy(col).requires_grad_(True)
    clip = torch.from_numpy(cv).requires_grad_(True)
    v, i, c, o = camera.split_clipped(clip, torch.from_numpy(idx), colors, torch.from_numpy(op))
    (c.sum() + v.sum()).backward()
    assert torch.isfinite(colors.grad).all() and torch.isfinite(clip.grad).all() and float(colors.grad.abs().sum()) > 0


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_split_clipped_on_the_device_matches_triangle_loop(seed, cuda):
    """The same comparison with the tensors on the GPU: split_clipped's stable argsort, nonzero and gathers run as
    device kernels there (notebooks/renderer.ipynb cell 15 runs it on cuda tensors too)."""
    cv, idx, col, op = _mesh(seed)
    counts = ((cv[idx][:, :, 2] + cv[idx][:, :, 3]) >= 0).sum(axis=1)
    assert set(counts.tolist()) == {0, 1, 2, 3}
    v, i, c, o = camera.split_clipped(*(torch.from_numpy(a).to(cuda) for a in (cv, idx, col, op)))
    assert v.device.type == "cuda" and i.device.type == "cuda" and i.dtype == torch.int32
    wv, wc, wo = _split_loop(cv, idx, col, op)
    n = int((counts == 3).sum() + (counts == 1).sum() + 2 * (counts == 2).sum())
    np.testing.assert_array_equal(i.cpu().numpy(), np.arange(3 * n).reshape(n, 3))
    np.testing.assert_allclose(v.cpu().numpy(), wv, rtol=0, atol=1e-14)
    np.testing.assert_allclose(c.cpu().numpy(), wc, rtol=0, atol=1e-14)
    np.testing.assert_allclose(o.cpu().numpy(), wo, rtol=0, atol=1e-14)
    # and in the renderer's precision, against the float64 loop
    v32, i32, c32, o32 = camera.split_clipped(*(torch.from_numpy(a.astype(np.float32) if a.dtype == np.float64 else a).to(cuda)
                                                for a in (cv, idx, col, op)))
    assert v32.dtype == torch.float32 and v32.shape == (3 * n, 4)
    np.testing.assert_allclose(v32.cpu().numpy(), wv, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(c32.cpu().numpy(), wc, rtol=2e-5, atol=2e-5)


@pytest.mark.gpu
def test_projected_split_mesh_renders(cuda):
    """A mesh reaching behind the camera renders to finite values after splitting, and
    splitting a mesh that lies wholly in front changes nothing in the image."""
    import trigrad_amd
    import scenes as S
    W, H = 96, 64
    g = torch.Generator().manual_seed(3)
    pos = torch.randn((90, 3), generator=g) * torch.tensor([1.5, 1.0, 2.5])
    idx = torch.arange(90, dtype=torch.int32).reshape(30, 3)
    col, op = torch.rand((90, 3), generator=g), torch.rand(90, generator=g) * 0.7 + 0.2
    P = camera.perspective(50.0, W, H, 0.1, 50.0)
    for shift, crosses in ((-1.0, True), (-12.0, False)):
        p = pos.clone(); p[:, 2] += shift
        clip = camera.to_clip(p.to(cuda), P.to(cuda))
        v, i, c, o = camera.split_clipped(clip, idx.to(cuda), col.to(cuda), op.to(cuda))
        d_src = (clip[:, 2] + clip[:, 3])[idx.long().to(cuda)]
        assert bool(((d_src < 0).any(dim=1) & (d_src >= 0).any(dim=1)).any()) == crosses
        img, depth = trigrad_amd.render(camera.clip_to_render(v).contiguous(), i, c.contiguous(), o.contiguous(), W, H)
        assert torch.isfinite(img).all()
        if not crosses:
            img0, depth0 = trigrad_amd.render(camera.clip_to_render(clip).contiguous(), idx.to(cuda), col.to(cuda), op.to(cuda), W, H)
            assert torch.equal(img, img0) and torch.equal(depth, depth0)
