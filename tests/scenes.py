"""Seeded synthetic scenes: the five benchmark configurations and the fixture
scenes of the reference's test-suite, as plain numpy data.

A scene is a dict with
    vertices (V,4) float32  (x/w, y/w, z/w, 1/w) in NDC, the layout
                            reference src/trigrad/wrapper.py:131-141 documents
    indices  (M,3) int32
    colors   (V,3) float32
    opacities (V,) float32
    width, height           image size
    target   (H,W,4) float32 (benchmark configurations only)

The fixture scenes restate the geometry of reference tests/testcases.py (cited
per function); where the reference draws colours from an unseeded torch RNG
they are drawn here from a seeded numpy generator instead.
"""
import math

import numpy as np

F = np.float32


def add_w(xyz):
    """Append w = 1/z as the fourth component (reference tests/testcases.py:5-9)."""
    xyz = np.asarray(xyz, dtype=F)
    with np.errstate(divide="ignore"):
        w = (F(1) / xyz[:, 2:3]).astype(F)
    return np.concatenate([xyz, w], axis=1).astype(F)


def _scene(vertices, indices, colors, opacities, width, height, **extra):
    d = dict(vertices=np.ascontiguousarray(vertices, F), indices=np.ascontiguousarray(indices, np.int32),
             colors=np.ascontiguousarray(colors, F), opacities=np.ascontiguousarray(opacities, F),
             width=int(width), height=int(height))
    d.update(extra)
    return d


# ---- benchmark configurations ---------------------------------------------------

CONFIG_SIZES = {
    0: dict(M=1_000, W=256, H=256),
    1: dict(M=100_000, W=1024, H=1024),
    2: dict(M=1_000_000, W=1920, H=1080),
    3: dict(M=200_000, W=512, H=512),
    4: dict(level=8, W=1920, H=1080),
}


def triangle_soup(cfg, M=None, with_target=True):
    """Configurations 0-3: M independent triangles (V = 3M).

    One numpy Generator seeded with the configuration index; draw order:
    centroids, [edge scale, config 2], vertex offsets, depth, colours,
    opacities, target.  Vertex xy = centroid + N(0, sigma); sigma is 0.05 NDC
    for config 0 and given in pixels otherwise (converted per axis by 2/W and
    2/H).  The mean edge of this generator is sigma*sqrt(pi).  Depth d is per
    triangle, z = d and w = 1/d on all three vertices.
    """
    assert cfg in (0, 1, 2, 3)
    size = CONFIG_SIZES[cfg]
    W, H = size["W"], size["H"]
    M = size["M"] if M is None else int(M)
    rng = np.random.default_rng(cfg)
    cen = rng.uniform(-1.0, 1.0, size=(M, 1, 2))
    if cfg == 0:
        sig = np.full((M, 1, 2), 0.05)
    else:
        if cfg == 1:
            s_px = np.full((M,), 8.0)
        elif cfg == 2:
            s_px = rng.lognormal(mean=math.log(4.0), sigma=1.0, size=M)
        else:
            s_px = np.full((M,), 60.0)
        sig_px = s_px / math.sqrt(math.pi)
        sig = np.stack([sig_px * 2.0 / W, sig_px * 2.0 / H], axis=-1)[:, None, :]
    xy = cen + rng.standard_normal(size=(M, 3, 2)) * sig
    d = rng.uniform(0.1, 10.0, size=(M, 1))
    z = np.broadcast_to(d, (M, 3))
    verts = np.concatenate([xy, z[..., None], (1.0 / z)[..., None]], axis=-1).reshape(3 * M, 4)
    colors = rng.uniform(0.0, 1.0, size=(3 * M, 3))
    lo, hi = (0.02, 0.15) if cfg == 3 else (0.2, 0.95)
    opac = rng.uniform(lo, hi, size=(3 * M,))
    extra = {}
    if with_target:
        extra["target"] = rng.uniform(0.0, 1.0, size=(H, W, 4)).astype(F)
    idx = np.arange(3 * M, dtype=np.int32).reshape(M, 3)
    return _scene(verts, idx, colors, opac, W, H, name=f"config{cfg}", **extra)


def icosphere(level):
    """Unit icosphere: 20*4^level faces, 10*4^level+2 shared vertices (float64)."""
    t = (1.0 + math.sqrt(5.0)) / 2.0
    v = np.array([[-1, t, 0], [1, t, 0], [-1, -t, 0], [1, -t, 0], [0, -1, t], [0, 1, t], [0, -1, -t], [0, 1, -t],
                  [t, 0, -1], [t, 0, 1], [-t, 0, -1], [-t, 0, 1]], dtype=np.float64)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    f = np.array([[0, 11, 5], [0, 5, 1], [0, 1, 7], [0, 7, 10], [0, 10, 11], [1, 5, 9], [5, 11, 4], [11, 10, 2],
                  [10, 7, 6], [7, 1, 8], [3, 9, 4], [3, 4, 2], [3, 2, 6], [3, 6, 8], [3, 8, 9], [4, 9, 5], [2, 4, 11],
                  [6, 2, 10], [8, 6, 7], [9, 8, 1]], dtype=np.int64)
    for _ in range(level):
        e = np.concatenate([f[:, [0, 1]], f[:, [1, 2]], f[:, [2, 0]]], axis=0)
        e.sort(axis=1)
        code = e[:, 0] * (v.shape[0] + 1) + e[:, 1]
        uniq, inv = np.unique(code, return_inverse=True)
        a, b = uniq // (v.shape[0] + 1), uniq % (v.shape[0] + 1)
        mid = v[a] + v[b]
        mid /= np.linalg.norm(mid, axis=1, keepdims=True)
        n0 = v.shape[0]
        v = np.concatenate([v, mid], axis=0)
        nf = f.shape[0]
        m01, m12, m20 = n0 + inv[:nf], n0 + inv[nf:2 * nf], n0 + inv[2 * nf:]
        f = np.concatenate([np.stack([f[:, 0], m01, m20], 1), np.stack([f[:, 1], m12, m01], 1),
                            np.stack([f[:, 2], m20, m12], 1), np.stack([m01, m12, m20], 1)], axis=0)
    return v, f


def perspective(fov_deg, aspect, near, far):
    """OpenGL-style projection matrix (the convention of reference viewer.py:96-111)."""
    t = math.tan(math.radians(fov_deg) / 2) * near
    r = t * aspect
    return np.array([[near / r, 0, 0, 0], [0, near / t, 0, 0],
                     [0, 0, -(far + near) / (far - near), -(2 * far * near) / (far - near)], [0, 0, -1, 0]], dtype=np.float64)


def project(points, PV):
    """World points (N,3) -> (x/w, y/w, z/w, 1/w) (reference viewer.py:271-279)."""
    h = np.concatenate([points, np.ones((points.shape[0], 1))], axis=1) @ PV.T
    return np.concatenate([h[:, :3] / h[:, 3:4], 1.0 / h[:, 3:4]], axis=1)


def icosphere_scene(level=None, with_target=True):
    """Configuration 4: shared-vertex icosphere, jitter N(0,1e-3), seeded random
    rotation, perspective camera (fov 30 deg) at the distance where the sphere
    spans about 1000 px of a 1920x1080 frame."""
    size = CONFIG_SIZES[4]
    W, H = size["W"], size["H"]
    level = size["level"] if level is None else level
    rng = np.random.default_rng(4)
    v, f = icosphere(level)
    q = rng.standard_normal(4)
    q /= np.linalg.norm(q)
    a, b, c, d = q
    R = np.array([[a * a + b * b - c * c - d * d, 2 * (b * c - a * d), 2 * (b * d + a * c)],
                  [2 * (b * c + a * d), a * a - b * b + c * c - d * d, 2 * (c * d - a * b)],
                  [2 * (b * d - a * c), 2 * (c * d + a * b), a * a - b * b - c * c + d * d]])
    v = (v + rng.standard_normal(v.shape) * 1e-3) @ R.T
    view = np.eye(4)
    view[2, 3] = -4.15
    PV = perspective(30.0, W / H, 0.1, 100.0) @ view
    verts = project(v, PV)
    colors = rng.uniform(0.0, 1.0, size=(v.shape[0], 3))
    opac = np.full((v.shape[0],), 0.9)
    extra = {}
    if with_target:
        extra["target"] = rng.uniform(0.0, 1.0, size=(H, W, 4)).astype(F)
    return _scene(verts, f.astype(np.int32), colors, opac, W, H, name="config4", **extra)


def config(cfg, with_target=True, **kw):
    if cfg == 4:
        return icosphere_scene(with_target=with_target, **kw)
    return triangle_soup(cfg, with_target=with_target, **kw)


def sort_keys(K, T, seed=0):
    """Synthetic input of the standalone sort benchmark: tile uniform in [0,T),
    depth bits of U[0.1,10] floats, payload = index."""
    rng = np.random.default_rng(seed)
    tile = rng.integers(0, T, size=K, dtype=np.uint64)
    depth = rng.uniform(0.1, 10.0, size=K).astype(F).view(np.uint32).astype(np.uint64)
    keys = (tile << np.uint64(32)) | (depth ^ np.uint64(0x80000000))
    return keys, np.arange(K, dtype=np.int32)


# ---- fixture scenes of the reference's tests ---------------------------------------

def overlapping_squares(n, mins=0.1, maxs=0.9, seed=0, width=50, height=50):
    """n nested axis-aligned squares, square i at z = 2(i+1), one colour per
    square (reference tests/testcases.py:12-36)."""
    rng = np.random.default_rng(seed)
    half = np.linspace(mins, maxs, n, dtype=F) / F(2)
    f = F(1.00001)
    sx = np.array([-1, 1, 1, -1], dtype=F)
    sy = np.array([-1, -1, 1, 1], dtype=F)
    xyz = np.empty((n, 4, 3), dtype=F)
    xyz[:, :, 0] = (f * half)[:, None] * sx
    xyz[:, :, 1] = half[:, None] * sy
    xyz[:, :, 2] = np.arange(1, n + 1, dtype=F)[:, None]
    xyz = xyz.reshape(4 * n, 3) * F(2)
    base = 4 * np.arange(n, dtype=np.int32)[:, None]
    idx = np.concatenate([base + np.array([0, 1, 2], np.int32), base + np.array([0, 2, 3], np.int32)], axis=1).reshape(2 * n, 3)
    colors = np.repeat(rng.uniform(0, 1, size=(n, 3)), 4, axis=0)
    return _scene(add_w(xyz), idx, colors, np.full(4 * n, 0.99, F), width, height, name="overlapping_squares")


def large_triangles(n, r=0.5, unicolor=False, seed=0, width=50, height=50):
    """n equilateral triangles of circumradius r centred at (0.5,0.5), random
    rotation, triangle i at z = i+1 (reference tests/testcases.py:73-102)."""
    rng = np.random.default_rng(seed)
    ang = rng.uniform(0, 2 * math.pi, size=n)[:, None] + np.array([0, 2 * math.pi / 3, 4 * math.pi / 3])[None, :]
    xyz = np.stack([np.cos(ang) * r + 0.5, np.sin(ang) * r + 0.5, np.broadcast_to(np.arange(1, n + 1)[:, None], (n, 3))], axis=-1)
    colors = rng.uniform(0, 1, size=(n, 3, 3))
    if unicolor:
        colors[:, 1:] = colors[:, :1]
    idx = np.arange(3 * n, dtype=np.int32).reshape(n, 3)
    return _scene(add_w(xyz.reshape(3 * n, 3)), idx, colors.reshape(3 * n, 3), np.full(3 * n, 0.99, F), width, height,
                  name="large_triangles")


def depth_overlap(width=64, height=64):
    """Two interpenetrating triangles, z from 2 to 3 (reference tests/testcases.py:39-70)."""
    xyz = np.array([[-1, -1, 3], [1, -1, 3], [0, 1, 2], [-1, 1, 3], [1, 1, 3], [0, -1, 2]], dtype=F)
    colors = np.array([[1, 0, 0]] * 3 + [[0, 0, 1]] * 3, dtype=F)
    return _scene(add_w(xyz), [[0, 1, 2], [3, 4, 5]], colors, np.ones(6, F), width, height, name="depth_overlap")


def overlapping_triangles(width=64, height=64):
    """Two facing triangles at z = 1 and z = 2 (reference tests/testcases.py:105-135)."""
    xy = np.array([[0.1, 0.1], [0.1, 0.9], [0.75, 0.5], [0.9, 0.1], [0.9, 0.9], [0.25, 0.5]], dtype=F) * F(2) - F(1)
    xyz = np.concatenate([xy, np.array([[1], [1], [1], [2], [2], [2]], dtype=F)], axis=1)
    colors = np.array([[1, 0, 0]] * 3 + [[0, 0, 1]] * 3, dtype=F)
    return _scene(add_w(xyz), [[0, 1, 2], [3, 4, 5]], colors, np.full(6, 0.5, F), width, height, name="overlapping_triangles")


def unit_square(width=64, height=64):
    """Two triangles forming a square; the *2-1 applies to z as well, so z = -1
    and w = -1 (reference tests/testcases.py:138-165)."""
    xyz = np.array([[0.1, 0.1, 0], [0.1, 0.9, 0], [0.9, 0.1, 0], [0.9, 0.9, 0]], dtype=F) * F(2) - F(1)
    colors = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]], dtype=F)
    return _scene(add_w(xyz), [[0, 1, 2], [1, 2, 3]], colors, np.full(4, 0.8, F), width, height, name="unit_square")


def grid_mesh(nx, ny, minx=-1.0, maxx=1.0, miny=-1.0, maxy=1.0, seed=0, width=500, height=500):
    """Staggered triangle grid at z = 1: even rows hold nx vertices, odd rows nx-1
    vertices shifted by half a step (reference tests/testcases.py:168-193)."""
    rng = np.random.default_rng(seed)
    step = (maxx - minx) / (nx - 1)
    verts, tris = [], []
    for iy in range(ny):
        y = miny + iy * (maxy - miny) / (ny - 1)
        odd = iy % 2 == 1
        count = nx - 1 if odd else nx
        first = len(verts)
        for ix in range(count):
            verts.append((minx + (step / 2 if odd else 0.0) + ix * step, y, 1.0))
        if iy == ny - 1:
            continue
        n = first + np.arange(count)
        ix = np.arange(count)
        right = (ix < nx - 2) | ((ix < nx - 1) & (not odd))
        centre = np.full(count, odd) | ((ix > 0) & (ix < nx - 1))
        for k in range(count):  # per vertex: right triangle first, then centre triangle
            if right[k]:
                tris.append((n[k], n[k] + 1, n[k] + nx))
            if centre[k]:
                tris.append((n[k], n[k] + nx, n[k] + nx - 1))
    verts = np.array(verts, dtype=F)
    colors = rng.uniform(0, 1, size=(verts.shape[0], 3))
    return _scene(add_w(verts), np.array(tris, dtype=np.int32), colors, np.ones(verts.shape[0], F), width, height, name="grid_mesh")


def overlap_mesh(seed=0, width=64, height=64):
    """Ten triangles at z = 0, hence w = +inf (reference tests/testcases.py:196-230)."""
    rng = np.random.default_rng(seed)
    xyz = np.array([[-0.5, 0, 0], [0.5, 0, 0], [-0.2, 1.2, 0], [0.0, 0.3, 0], [-0.5, 1, 0], [0.5, 1, 0], [0, 1.5, 0],
                    [0, -0.5, 0], [1, -0.5, 0]], dtype=F)
    idx = [[0, 3, 2], [1, 2, 3], [0, 1, 3], [0, 2, 4], [1, 5, 2], [5, 6, 2], [4, 2, 6], [7, 1, 0], [8, 1, 7], [8, 5, 1]]
    return _scene(add_w(xyz), idx, rng.uniform(0, 1, size=(9, 3)), np.full(9, 0.7, F), width, height, name="overlap_mesh")


def random_soup(M, W, H, seed=0, sigma_px=6.0, opacity=(0.2, 0.95), zrange=(0.1, 10.0), varying_w=False, shared=False):
    """Small general-purpose scene for parity tests: like triangle_soup, with
    optional per-vertex depth (three different w per triangle) and optional
    vertex sharing (indices drawn at random from a smaller vertex pool)."""
    rng = np.random.default_rng(seed)
    cen = rng.uniform(-1.05, 1.05, size=(M, 1, 2))
    sig = np.array([sigma_px * 2.0 / W, sigma_px * 2.0 / H])
    xy = cen + rng.standard_normal(size=(M, 3, 2)) * sig
    if varying_w:
        z = rng.uniform(*zrange, size=(M, 3))
    else:
        z = np.broadcast_to(rng.uniform(*zrange, size=(M, 1)), (M, 3))
    verts = np.concatenate([xy, z[..., None], (1.0 / z)[..., None]], axis=-1).reshape(3 * M, 4)
    idx = np.arange(3 * M, dtype=np.int32).reshape(M, 3)
    if shared:
        pool = max(3, M // 2)
        pxy = rng.uniform(-1.0, 1.0, size=(pool, 2))
        pz = rng.uniform(*zrange, size=(pool, 1))
        verts = np.concatenate([pxy, pz, 1.0 / pz], axis=1)
        near = np.argsort(((pxy[:, None, :] - pxy[None, :, :]) ** 2).sum(-1), axis=1)[:, :6]
        a = rng.integers(0, pool, size=M)
        pick = np.stack([rng.permutation(5)[:2] + 1 for _ in range(M)])
        idx = np.stack([a, near[a, pick[:, 0]], near[a, pick[:, 1]]], axis=1).astype(np.int32)
    V = verts.shape[0]
    colors = rng.uniform(0, 1, size=(V, 3))
    opac = rng.uniform(*opacity, size=(V,))
    target = rng.uniform(0, 1, size=(H, W, 4)).astype(F)
    return _scene(verts, idx, colors, opac, W, H, target=target, name="random_soup")
