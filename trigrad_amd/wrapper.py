"""Public entry point: `render` and its autograd Function, with the signatures,
defaults, checks and return values of reference src/trigrad/wrapper.py:12-158."""
from typing import Tuple

import torch
from torch.autograd import Function

from . import _C
from .util import create_check

check_tensor = create_check("cuda", lambda: _C.precision)
precision = _C.precision  # the scalar type at import (TRIGRAD_PRECISION); _C.set_precision changes what the checks expect


class Renderer(Function):
    @staticmethod
    def forward(
        ctx,
        vertices: torch.Tensor,
        indices: torch.Tensor,
        colors: torch.Tensor,
        opacities: torch.Tensor,
        width: int = 500,
        height: int = 500,
        tile_width: int = 16,
        tile_height: int = 16,
        early_stopping_threshold: float = 1 / 256,
        record_timing: bool = False,
        per_pixel_sort: bool = True,
        max_layers: int = 32,
    ):
        n_vertices, _ = vertices.shape
        check_tensor(vertices, "vertices", (n_vertices, 4))
        check_tensor(colors, "colors", (n_vertices, 3))
        check_tensor(opacities, "opacities", (n_vertices,))
        n_triangles, _ = indices.shape
        check_tensor(indices, "indices", (n_triangles, 3), torch.int32)
        if max_layers <= 0:
            max_layers = n_triangles + 1  # wrapper.py:35-36: "no limit"

        ctx.render_args = (width, height, tile_width, tile_height, early_stopping_threshold, per_pixel_sort, max_layers)
        ctx.set_materialize_grads(False)  # an output the loss does not use arrives as None instead of a zero tensor
        if n_triangles < 1:
            # wrapper.py:46-53: nothing to draw -- transparent black, infinitely far
            ctx.skipped = True
            image = torch.zeros((height, width, 4), dtype=colors.dtype, device=colors.device)
            image[..., 3] = 1.0
            depthmap = torch.full((height, width), float("inf"), dtype=colors.dtype, device=colors.device)
            timings = None
            ctx.save_for_backward(vertices, indices, colors, opacities)
        else:
            ctx.skipped = False
            (image, depthmap, final_weights, sorted_ids, offsets, bary_transforms, ends, timings, resume) = _C._forward_full(
                vertices, indices, colors, opacities, width, height, tile_width, tile_height, early_stopping_threshold,
                not record_timing, per_pixel_sort, max_layers)
            last, last_depth, status_check, fragments, hit_masks = resume
            # private to this Function: where the reverse traversal starts, and the blend order (per-pixel
            # order, max_layers <= 32) or the hit masks (tile order); the list kernels' status word, which the
            # backward pass looks at before it trusts the lists
            extras = [t for t in (last_depth, fragments, hit_masks) if t is not None]
            ctx.has_last_depth = last_depth is not None
            ctx.has_fragments = fragments is not None
            ctx.has_hit_masks = hit_masks is not None
            ctx.status_check = status_check
            saved = [vertices, indices, colors, opacities, sorted_ids, offsets, bary_transforms, image, depthmap, final_weights,
                     ends, last]
            ctx.save_for_backward(*saved, *extras)
        if record_timing:
            return image, depthmap, timings
        return image, depthmap

    @staticmethod
    def backward(ctx, grad_image, grad_depthmap, grad_timings=None):
        if ctx.skipped:
            grad_vertices = torch.zeros_like(ctx.saved_tensors[0])
            grad_colors = torch.zeros_like(ctx.saved_tensors[2])
            grad_opacities = torch.zeros_like(ctx.saved_tensors[3])
        else:
            saved = ctx.saved_tensors
            last = saved[11]
            extras = list(saved[12:])
            last_depth = extras.pop(0) if ctx.has_last_depth else None
            fragments = extras.pop(0) if ctx.has_fragments else None
            hit_masks = extras.pop(0) if ctx.has_hit_masks else None
            width, height, tile_width, tile_height, threshold, per_pixel_sort, max_layers = ctx.render_args
            if grad_image is None:
                grad_image = torch.zeros_like(saved[7])
            grad_vertices, grad_colors, grad_opacities = _C.render_backward(
                grad_image, grad_depthmap, *saved[:11], width, height, tile_width, tile_height, threshold, per_pixel_sort,
                max_layers, resume=(last, last_depth, ctx.status_check, fragments, hit_masks))
        # one slot per forward argument (wrapper.py:99-112)
        return (grad_vertices, None, grad_colors, grad_opacities, None, None, None, None, None, None, None, None)


def render(
    vertices: torch.Tensor,
    indices: torch.Tensor,
    colors: torch.Tensor,
    opacities: torch.Tensor,
    width: int = 500,
    height: int = 500,
    tile_width: int = 16,
    tile_height: int = 16,
    early_stopping_threshold: float = 1 / 256,
    record_timing: bool = False,
    per_pixel_sort: bool = True,
    max_layers: int = 32,
) -> Tuple[torch.Tensor, ...]:
    """
    Render semi-transparent triangles with the tile rasterizer.
        vertices : (N, 4) vertices (x'/w', y'/w', z'/w', 1/w') in [-1,1] clip space
        indices : (M, 3) int32 vertex indices of the triangles
        colors : (N, 3) vertex colours
        opacities : (N,) vertex opacities
        per_pixel_sort : order fragments per pixel (True) or per tile (False)
        max_layers : maximum number of fragments composited per pixel, <= 0 for no limit

    Returns:
        image : (height, width, 4); channel 3 holds the remaining transmittance, not opacity
        depthmap : (height, width)
        timings (only if record_timing) : dict of seconds per stage
    """
    if tile_width * tile_height > 1024:
        raise ValueError("tile_width * tile_height must be <= 1024")
    return Renderer.apply(vertices, indices, colors, opacities, width, height, tile_width, tile_height,
                          early_stopping_threshold, record_timing, per_pixel_sort, max_layers)
