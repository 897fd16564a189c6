"""trigrad_amd -- MI355X (gfx950) implementation of trigrad's differentiable tile
rasterizer behind the reference's Python entry point (`render`, `precision`)."""
from . import camera
from .tests_wrapper import barycentric, interpolate3_scalar, interpolate3_vector
from ._C import force_tickets, set_precision, verify_frames
from .wrapper import Renderer, precision, render

__all__ = ["render", "barycentric", "interpolate3_scalar", "interpolate3_vector", "precision", "Renderer", "camera", "set_precision",
           "verify_frames", "force_tickets"]

__version__ = "0.1.0"
