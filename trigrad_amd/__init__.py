"""trigrad_amd -- MI355X (gfx950) implementation of trigrad's differentiable tile
rasterizer behind the reference's Python entry point (`render`, `precision`)."""
from .wrapper import Renderer, precision, render

__all__ = ["render", "precision", "Renderer"]

__version__ = "0.1.0"
