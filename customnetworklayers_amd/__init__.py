"""MI355X-native TV / TGV FISTA inpainting layers (drop-in for the reference's cudaTV / cudaTGV)."""
from .cudaTV.TVInpainting import TVInpaint, TVInpaintingFunction  # noqa: F401

from .cudaTGV.TGVInpainting import TGVInpaint, TGVInpaintingFunction  # noqa: F401

__all__ = ["TVInpaint", "TVInpaintingFunction", "TGVInpaint", "TGVInpaintingFunction"]
