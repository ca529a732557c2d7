"""MI355X-native TV / TGV FISTA inpainting layers (drop-in for the reference's cudaTV / cudaTGV) and the two
small layers upstream of them (cudaQuadFit, cudaMedian)."""
from .cudaTV.TVInpainting import TVInpaint, TVInpaintingFunction  # noqa: F401

from .cudaTGV.TGVInpainting import TGVInpaint, TGVInpaintingFunction  # noqa: F401

from .cudaQuadFit.QuadFitting import QuadFittingFromFlow, QuadFittingFromFlowFunction  # noqa: F401
from .cudaMedian.median import Median, MedianFunction  # noqa: F401

__all__ = ["TVInpaint", "TVInpaintingFunction", "TGVInpaint", "TGVInpaintingFunction", "QuadFittingFromFlow",
           "QuadFittingFromFlowFunction", "Median", "MedianFunction"]
