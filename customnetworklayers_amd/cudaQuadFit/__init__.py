"""Quadratic sub-pixel fit of a matching cost (drop-in for the reference's cudaQuadFit)."""
from .QuadFitting import QuadFittingFromFlow, QuadFittingFromFlowFunction  # noqa: F401
