"""Top-level alias so that `from QuadFitting import QuadFittingFromFlow` keeps working as with the reference's cudaQuadFit/QuadFitting.py."""
from customnetworklayers_amd.cudaQuadFit.QuadFitting import QuadFittingFromFlow, QuadFittingFromFlowFunction  # noqa: F401
