"""Top-level alias so that `import QuadFit_cuda_ext` keeps working as with the reference build."""
from customnetworklayers_amd.cudaQuadFit.QuadFit_cuda_ext import backward, dummy, dummy_only, forward  # noqa: F401
