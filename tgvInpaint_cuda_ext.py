"""Top-level alias so that `import tgvInpaint_cuda_ext` keeps working as with the reference build."""
from customnetworklayers_amd.cudaTGV.tgvInpaint_cuda_ext import *  # noqa: F401,F403
from customnetworklayers_amd.cudaTGV.tgvInpaint_cuda_ext import backward, dummy, dummy_only, forward  # noqa: F401
