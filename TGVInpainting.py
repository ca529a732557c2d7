"""Top-level alias so that `from TGVInpainting import TGVInpaint` keeps working as with the reference's cudaTGV/TGVInpainting.py."""
from customnetworklayers_amd.cudaTGV.TGVInpainting import TGVInpaint, TGVInpaintingFunction  # noqa: F401
