"""Top-level alias so that `from TVInpainting import TVInpaint` keeps working as with the reference's cudaTV/TVInpainting.py."""
from customnetworklayers_amd.cudaTV.TVInpainting import TVInpaint, TVInpaintingFunction  # noqa: F401
