from .TGVInpainting import TGVInpaint, TGVInpaintingFunction  # noqa: F401
