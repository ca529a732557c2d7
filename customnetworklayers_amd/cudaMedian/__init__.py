"""Median of a per-pixel displacement histogram (drop-in for the reference's cudaMedian)."""
from .median import Median, MedianFunction  # noqa: F401
