"""Top-level alias so that `from median import Median` keeps working as with the reference's cudaMedian/median.py."""
from customnetworklayers_amd.cudaMedian.median import Median, MedianFunction  # noqa: F401
