"""MI355X-native histogram tree growing behind arboretum's C-ABI and Python API."""
from .core import (ArboretumClassifier, ArboretumError, ArboretumRegression, DMatrix, Garden,
                   copy_probe, device_count, hist_sum, hist_sum_no_alloc, hist_sum_plan, load, train)

__all__ = ["DMatrix", "Garden", "train", "load", "ArboretumRegression", "ArboretumClassifier",
           "ArboretumError", "device_count", "hist_sum", "hist_sum_no_alloc", "hist_sum_plan"]
