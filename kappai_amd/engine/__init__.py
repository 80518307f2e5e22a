from .batch import RowBatch, StepEntry, layout_rows
from .step import StepRunner

__all__ = ["RowBatch", "StepEntry", "layout_rows", "StepRunner"]
