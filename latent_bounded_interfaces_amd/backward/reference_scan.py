"""Module name of the reference for the scan step configured by mode name (reference
backward/reference_scan.py); the function itself lives beside the step it wraps."""
from .scan import ReferenceScanEngine, ScanADEngine, lbi_reference_scan_backward_step, lbi_scan_backward_step

__all__ = ["ReferenceScanEngine", "ScanADEngine", "lbi_reference_scan_backward_step", "lbi_scan_backward_step"]
