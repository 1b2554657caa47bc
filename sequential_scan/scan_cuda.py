"""``sequential_scan.scan_cuda`` of the reference: ``SequentialScan``, ``SequentialScanSingle``,
``scan`` and ``scan_single``, from this package."""
from fast_sequential_scan_amd.scan_cuda import SequentialScan, SequentialScanSingle, scan, scan_single  # noqa: F401

__all__ = ["SequentialScan", "SequentialScanSingle", "scan", "scan_single"]
