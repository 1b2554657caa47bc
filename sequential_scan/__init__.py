"""Drop-in name of the reference package: ``from sequential_scan import scan_cu``
keeps working and resolves to the MI355X implementation."""
from fast_sequential_scan_amd import SequentialScan, SequentialScanSingle, scan_cu, scan_cu_single, scan_tr

__all__ = ["scan_cu", "scan_cu_single", "scan_tr", "SequentialScan", "SequentialScanSingle"]
