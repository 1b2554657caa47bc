"""``sequential_scan.common`` of the reference: the same helper names, from this package."""
from fast_sequential_scan_amd.common import *  # noqa: F401,F403
from fast_sequential_scan_amd.common import __all__  # noqa: F401
