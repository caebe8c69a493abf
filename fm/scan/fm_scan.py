"""Import path of the reference (`from fm.scan.fm_scan import fm_scan`), served by fm_amd."""
from fm_amd.scan.fm_scan import (FM_Scan, fm_memory, fm_scan, fm_scan_backward,  # noqa: F401
                                 fm_scan_backward_reduced, fm_scan_forward, module)
