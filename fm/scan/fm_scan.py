"""Import path of the reference (`from fm.scan.fm_scan import fm_scan`), served by fm_amd."""
from fm_amd.scan.fm_scan import (FM_Layer, FM_Memory, FM_Readout, FM_Scan, fm_layer, fm_memory, fm_readout,  # noqa: F401
                                 fm_readout_backward, fm_readout_forward, fm_scan, fm_scan_backward,
                                 fm_scan_backward_reduced, fm_scan_forward, module)
