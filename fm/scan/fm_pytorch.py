"""Import path of the reference (`from fm.scan.fm_pytorch import fm_scan_pytorch`), served by fm_amd."""
from fm_amd.scan.fm_pytorch import fm_scan_pytorch  # noqa: F401
