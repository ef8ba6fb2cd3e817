from dest3d_amd.issm_combined import ISSM_chunk_scan_combined, ISSMChunkScanCombinedFn  # noqa: F401
