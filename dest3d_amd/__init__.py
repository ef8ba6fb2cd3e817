"""MI355X-native implementation of DEST's interactive-SSM chunked scan and its gated
RMSNorm epilogue (hand-written gfx950 HIP kernels behind a C ABI)."""
from .issm_combined import ISSM_chunk_scan_combined, ISSM_biscan_combined, ISSMChunkScanCombinedFn  # noqa: F401
from .layernorm_gated import LayerNorm, RMSNorm, layernorm_fn, rmsnorm_fn  # noqa: F401
