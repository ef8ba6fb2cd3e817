"""Import shim: lets DEST's models/dest_module.py keep its two imports
(`from issm_triton.issm_combined import ISSM_chunk_scan_combined`,
`from issm_triton.layernorm_gated import RMSNorm`) while the work runs in dest3d_amd."""
