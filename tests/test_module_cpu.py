"""Host-side checks of the MultiHeadISSMScan mirror that need no GPU."""


def test_reference_state_dict_names():
    """The parameter names and shapes a reference checkpoint holds for this module
    (dest_module.py:469-513) load into the mirror."""
    from dest3d_amd.scan_module import MultiHeadISSMScan
    m = MultiHeadISSMScan(d_model=288, d_state=256, d_dist=16, chunk_size=256, nheads=8, expand=1)
    want = {
        "dt_bias": (8,), "A_log": (8,), "D": (8,), "key_proj.weight": (2 * 288 + 2 + 8, 288),
        "key_conv.dwconv.weight": (290, 1, 7), "key_conv.dwconv.bias": (290,),
        "key_conv_back.dwconv.weight": (290, 1, 7), "key_conv_back.dwconv.bias": (290,),
        "query_proj.weight": (288, 288), "bc_proj.weight": (2, 16), "dt_proj.weight": (8, 16),
        "out_key_proj.weight": (288, 288), "out_query_proj.weight": (288, 288), "key_norm.weight": (288,),
        "query_norm.weight": (288,), "query_norm.bias": (288,),
    }
    assert {k: tuple(v.shape) for k, v in m.state_dict().items()} == want
