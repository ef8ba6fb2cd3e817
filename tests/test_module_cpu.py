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


def test_reversed_branch_convolves_the_forward_branch_output():
    """dest_module.py:530 reassigns xbc = key_conv(xbc); :534 then calls key_conv_back on THAT tensor.  With both
    depthwise kernels set to the identity tap and zero bias a convolution + SiLU is SiLU alone, so the reversed-order
    branch must see silu(silu(u)) -- visibly different from silu(u), which is what it would see if it read the
    key_proj output.  Checked on the restatement the GPU parity tests compare with."""
    import torch
    import torch.nn.functional as F
    from oracle.module_ref import multi_head_issm_scan_ref
    from dest3d_amd.scan_module import MultiHeadISSMScan
    torch.manual_seed(3)
    D, K, H, M = 24, 6, 2, 16
    m = MultiHeadISSMScan(d_model=D, d_state=K, d_dist=M, chunk_size=256, nheads=H, expand=1).double()
    with torch.no_grad():
        for conv in (m.key_conv.dwconv, m.key_conv_back.dwconv):
            conv.weight.zero_()
            conv.weight[:, 0, 3] = 1.0
            conv.bias.zero_()
    sd = m.state_dict()
    g = torch.Generator().manual_seed(4)
    in_key = torch.randn(2, 9, D, generator=g, dtype=torch.float64)
    in_query = torch.randn(2, K, D, generator=g, dtype=torch.float64)
    dist = 0.5 * torch.randn(2, 9, K, M, generator=g, dtype=torch.float64)
    got = {}
    cfg = dict(nheads=H, ngroups=1, d_inner=D, d_state=K, use_biscan=True)
    multi_head_issm_scan_ref(sd, cfg, in_key, in_query, dist, None, intermediates=got)
    u = (in_key @ sd["key_proj.weight"].T)[..., D:2 * D + 2]
    once, twice = F.silu(u), F.silu(F.silu(u))
    assert torch.allclose(got["x"], once[..., :D], atol=1e-14)
    assert torch.allclose(got["x_back"], twice[..., :D], atol=1e-14)
    assert (once - twice).abs().max() > 0.1                      # the two readings are far apart
    # the bias columns of the reversed branch follow the same chain
    assert torch.allclose(got["B_back"] - got["B"], (twice[..., D:D + 1] - once[..., D:D + 1]).unsqueeze(-1).expand_as(got["B"]),
                          atol=1e-13)


def test_reversed_branch_sees_zero_padding_of_the_convolved_tensor():
    """The second convolution pads ITS input (the first one's output) with zeros; it does not see the first convolution
    evaluated on padding.  With a first-conv bias b the latter would be silu(b) != 0 just outside the sequence."""
    import torch
    import torch.nn.functional as F
    from oracle.module_ref import point_lite_conv
    g = torch.Generator().manual_seed(5)
    C = 3
    sd = {"a.dwconv.weight": torch.randn(C, 1, 7, generator=g, dtype=torch.float64),
          "a.dwconv.bias": torch.full((C,), 2.0, dtype=torch.float64),
          "b.dwconv.weight": torch.ones(C, 1, 7, dtype=torch.float64), "b.dwconv.bias": torch.zeros(C, dtype=torch.float64)}
    u = torch.randn(1, 5, C, generator=g, dtype=torch.float64)
    y0 = point_lite_conv(sd, "a", u)
    y1 = point_lite_conv(sd, "b", y0)
    # all-ones taps over a 5-token sequence with padding 3: every output is the plain sum of y0 over the tokens in reach
    want = torch.stack([y0[0, max(0, l - 3):l + 4].sum(0) for l in range(5)])
    assert torch.allclose(y1[0], F.silu(want), atol=1e-13)
