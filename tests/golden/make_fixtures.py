"""Writes the golden vectors of tests/golden/*.npz: seeded inputs of tiny ISSM scans and gated
RMSNorm rows together with the outputs and gradients of the fp64 oracle (oracle/issm_ref.py).

The reference ships no vectors for this path (its test_issm.py:97-111 only prints relative
errors), so these pin the oracle against silent edits and give the GPU tests fixed data.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import issm_ref as R  # noqa: E402

SCAN_CASES = {
    # name: (B, L, H, P, N, G, seed, softplus, gate[, positions where the sequence id of a packed row goes up])
    "scan_b1_l24_h2_p4_n8": (1, 24, 2, 4, 8, 1, 101, True, False),
    "scan_b2_l70_h4_p8_n12_g2_gate": (2, 70, 4, 8, 12, 2, 102, False, True),
    "scan_b2_l90_h2_p4_n8_packed": (2, 90, 2, 4, 8, 1, 103, True, False, ((7, 64, 65), (30,))),
}


def scan_case(Bsz, L, H, P, N, G, seed, softplus, gate, cuts=None):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    u = lambda *s: torch.rand(*s, generator=g, dtype=torch.float64)
    ins = dict(x=r(Bsz, L, H, P), A=-torch.exp(u(H, N) * 2.5), B=r(Bsz, L, G, N) / N ** 0.5,
               C=r(Bsz, L, G, N) / N ** 0.5, D=r(H), h0=r(Bsz, H, P, N) * 0.5)
    if softplus:
        ins["dt"] = u(Bsz, L, H, N) * 3.0 - 4.0
        ins["dt_bias"] = r(H, N) * 0.2
        limit = (0.03, 0.25)
    else:
        ins["dt"] = torch.nn.functional.softplus(u(Bsz, L, H, N) * 3.0 - 4.0)
        limit = (0.0, float("inf"))
    if gate:
        ins["z"] = r(Bsz, L, H, P)
    dy, dfinal = r(Bsz, L, H, P), r(Bsz, H, P, N)
    leaf = {k: v.clone().requires_grad_() for k, v in ins.items()}
    seq = None
    if cuts is not None:
        seq = torch.zeros(Bsz, L, dtype=torch.int32)
        for b, cs in enumerate(cuts):
            for c in cs:
                seq[b, c:] += 1
    y, fin = R.issm_scan_sequential(leaf["x"], leaf["dt"], leaf["A"], leaf["B"], leaf["C"], D=leaf["D"],
                                    z=leaf.get("z"), dt_bias=leaf.get("dt_bias"), initial_states=leaf["h0"],
                                    dt_softplus=softplus, dt_limit=limit, seq_idx=seq)
    ((y * dy).sum() + (fin * dfinal).sum()).backward()
    out = {"in_" + k: v.numpy() for k, v in ins.items()}
    if seq is not None:
        out["seq_idx"] = seq.numpy()
    out.update(dy=dy.numpy(), dfinal=dfinal.numpy(), y=y.detach().numpy(), final=fin.detach().numpy(),
               softplus=np.array(softplus), dt_limit=np.array(R.limits_as_fp32(limit)))
    out.update({"grad_" + k: v.grad.numpy() for k, v in leaf.items()})
    return out


def norm_case(rows, cols, group, before_gate, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x, z, w, dy = r(rows, cols), r(rows, cols), 1.0 + 0.1 * r(cols), r(rows, cols)
    leaf = [t.clone().requires_grad_() for t in (x, z, w)]
    y = R.gated_rmsnorm_ref(leaf[0], leaf[2], z=leaf[1], eps=1e-5, group_size=group, norm_before_gate=before_gate)
    (y * dy).sum().backward()
    return dict(x=x.numpy(), z=z.numpy(), w=w.numpy(), dy=dy.numpy(), y=y.detach().numpy(), dx=leaf[0].grad.numpy(),
                dz=leaf[1].grad.numpy(), dw=leaf[2].grad.numpy(), group=np.array(group), before_gate=np.array(before_gate))


def layernorm_case(rows, cols, group, before_gate, seed):
    """LayerNorm statistics (mean subtracted) with a bias, gated."""
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x, z, w, b, dy = r(rows, cols) + 0.5, r(rows, cols), 1.0 + 0.1 * r(cols), 0.3 * r(cols), r(rows, cols)
    leaf = [t.clone().requires_grad_() for t in (x, z, w, b)]
    y = R.gated_rmsnorm_ref(leaf[0], leaf[2], z=leaf[1], eps=1e-5, group_size=group, norm_before_gate=before_gate,
                            bias=leaf[3], layer_norm=True)
    (y * dy).sum().backward()
    return dict(x=x.numpy(), z=z.numpy(), w=w.numpy(), b=b.numpy(), dy=dy.numpy(), y=y.detach().numpy(),
                dx=leaf[0].grad.numpy(), dz=leaf[1].grad.numpy(), dw=leaf[2].grad.numpy(), db=leaf[3].grad.numpy(),
                group=np.array(group), before_gate=np.array(before_gate))


def main(force=False):
    """Writes the fixtures that are missing (all of them with --force: the data are a pure function of the seeds)."""
    jobs = {name: (lambda c=c: scan_case(*c)) for name, c in SCAN_CASES.items()}
    jobs["rmsnorm_r6_c32"] = lambda: norm_case(6, 32, 32, True, 201)
    jobs["rmsnorm_r5_c48_g16_gatefirst"] = lambda: norm_case(5, 48, 16, False, 202)
    jobs["layernorm_r6_c32_bias"] = lambda: layernorm_case(6, 32, 32, True, 203)
    jobs["layernorm_r5_c48_g16_bias_gatefirst"] = lambda: layernorm_case(5, 48, 16, False, 204)
    for name, make in jobs.items():
        path = os.path.join(HERE, name + ".npz")
        if force or not os.path.exists(path):
            np.savez_compressed(path, **make())


if __name__ == "__main__":
    main(force="--force" in sys.argv)
