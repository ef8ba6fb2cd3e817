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
    # name: (B, L, H, P, N, G, seed, softplus, gate)
    "scan_b1_l24_h2_p4_n8": (1, 24, 2, 4, 8, 1, 101, True, False),
    "scan_b2_l70_h4_p8_n12_g2_gate": (2, 70, 4, 8, 12, 2, 102, False, True),
}


def scan_case(Bsz, L, H, P, N, G, seed, softplus, gate):
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
    y, fin = R.issm_scan_sequential(leaf["x"], leaf["dt"], leaf["A"], leaf["B"], leaf["C"], D=leaf["D"],
                                    z=leaf.get("z"), dt_bias=leaf.get("dt_bias"), initial_states=leaf["h0"],
                                    dt_softplus=softplus, dt_limit=limit)
    ((y * dy).sum() + (fin * dfinal).sum()).backward()
    out = {"in_" + k: v.numpy() for k, v in ins.items()}
    out.update(dy=dy.numpy(), dfinal=dfinal.numpy(), y=y.detach().numpy(), final=fin.detach().numpy(),
               softplus=np.array(softplus), dt_limit=np.array(limit))
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


def main():
    for name, c in SCAN_CASES.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **scan_case(*c))
    np.savez_compressed(os.path.join(HERE, "rmsnorm_r6_c32.npz"), **norm_case(6, 32, 32, True, 201))
    np.savez_compressed(os.path.join(HERE, "rmsnorm_r5_c48_g16_gatefirst.npz"), **norm_case(5, 48, 16, False, 202))


if __name__ == "__main__":
    main()
