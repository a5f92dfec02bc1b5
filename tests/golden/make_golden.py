"""Writes tests/golden/ns_golden.npz, step_golden.npz, aol4_golden.npz and ops_golden.npz from the CPU oracle.

The reference ships no golden vectors and its Newton-Schulz contract (muon.py:265-291) is
comment text, so these fixtures come from oracle/muon_oracle.py, whose functions are pinned by
closed forms and invariants in tests/test_oracle.py.  Run from the repo root:

    python tests/golden/make_golden.py          # all of them
    python tests/golden/make_golden.py ops      # ops_golden.npz alone
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import muon_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().astype(np.uint16)


def aol4():
    """Fixtures of the 4-iteration AOL-rescaled variant (oracle.ns_aol4, pinned by its SVD closed form)."""
    torch.manual_seed(20251126)
    out = {}
    for name, shape, std in [("wide_16x48", (16, 48), 1e-3), ("tall_48x16", (48, 16), 1e-3),
                             ("square_24x24", (24, 24), 1.0), ("wide_40x136", (40, 136), 1e-2),
                             ("batched_3x12x20", (3, 12, 20), 1.0)]:
        G = torch.randn(*shape) * std * (torch.rand(*shape[:-1], 1) * 3 + 0.05)
        out[name + "/in"] = G.numpy()
        out[name + "/bf16"] = bf16_bits(O.ns_aol4(G))
        out[name + "/fp64_closed_form"] = O.ns_aol4_closed_form(G.bfloat16().double().numpy())
    np.savez_compressed(os.path.join(HERE, "aol4_golden.npz"), **out)


def ops():
    """Fixtures of the three product operators (oracle.ns_line_1/2/3, muon.py:420-457, 547-588, 705-745):
    bf16 inputs, the oracle's bf16 results and the exact value of each expression (computed in
    float64 from the bf16 operands the operator is given, stored as float32)."""
    g = torch.Generator().manual_seed(20251127)
    out = {}
    for name, shape in [("small_24x40", (24, 40)), ("ragged_70x130", (70, 130)), ("batched_3x20x36", (3, 20, 36))]:
        X = (torch.randn(*shape, generator=g) * 0.1).bfloat16()
        A = O.ns_line_1(X)
        B = O.ns_line_2(A, 2.0315, -4.7750)
        C = O.ns_line_3(B, X, 3.4445)
        Xd, Ad, Bd = X.double(), A.double(), B.double()
        out[name + "/X"] = bf16_bits(X)
        out[name + "/line1"] = bf16_bits(A)
        out[name + "/line2"] = bf16_bits(B)
        out[name + "/line3"] = bf16_bits(C)
        out[name + "/line1_exact"] = (Xd @ Xd.mT).float().numpy()
        out[name + "/line2_exact"] = (2.0315 * (Ad @ Ad.mT) - 4.7750 * Ad).float().numpy()
        out[name + "/line3_exact"] = (3.4445 * Xd + Bd @ Xd).float().numpy()
    np.savez_compressed(os.path.join(HERE, "ops_golden.npz"), **out)


def main():
    if sys.argv[1:] == ["ops"]:
        ops()
        print("wrote ops_golden.npz")
        return
    aol4()
    ops()
    torch.manual_seed(20251125)
    ns = {}
    for name, shape, std in [("wide_16x48", (16, 48), 1e-3), ("tall_48x16", (48, 16), 1e-3),
                             ("square_8x8", (8, 8), 1.0), ("odd_5x3", (5, 3), 0.02),
                             ("wide_40x136", (40, 136), 1e-2), ("batched_3x12x20", (3, 12, 20), 1.0)]:
        G = torch.randn(*shape) * std
        ns[name + "/in"] = G.numpy()
        ns[name + "/bf16"] = bf16_bits(O.ns5_bf16(G))
        ns[name + "/fp32"] = O.ns5_fp32(G).numpy()
        if G.ndim == 2:
            ns[name + "/fp64_closed_form"] = O.ns5_fp64_closed_form(G)
    np.savez_compressed(os.path.join(HERE, "ns_golden.npz"), **ns)

    # three SingleDeviceMuonWithAuxAdam steps on a tiny mixed parameter set (muon.py:202-260)
    st = {}
    shapes_muon = [(24, 40), (40, 24), (6, 4, 3, 3)]
    shapes_adam = [(50, 8), (8,)]
    pm = [torch.nn.Parameter(torch.randn(*s) * 0.02) for s in shapes_muon]
    pa = [torch.nn.Parameter(torch.randn(*s) * 0.02) for s in shapes_adam]
    opt = O.OracleSingleDeviceMuonWithAuxAdam([
        dict(params=pm, use_muon=True, lr=0.02, weight_decay=0.01),
        dict(params=pa, use_muon=False, lr=3e-4, betas=(0.9, 0.95), weight_decay=0.01)])
    for i, p in enumerate(pm + pa):
        st[f"p{i}/init"] = p.detach().numpy().copy()
    for step in range(3):
        for i, p in enumerate(pm + pa):
            g = torch.randn_like(p) * 1e-3
            st[f"p{i}/grad{step}"] = g.numpy().copy()
            p.grad = g.clone()
        opt.step()
        for i, p in enumerate(pm + pa):
            st[f"p{i}/after{step}"] = p.detach().numpy().copy()
    for i, p in enumerate(pm):
        st[f"p{i}/momentum_buffer"] = opt.state[p]["momentum_buffer"].numpy().copy()
    for i, p in enumerate(pa):
        st[f"p{len(pm) + i}/exp_avg"] = opt.state[p]["exp_avg"].numpy().copy()
        st[f"p{len(pm) + i}/exp_avg_sq"] = opt.state[p]["exp_avg_sq"].numpy().copy()
    np.savez_compressed(os.path.join(HERE, "step_golden.npz"), **st)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
