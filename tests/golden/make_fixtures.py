"""Writes the golden vectors under tests/golden/ from the CPU oracle.

The reference's own tests hold no Muon vectors (no reference test executes Muon), and the
reference is not imported here: the oracle is pinned by the closed-form and invariant
checks in tests/test_oracle.py, and these files freeze its outputs so that later changes to
the oracle or the HIP path are caught.  Run from the repo root:
    python tests/golden/make_fixtures.py
Inputs are regenerated from the seeds stored in each file; bf16 tensors are stored as
uint16 bit patterns.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import muon_oracle as O  # noqa: E402
from tests.helpers import MUON_HP, make_param_set, u16_from_bf16  # noqa: E402

NS_CASES = [(64, 160, 101), (160, 64, 102), (33, 47, 103), (128, 896, 104), (256, 256, 105)]
STEP_SPEC = dict(q=(64, 64), k=(32, 64), v=(32, 64), o=(64, 64), gate=(160, 64), up=(160, 64), down=(64, 160))


def ns_input(rows, cols, seed):
    return torch.randn(rows, cols, generator=torch.Generator().manual_seed(seed))


def main():
    torch.set_num_threads(1)  # one thread: a fixed accumulation order
    out = {}
    for rows, cols, seed in NS_CASES:
        G = ns_input(rows, cols, seed)
        for steps in (1, 5):
            out[f"ns_{rows}x{cols}_seed{seed}_steps{steps}"] = u16_from_bf16(O.newton_schulz(G, steps))
    np.savez_compressed(os.path.join(HERE, "ns_small.npz"), **out)

    weights, grads = make_param_set(STEP_SPEC, layers=1, seed=7, steps=3)
    params = [torch.nn.Parameter(w.clone()) for _, w in weights]
    hp = dict(MUON_HP)
    groups = [dict(params=sorted(params, key=lambda x: x.size(), reverse=True), use_muon=True, **hp)]
    order = [next(i for i, p in enumerate(params) if p is q) for q in groups[0]["params"]]
    orc = O.OracleMuon(groups)
    out = {"order": np.array(order)}
    for step in range(3):
        for p, g in zip(params, grads[step]):
            p.grad = g.clone()
        orc.step()
        for j, p in enumerate(groups[0]["params"]):
            out[f"step{step}_update{j}"] = u16_from_bf16(orc.last_updates[(0, j)])
            if step == 2:
                out[f"final_param{j}"] = p.detach().numpy().copy()
                out[f"final_momentum{j}"] = orc.state[(0, j)]["momentum_buffer"].numpy().copy()
    np.savez_compressed(os.path.join(HERE, "step_small.npz"), **out)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
