"""Writes tests/golden/golden.npz: inputs and expected outputs of the CPU oracle (oracle/eager.py)
for configuration c1 (2 partials, 16 x 1024 bf16, seed 0) and three tiny quant cases.  The reference has no golden vectors and
its package is not imported here: these fixtures freeze this build's oracle so that a later change
to it (or a different torch CPU build) is noticed.  bf16/fp16 arrays are stored as uint16 bits.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import eager  # noqa: E402


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    cases = {}
    p, r, g, eps, quant = eager.make_config("c1")
    cases["c1"] = (p, r, g, eps, quant, "bf16")
    for name, dtype, dn, quant in (("q_fp8_token", torch.bfloat16, "bf16", "fp8_token"),
                                   ("q_fp8_group", torch.bfloat16, "bf16", "fp8_group"),
                                   ("q_int8_token", torch.float16, "f16", "int8_token")):
        p, r, g = eager.make_inputs(2, 4, 256, dtype, 1.0, seed=100 + len(cases))
        cases[name] = (p, r, g, 1e-6, quant, dn)
    out = {}
    for name, (p, r, g, eps, quant, dn) in cases.items():
        o = eager.reduce_rms(p, r, g, eps, quant)
        out[name + "/dtype"] = np.array(dn)
        out[name + "/quant"] = np.array(quant)
        out[name + "/eps"] = np.array(eps, dtype=np.float64)
        out[name + "/parts"] = bits(p)
        out[name + "/residual"] = bits(r)
        out[name + "/gamma"] = bits(g)
        out[name + "/residual_out"] = bits(o["residual_out"])
        out[name + "/norm_out"] = bits(o["norm_out"])
        if quant != "none":
            out[name + "/q"] = o["q"].view(torch.uint8).numpy()
            out[name + "/scale"] = o["scale"].numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
