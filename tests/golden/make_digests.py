"""Writes tests/golden/digests.json: SHA-256 of the inputs and of the CPU oracle's outputs
(oracle/eager.py) for the full-size configurations c2, c3, c4 and c5 at 4096 tokens, whose tensors are
too large to commit.  Inputs regenerate from their seeds (CPU torch.Generator); the input digest tells a
test whether the host's torch produced the same inputs before it compares anything else.

    python tests/golden/make_digests.py
"""
import hashlib
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import eager  # noqa: E402

CASES = (("c2", None), ("c3", None), ("c4", None), ("c5", 4096))


def sha(*tensors):
    h = hashlib.sha256()
    for t in tensors:
        h.update(t.contiguous().view(torch.uint8).numpy().tobytes())
    return h.hexdigest()


def digest_case(name, tokens):
    p, r, g, eps, quant = eager.make_config(name, tokens=tokens)
    o = eager.reduce_rms(p, r, g, eps, quant)
    d = {"tokens": int(r.shape[0]), "hidden": int(r.shape[1]), "nranks": int(p.shape[0]), "quant": quant,
         "inputs": sha(p, r, g), "residual_out": sha(o["residual_out"]), "norm_out": sha(o["norm_out"])}
    if quant != "none":
        d["q"] = sha(o["q"])
        d["scale"] = sha(o["scale"])
    return d


def main():
    # norm_out / q / scale depend on the order torch's CPU mean() adds in, which follows the host's vector ISA
    out = {"cpu_capability": torch.backends.cpu.get_cpu_capability()}
    for name, tokens in CASES:
        key = name if tokens is None else "%s@%d" % (name, tokens)
        out[key] = digest_case(name, tokens)
        print(key, out[key]["residual_out"][:16], flush=True)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "digests.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()
