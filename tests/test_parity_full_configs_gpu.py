"""GPU parity at the benchmark configurations' full sizes: the HIP path (tde_reduce_rms through the C ABI) against
the CPU oracle on identical seeded CPU-generated inputs.  Every output must be bit-identical: residual, normed rows,
scales and codes (the stated bounds -- normed within 1 ulp, codes within one quant step, scales within 1e-6 relative --
are met with zero differences).

With TDE_PARITY_COUNTS=<file> in the environment every case appends one JSON line of mismatch counts to that file."""
import json
import os

import pytest
import torch

from oracle import eager

from helpers import check_against_oracle, run_hip

pytestmark = pytest.mark.gpu

CASES = [("c1", None), ("c2", None), ("c3", None), ("c4", None),
         ("c5", 1), ("c5", 64), ("c5", 512), ("c5", 4096), ("c5", 32768)]


@pytest.mark.parametrize("name,tokens", CASES)
def test_full_size_configuration_against_oracle(cuda_device, name, tokens):
    parts, residual, gamma, eps, quant = eager.make_config(name, tokens=tokens)
    label = name if tokens is None else "%s@%d" % (name, tokens)
    print("full-size case", label, tuple(parts.shape), parts.dtype, quant, flush=True)
    want = eager.reduce_rms(parts, residual, gamma, eps, quant)
    got = run_hip(parts, residual, gamma, eps, quant)
    stats = check_against_oracle(got, want, quant, gamma=gamma, eps=eps)
    stats.update(config=label, shape=list(parts.shape), dtype=str(parts.dtype), quant=quant,
                 elements=int(residual.numel()), scales=int(want["scale"].numel()) if "scale" in want else 0)
    print("  stats", stats, flush=True)
    counts_file = os.environ.get("TDE_PARITY_COUNTS")
    if counts_file:
        with open(counts_file, "a") as f:
            f.write(json.dumps(stats) + "\n")
