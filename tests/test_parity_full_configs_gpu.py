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

from helpers import bits_equal, check_against_oracle, check_nonfinite, run_hip

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


@pytest.mark.parametrize("name,tokens", [("c3", None), ("c4", 2048), ("c5", 4096)])
def test_full_size_configuration_with_nonfinite_values_sprinkled_in(cuda_device, name, tokens):
    """The configuration's seeded inputs with one element in 20 000 of the partials and of the residual replaced by
    NaN, +inf or -inf (seeded positions): every output against the oracle with NaN matching NaN, and the rows that
    stayed finite bit for bit."""
    parts, residual, gamma, eps, quant = eager.make_config(name, tokens=tokens)
    g = torch.Generator().manual_seed(977)
    special = torch.tensor([float("nan"), float("inf"), float("-inf")], dtype=parts.dtype)
    for t in (parts, residual):
        flat = t.view(-1)
        idx = torch.randint(0, flat.numel(), (max(flat.numel() // 20000, 3),), generator=g)
        flat[idx] = special[torch.randint(0, 3, (idx.numel(),), generator=g)]
    print("full-size non-finite case", name, tuple(parts.shape), parts.dtype, quant, flush=True)
    want = eager.reduce_rms(parts, residual, gamma, eps, quant)
    got = run_hip(parts, residual, gamma, eps, quant)
    check_nonfinite(got, want, quant)
    finite_rows = torch.isfinite(want["norm_out"].float()).all(dim=1)
    assert 0 < int(finite_rows.sum()) < finite_rows.numel()      # both kinds of rows are there
    assert bits_equal(got["norm_out"][finite_rows], want["norm_out"][finite_rows])
    assert bits_equal(got["q"][finite_rows], want["q"][finite_rows])
