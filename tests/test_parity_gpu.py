"""GPU parity: the HIP path, called through the C ABI (tde_reduce_rms), against the CPU oracle on the
same seeded inputs.  Bar: residual bit-exact, normed <= 1 ulp, codes <= 1 quant step, scales <= 1e-6
relative (test/test_all_reduce_fusion.py:23-28,75-76 is the composition the oracle restates)."""
import pytest
import torch

from oracle import eager
from torch_dist_ext_amd import _capi

from helpers import bits_equal, check_against_oracle, run_hip

pytestmark = pytest.mark.gpu


def _case(name, parts, residual, gamma, eps, quant, **kw):
    print("case", name, tuple(parts.shape), residual.dtype, quant, kw, flush=True)
    want = eager.reduce_rms(parts, residual, gamma, eps, quant)
    got = run_hip(parts, residual, gamma, eps, quant, **kw)
    stats = check_against_oracle(got, want, quant)
    print("  stats", stats, flush=True)
    return got, want, stats


def test_c1_plumbing(cuda_device):
    p, r, g, eps, quant = eager.make_config("c1")
    _case("c1", p, r, g, eps, quant)


def test_c2_decode(cuda_device):
    p, r, g, eps, quant = eager.make_config("c2")
    _case("c2", p, r, g, eps, quant)


@pytest.mark.parametrize("quant", ["none", "fp8_token", "fp8_group", "int8_token"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [2, 4, 8])
def test_small_all_modes(cuda_device, quant, dtype, n):
    p, r, g = eager.make_inputs(n, 37, 1024, dtype, 1.0, seed=11 + n)
    _case("small", p, r, g, 1e-6, quant)


def test_c3_reduced_tokens(cuda_device):
    p, r, g, eps, quant = eager.make_config("c3", tokens=256)
    _case("c3@256", p, r, g, eps, quant)


def test_c4_reduced_tokens(cuda_device):
    p, r, g, eps, quant = eager.make_config("c4", tokens=192)
    _case("c4@192", p, r, g, eps, quant)


@pytest.mark.parametrize("tokens", [1, 64, 512])
def test_c5_outliers(cuda_device, tokens):
    p, r, g, eps, quant = eager.make_config("c5", tokens=tokens)
    _case("c5@%d" % tokens, p, r, g, eps, quant)


@pytest.mark.parametrize("quant", ["none", "fp8_token", "fp8_group", "int8_token"])
def test_staged_equals_fused(cuda_device, quant):
    p, r, g = eager.make_inputs(4, 130, 2048, torch.bfloat16, 1.0, seed=21)
    a = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_FUSED)
    b = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_STAGED)
    for k in a:
        assert bits_equal(a[k], b[k]), k


def test_pointer_table_equals_direct(cuda_device):
    p, r, g = eager.make_inputs(8, 33, 4096, torch.bfloat16, 0.5, seed=22)
    a = run_hip(p, r, g, 1e-5, "fp8_token")
    b = run_hip(p, r, g, 1e-5, "fp8_token", use_table=True, rank=3)
    for k in a:
        assert bits_equal(a[k], b[k]), k
