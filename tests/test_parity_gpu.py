"""GPU parity: the HIP path, called through the C ABI (tde_reduce_rms), against the CPU oracle on the
same seeded inputs.  Bar: every output bit-identical (stated: residual bit-exact, normed <= 1 ulp, codes <= 1
quant step, scales <= 1e-6 relative; test/test_all_reduce_fusion.py:23-28,75-76 is the composition the oracle
restates)."""
import os

import pytest
import torch

from oracle import eager
from torch_dist_ext_amd import _capi

from helpers import bits_equal, check_against_oracle, check_nonfinite, run_hip, ulp_distance

pytestmark = pytest.mark.gpu


def _case(name, parts, residual, gamma, eps, quant, strict=None, **kw):
    print("case", name, tuple(parts.shape), residual.dtype, quant, kw, flush=True)
    want = eager.reduce_rms(parts, residual, gamma, eps, quant)
    got = run_hip(parts, residual, gamma, eps, quant, **kw)
    stats = check_against_oracle(got, want, quant, gamma=gamma, eps=eps, strict=strict)
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


@pytest.mark.parametrize("tokens", [1, 64, 512, 4096])
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
    # and the staged outputs against the oracle themselves, not only against the fused kernel
    check_against_oracle(b, eager.reduce_rms(p, r, g, 1e-6, quant), quant, gamma=g, eps=1e-6)


def _rank_order_sum(parts):
    acc = torch.zeros(parts.shape[1:], dtype=torch.float32)
    for r in range(parts.shape[0]):
        acc = acc + parts[r].float()
    return acc.to(parts.dtype)


@pytest.mark.parametrize("n,rank,tokens,hidden,dtype,quant", [
    (4, 0, 130, 2048, torch.bfloat16, "none"),
    (4, 3, 130, 2048, torch.bfloat16, "fp8_token"),
    (8, 5, 67, 4096, torch.bfloat16, "fp8_group"),
    (8, 7, 3, 1024, torch.float16, "int8_token"),   # fewer rows than ranks: rank 7 owns none
    (2, 1, 129, 1024, torch.float32, "none"),
    (8, 2, 40, 8192, torch.bfloat16, "fp8_token"),
    (4, 1, 33, 1000, torch.bfloat16, "none"),       # row not a multiple of the span
])
def test_staged_owned_rows(cuda_device, n, rank, tokens, hidden, dtype, quant):
    """One rank of the reference's two-shot (all_reduce_fusion_impl.h:365-393): stage A sums only
    rows == rank (mod N); the peers' rows of the stage are already there.  The owned rows start as
    NaN, the others as the oracle's sums: the final outputs must equal the fused path bit for bit,
    the owned rows of the stage must be the rank-order sums and the other rows must be untouched."""
    p, r, g = eager.make_inputs(n, tokens, hidden, dtype, 1.0, seed=300 + n + rank)
    sums = _rank_order_sum(p)
    init = sums.clone()
    init[rank::n] = float("nan")
    a = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_FUSED, rank=rank)
    b = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_STAGED_OWNED, rank=rank, stage_init=init)
    assert bits_equal(b.pop("stage"), sums)
    for k in a:
        assert bits_equal(a[k], b[k]), k
    check_against_oracle(b, eager.reduce_rms(p, r, g, 1e-6, quant), quant, gamma=g, eps=1e-6)
    # a wrong share is visible: with nothing pre-filled, rows of other ranks stay NaN
    if tokens > 1:
        c = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_STAGED_OWNED, rank=rank,
                    stage_init=torch.full_like(sums, float("nan")))
        own = torch.zeros(tokens, dtype=torch.bool)
        own[rank::n] = True
        assert bits_equal(c["stage"][own], sums[own])
        assert torch.isnan(c["stage"][~own].float()).all()
        assert bits_equal(c["residual_out"][own], a["residual_out"][own])
        assert torch.isnan(c["residual_out"][~own].float()).all()


@pytest.mark.parametrize("n,tokens,hidden,dtype,quant", [
    (4, 130, 2048, torch.bfloat16, "fp8_token"), (8, 67, 4096, torch.float16, "fp8_group"),
    (2, 129, 1024, torch.float32, "none"), (8, 5, 8192, torch.bfloat16, "int8_token"),
])
def test_two_shot_emulated_by_phase_calls(cuda_device, n, tokens, hidden, dtype, quant):
    """The whole two-shot on one GPU: N tde_stage_reduce calls, one per rank's share of the rows, all
    into the same (NaN-filled) stage, then one tde_stage_norm.  Bit-identical to the fused path."""
    p, r, g = eager.make_inputs(n, tokens, hidden, dtype, 1.0, seed=400 + n)
    a = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_FUSED)
    calls = [(("reduce",), k) for k in range(n)] + [(("norm",), 0)]
    b = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_STAGED_OWNED, calls=calls,
                stage_init=torch.full((tokens, hidden), float("nan"), dtype=dtype))
    assert bits_equal(b.pop("stage"), _rank_order_sum(p))
    for k in a:
        assert bits_equal(a[k], b[k]), k
    want = eager.reduce_rms(p, r, g, 1e-6, quant)
    check_against_oracle(b, want, quant, gamma=g, eps=1e-6)
    # and the all-rows staged algorithm split the same way
    c = run_hip(p, r, g, 1e-6, quant, algo=_capi.ALGO_STAGED, calls=[(("reduce",), 0), (("norm",), 0)])
    for k in a:
        assert bits_equal(a[k], c[k]), k
    check_against_oracle(c, want, quant, gamma=g, eps=1e-6)


def test_phase_calls_need_a_staged_algorithm(cuda_device):
    p, r, g = eager.make_inputs(4, 8, 1024, torch.bfloat16, 1.0, seed=5)
    for phases in (("reduce",), ("norm",)):
        with pytest.raises(_capi.TdeError) as ei:
            run_hip(p, r, g, 1e-6, "none", algo=_capi.ALGO_FUSED, calls=[(phases, 0)],
                    stage_init=torch.zeros(8, 1024, dtype=torch.bfloat16))
        assert ei.value.status == _capi.EALGO


def test_pointer_table_equals_direct(cuda_device):
    p, r, g = eager.make_inputs(8, 33, 4096, torch.bfloat16, 0.5, seed=22)
    a = run_hip(p, r, g, 1e-5, "fp8_token")
    b = run_hip(p, r, g, 1e-5, "fp8_token", use_table=True, rank=3)
    for k in a:
        assert bits_equal(a[k], b[k]), k


# Shapes of the reference's own tests: tokens {128,129} x 1024 x N=4 in fp32/bf16/fp16
# (test/test_all_reduce_fusion.py:78-87) and the fp32 grid of test/unit_test.cpp:322-323, whose
# hidden sizes 508 and 124 leave the last wavefront partly empty.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens", [128, 129])
def test_reference_python_test_shapes(cuda_device, dtype, tokens):
    g = torch.Generator().manual_seed(tokens)
    parts = torch.randn((4, tokens, 1024), generator=g).to(dtype)
    residual = torch.randn((tokens, 1024), generator=g).to(dtype)
    gamma = torch.randn((1024,), generator=g).to(dtype)  # the reference draws gamma from N(0,1)
    _case("pytest-shape", parts, residual, gamma, 1e-6, "none")


@pytest.mark.parametrize("hidden", [1024, 508, 124])
@pytest.mark.parametrize("tokens", [513, 127, 3])
def test_reference_unit_test_shapes_fp32(cuda_device, tokens, hidden):
    g = torch.Generator().manual_seed(tokens * 7 + hidden)
    parts = torch.rand((8, tokens, hidden), generator=g)
    residual = torch.rand((tokens, hidden), generator=g)
    gamma = torch.rand((hidden,), generator=g)
    _case("unit-shape", parts, residual, gamma, 1e-6, "none")


# ---- edge cases -----------------------------------------------------------------------------------------

def test_empty_input_is_a_no_op(cuda_device):
    p, r, g = eager.make_inputs(2, 0, 1024, torch.bfloat16, 1.0, seed=1)
    got = run_hip(p, r, g, 1e-6, "fp8_token")
    assert got["residual_out"].shape == (0, 1024) and got["q"].numel() == 0


@pytest.mark.parametrize("hidden", [8, 64, 1016, 8192])
@pytest.mark.parametrize("quant", ["none", "int8_token"])
def test_ragged_and_extreme_hidden(cuda_device, hidden, quant):
    p, r, g = eager.make_inputs(2, 5, hidden, torch.bfloat16, 1.0, seed=hidden)
    _case("hidden", p, r, g, 1e-6, quant)


def test_all_zero_rows_and_signed_zero(cuda_device):
    p, r, g = eager.make_inputs(4, 6, 512, torch.bfloat16, 1.0, seed=2)
    p[:, 1] = 0.0
    r[1] = 0.0
    p[:, 3] = -0.0
    r[3] = -0.0
    for quant in ("none", "fp8_token", "fp8_group", "int8_token"):
        got, want, _ = _case("zeros", p, r, g, 1e-6, quant)
        assert torch.all(got["residual_out"][3].view(torch.int16) == 0)   # -0 partials sum to +0
        if quant != "none":
            assert torch.all(got["scale"].reshape(6, -1)[1] == 0) and torch.all(got["q"][1].float() == 0)


def test_rank_order_vector_on_gpu(cuda_device):
    vals = [2.0 ** 24, 1.0, -(2.0 ** 24), 1.0]
    parts = torch.tensor(vals, dtype=torch.bfloat16).view(4, 1, 1).expand(4, 3, 256).contiguous()
    r = torch.zeros((3, 256), dtype=torch.bfloat16)
    g = torch.ones((256,), dtype=torch.bfloat16)
    got = run_hip(parts, r, g, 1e-6, "none")
    assert torch.all(got["residual_out"].float() == 1.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("vpt", [1, 2, 4])
def test_rank_order_vector_every_geometry(cuda_device, vpt, dtype):
    """The order-sensitive sum in every accumulation path (vector by vector; rank by rank as the loads arrive with four
    vectors per thread), four and eight partials: ((((0 + a) + 1) - a) + 1) = 1 only in rank order, with a large enough
    for a + 1 to round back to a."""
    # fp16 cannot hold 2^24, but 2^15 + 2^-10 rounds back to 2^15 in the fp32 accumulator just the same
    big, small = (2.0 ** 24, 1.0) if dtype != torch.float16 else (2.0 ** 15, 2.0 ** -10)
    hidden = 2048
    for vals in ([big, small, -big, small], [big, small, -big, small, big, small, -big, small]):
        n = len(vals)
        parts = torch.tensor(vals, dtype=dtype).view(n, 1, 1).expand(n, 5, hidden).contiguous()
        r = torch.zeros((5, hidden), dtype=dtype)
        g = torch.ones((hidden,), dtype=dtype)
        want = eager.reduce_rms(parts, r, g, 1e-6, "none")
        assert torch.all(want["residual_out"].float() == small)
        got = run_hip(parts, r, g, 1e-6, "none", vecs_per_thread=vpt)
        assert torch.all(got["residual_out"].float() == small), (vpt, n)


def test_sum_of_ones_row_reduction_all_wave_counts(cuda_device):
    # mean(x^2) of a row of ones is exactly 1 for every hidden: checks the 64-lane + LDS reduction tree
    for hidden in (8, 64, 1016, 1024, 5120, 7168, 8192):
        parts = torch.zeros((2, 3, hidden), dtype=torch.bfloat16)
        r = torch.ones((3, hidden), dtype=torch.bfloat16)
        g = torch.ones((hidden,), dtype=torch.bfloat16)
        got = run_hip(parts, r, g, 0.0, "none")
        assert torch.all(got["norm_out"].float() == 1.0), hidden


@pytest.mark.parametrize("vpt", [1, 2, 4])
@pytest.mark.parametrize("hidden,rows_per_block", [(8192, 0), (1024, 0), (1024, 2), (1024, 4)])
def test_every_launch_geometry_agrees(cuda_device, vpt, hidden, rows_per_block):
    """Forced vectors-per-thread and rows per workgroup (tde_problem's per-call overrides)."""
    p, r, g = eager.make_inputs(8, 41, hidden, torch.bfloat16, 0.5, seed=77)
    base = run_hip(p, r, g, 1e-5, "fp8_token")
    other = run_hip(p, r, g, 1e-5, "fp8_token", vecs_per_thread=vpt, rows_per_block=rows_per_block)
    code = _capi.make_problem(_capi.BF16, 8, 41, hidden, 1e-5, vecs_per_thread=vpt, rows_per_block=rows_per_block)
    plan = _capi.plan(code)
    assert plan.vecs_per_thread == vpt and (rows_per_block == 0 or plan.rows_per_block == rows_per_block)
    want = eager.reduce_rms(p, r, g, 1e-5, "fp8_token")
    check_against_oracle(other, want, "fp8_token", gamma=g, eps=1e-5)
    for key in base:
        assert bits_equal(base[key], other[key]), key


@pytest.mark.parametrize("limit", [1, 2, 3, 8])
@pytest.mark.parametrize("n,hidden,dtype,quant", [(8, 8192, torch.bfloat16, "fp8_token"), (4, 7168, torch.bfloat16, "fp8_group"),
                                                  (4, 5120, torch.float16, "int8_token"), (2, 1024, torch.float32, "none")])
def test_every_workgroup_limit_agrees(cuda_device, limit, n, hidden, dtype, quant):
    """A forced limit on resident workgroups per CU pads the launch's dynamic LDS (beyond 64 KiB for limits 1 and 2,
    which needs the kernel's LDS ceiling raised first) and changes nothing else."""
    p, r, g = eager.make_inputs(n, 53, hidden, dtype, 0.5, seed=91)
    base = run_hip(p, r, g, 1e-5, quant, workgroups_per_cu=-1)
    other = run_hip(p, r, g, 1e-5, quant, workgroups_per_cu=limit)
    check_against_oracle(other, eager.reduce_rms(p, r, g, 1e-5, quant), quant, gamma=g, eps=1e-5)
    for key in base:
        assert bits_equal(base[key], other[key]), key


@pytest.mark.parametrize("tokens,hidden,dtype,quant", [(1100, 8192, torch.bfloat16, "fp8_token"), (4100, 2048, torch.float16, "int8_token"),
                                                       (1030, 7168, torch.bfloat16, "int8_token"), (1100, 8192, torch.float16, "fp8_group"),
                                                       (1100, 4096, torch.float32, "none"), (1050, 4096, torch.float32, "fp8_token"),
                                                       (1100, 8192, torch.bfloat16, "none"), (1100, 8192, torch.bfloat16, "fp8_static")])
def test_wide_instantiation_agrees_with_the_plain_one(cuda_device, tokens, hidden, dtype, quant):
    """Eight partials with four vectors per thread at 4 to 24 workgroups per CU run the row kernel compiled for two
    wavefronts per SIMD, with gamma requested ahead of the row (the plan reports it as two workgroups per CU);
    tune_workgroups_per_cu = -1 keeps the plain instantiation.  Same bits from both, and the oracle's."""
    p, r, g = eager.make_inputs(8, tokens, hidden, dtype, 0.5, seed=191)
    dcode = {torch.bfloat16: _capi.BF16, torch.float16: _capi.F16, torch.float32: _capi.F32}[dtype]
    qcode = {"none": _capi.QUANT_NONE, "fp8_token": _capi.QUANT_FP8_TOKEN, "fp8_group": _capi.QUANT_FP8_GROUP,
             "int8_token": _capi.QUANT_INT8_TOKEN, "fp8_static": _capi.QUANT_FP8_STATIC}[quant]
    static = 0.013 if quant == "fp8_static" else 0.0
    auto = _capi.plan(_capi.make_problem(dcode, 8, tokens, hidden, 1e-5, quant=qcode, static_scale=static))
    plain = _capi.plan(_capi.make_problem(dcode, 8, tokens, hidden, 1e-5, quant=qcode, static_scale=static, workgroups_per_cu=-1))
    assert auto.vecs_per_thread == 4 and auto.workgroups_per_cu == 2 and plain.workgroups_per_cu == 0
    assert auto.lds_bytes == plain.lds_bytes                      # no LDS padding: the registers are the limit
    wide = run_hip(p, r, g, 1e-5, quant, static_scale=static, use_table=(quant == "fp8_token"))   # also through the pointer table
    base = run_hip(p, r, g, 1e-5, quant, static_scale=static, workgroups_per_cu=-1)
    want = eager.reduce_rms(p, r, g, 1e-5, quant, static_scale=static) if quant == "fp8_static" else eager.reduce_rms(p, r, g, 1e-5, quant)
    check_against_oracle(wide, want, quant, gamma=g, eps=1e-5)
    for key in base:
        assert bits_equal(base[key], wide[key]), key


@pytest.mark.parametrize("n,tokens,hidden,dtype,quant,vpt", [
    (8, 16384, 4096, torch.bfloat16, "fp8_token", 2), (8, 8192, 6144, torch.float16, "int8_token", 2),
    (8, 2048, 6144, torch.bfloat16, "fp8_group", 4), (4, 32768, 2048, torch.bfloat16, "none", 2),
    (8, 4100, 1024, torch.float16, "fp8_token", 2)])
def test_long_launches_of_mid_length_rows(cuda_device, n, tokens, hidden, dtype, quant, vpt):
    """The geometries the plan picks for long launches of mid-length rows (two or four vectors per thread, several rows per
    workgroup, a limit on workgroups per CU), whole launches against the oracle."""
    dcode = _capi.BF16 if dtype == torch.bfloat16 else _capi.F16
    qcode = {"none": _capi.QUANT_NONE, "fp8_token": _capi.QUANT_FP8_TOKEN, "fp8_group": _capi.QUANT_FP8_GROUP, "int8_token": _capi.QUANT_INT8_TOKEN}[quant]
    assert _capi.plan(_capi.make_problem(dcode, n, tokens, hidden, 1e-5, quant=qcode)).vecs_per_thread == vpt
    p, r, g = eager.make_inputs(n, tokens, hidden, dtype, 0.5, seed=233)
    got = run_hip(p, r, g, 1e-5, quant)
    check_against_oracle(got, eager.reduce_rms(p, r, g, 1e-5, quant), quant, gamma=g, eps=1e-5)


def test_long_launch_with_automatic_workgroup_limit(cuda_device):
    """6144 rows of 8 partials: the plan limits the launch to two workgroups per CU (79 KiB of dynamic LDS each).
    Same bits as the unlimited launch, on the device."""
    dev = cuda_device
    n, t, h = 8, 6144, 5120
    prob = _capi.make_problem(_capi.BF16, n, t, h, 1e-5, quant=_capi.QUANT_FP8_TOKEN)
    plan = _capi.plan(prob)
    assert plan.workgroups_per_cu == 2 and plan.lds_bytes > 64 * 1024
    gen = torch.Generator(device=dev).manual_seed(17)
    parts = [(torch.randn((t, h), generator=gen, device=dev) * 0.5).to(torch.bfloat16) for _ in range(n)]
    res = torch.randn((t, h), generator=gen, device=dev).to(torch.bfloat16)
    gamma = (torch.rand((h,), generator=gen, device=dev) + 0.5).to(torch.bfloat16)
    outs = []
    for limit in (0, -1):
        res_out = torch.full_like(res, float("nan"))
        q = torch.full((t, h), 0xFF, dtype=torch.uint8, device=dev)
        sc = torch.full((t,), float("nan"), dtype=torch.float32, device=dev)
        call = _capi.make_problem(_capi.BF16, n, t, h, 1e-5, quant=_capi.QUANT_FP8_TOKEN, workgroups_per_cu=limit)
        _capi.reduce_rms(call, [p.data_ptr() for p in parts], res.data_ptr(), res_out.data_ptr(), gamma.data_ptr(),
                         q_out=q.data_ptr(), scale_out=sc.data_ptr(), stream=torch.cuda.current_stream(dev).cuda_stream)
        torch.cuda.synchronize(dev)
        outs.append((res_out, q, sc))
    for a, b in zip(*outs):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    acc = torch.zeros((t, h), device=dev)
    for p in parts:
        acc = acc + p.float()
    x = (acc.to(torch.bfloat16).float() + res.float()).to(torch.bfloat16)
    assert torch.equal(outs[0][0].view(torch.int16), x.view(torch.int16))
    assert torch.all(outs[0][1].view(torch.float8_e4m3fn).float().abs().amax(-1) == 448.0)


def test_full_size_c3_properties(cuda_device):
    """Configuration c3 at full size on the device only (the CPU oracle is not run at this size here):
    size-independent properties of the outputs."""
    dev = cuda_device
    gen = torch.Generator(device=dev).manual_seed(3)
    N, T, H = 8, 2048, 8192
    parts = [(torch.randn((T, H), generator=gen, device=dev) * 0.5).to(torch.bfloat16) for _ in range(N)]
    res = torch.randn((T, H), generator=gen, device=dev).to(torch.bfloat16)
    gamma = (torch.rand((H,), generator=gen, device=dev) + 0.5).to(torch.bfloat16)
    import torch_dist_ext_amd as tde
    out = tde.reduce_rms(parts, res, gamma, 1e-5, tde.QUANT_FP8_TOKEN, write_norm=True)
    torch.cuda.synchronize()
    # residual: the same fp32 rank-order sum written with torch ops on the device
    acc = torch.zeros((T, H), device=dev)
    for p in parts:
        acc = acc + p.float()
    x = (acc.to(torch.bfloat16).float() + res.float()).to(torch.bfloat16)
    assert torch.equal(out["residual_out"].view(torch.int16), x.view(torch.int16))
    # the remaining checks run on the host: torch's device division by a Python scalar multiplies by
    # a reciprocal and is not the IEEE quotient
    y = out["norm_out"].float().cpu()
    scale = out["scale"].cpu()
    assert torch.equal(scale, y.abs().amax(-1) / 448.0)                           # scale is amax/448 of the written rows
    q = out["q"].cpu().float()
    assert torch.all(q.abs().amax(-1) == 448.0)                                   # top code reached in every row
    rms = torch.sqrt((y / gamma.float().cpu()).pow(2).mean(-1))
    assert torch.all((rms - 1).abs() < 0.02)                                      # rows are normalized
    # the codes are the oracle's quantizer applied to the written rows, bit for bit
    q_own, s_own = eager.quant_fp8(out["norm_out"].cpu(), None)
    assert torch.equal(q_own.view(torch.uint8), out["q"].cpu().view(torch.uint8)) and torch.equal(s_own, scale)
    # idempotence of the epilogue: re-quantizing the dequantized row with the same scale gives the same codes
    deq = q * scale.view(-1, 1)
    q2 = (deq / scale.view(-1, 1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    assert torch.equal(q2.view(torch.uint8), out["q"].cpu().view(torch.uint8))
    # determinism: a second launch on the same inputs writes the same bits
    out2 = tde.reduce_rms(parts, res, gamma, 1e-5, tde.QUANT_FP8_TOKEN, write_norm=True)
    for k in out:
        assert torch.equal(out[k].view(torch.uint8), out2[k].view(torch.uint8)), k         # deterministic run to run


def _device_inputs(dev, n, t, h, dtype, sigma, seed, outliers=0):
    gen = torch.Generator(device=dev).manual_seed(seed)
    parts = []
    cols = torch.randperm(h, generator=torch.Generator().manual_seed(seed))[:outliers].to(dev) if outliers else None
    for _ in range(n):
        p = torch.randn((t, h), generator=gen, device=dev) * sigma
        if cols is not None:
            p[:, cols] *= 100.0
        parts.append(p.to(dtype))
    res = torch.randn((t, h), generator=gen, device=dev).to(dtype)
    gamma = (torch.rand((h,), generator=gen, device=dev) + 0.5).to(dtype)
    return parts, res, gamma


def _device_residual(parts, res):
    acc = torch.zeros(res.shape, device=res.device)
    for p in parts:
        acc = acc + p.float()
    return (acc.to(res.dtype).float() + res.float()).to(res.dtype)


@pytest.mark.parametrize("name,n,t,h,dtype,sigma,eps,quant,outliers", [
    ("c4", 4, 8192, 7168, torch.bfloat16, 1.0, 1e-6, "fp8_group", 0),
    ("c5@32768", 4, 32768, 5120, torch.float16, 1.0, 1e-6, "int8_token", 5),
])
def test_full_size_c4_c5_properties(cuda_device, name, n, t, h, dtype, sigma, eps, quant, outliers):
    """Configurations c4 and the largest c5 at full size.  Inputs are drawn on the device; the residual is checked
    against the same rank-order sum written with torch device ops, and the quant epilogue against the oracle's
    quantizer applied on the host to a band of the written normed rows (the whole tensor for the scales)."""
    import torch_dist_ext_amd as tde
    print("case", name, flush=True)
    parts, res, gamma = _device_inputs(cuda_device, n, t, h, dtype, sigma, seed=t, outliers=outliers)
    mode = {"fp8_group": tde.QUANT_FP8_GROUP, "int8_token": tde.QUANT_INT8_TOKEN}[quant]
    out = tde.reduce_rms(parts, res, gamma, eps, mode, write_norm=True)
    torch.cuda.synchronize()
    assert torch.equal(out["residual_out"].view(torch.int16), _device_residual(parts, res).view(torch.int16))
    del parts
    y = out["norm_out"]
    qmax = 127.0 if quant == "int8_token" else 448.0
    grp = h if quant == "int8_token" else 128
    amax = y.float().abs().view(t, h // grp, grp).amax(-1).cpu()
    assert torch.equal(out["scale"].cpu().view(t, -1), amax / qmax)          # host division: IEEE quotient
    band = slice(t // 2, t // 2 + 256)
    yb = y[band].cpu()
    if quant == "int8_token":
        q_own, s_own = eager.quant_int8(yb)
    else:
        q_own, s_own = eager.quant_fp8(yb, 128)
    assert bits_equal(q_own, out["q"][band].cpu()) and bits_equal(s_own.reshape(-1), out["scale"][band].cpu().reshape(-1))
    # every row/group with a non-zero maximum reaches the top code
    top = out["q"].view(torch.int8 if quant == "int8_token" else torch.float8_e4m3fn).float().abs().view(t, h // grp, grp).amax(-1)
    assert torch.all((top == qmax) | (out["scale"].view(t, -1) == 0))
    # rows are normalized: rms(norm/gamma) ~ 1 (second rounding and fp16/bf16 precision allow a small band)
    rms = torch.sqrt((y.float() / gamma.float()).pow(2).mean(-1))
    assert torch.all((rms - 1).abs() < 0.02)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("scale", [0.0078125, 0.013, 1.7])
def test_static_scale_fp8(cuda_device, dtype, scale):
    """Caller-given per-tensor scale: codes must be the oracle's static quantizer applied to the kernel's own
    normed rows, bit for bit (values beyond 448*scale saturate to the top code)."""
    p, r, g = eager.make_inputs(4, 45, 2048, dtype, 1.0, seed=41)
    print("case static", dtype, scale, flush=True)
    want = eager.reduce_rms(p, r, g, 1e-6, "fp8_static", static_scale=scale)
    got = run_hip(p, r, g, 1e-6, "fp8_static", static_scale=scale)
    assert "scale" not in got
    check_against_oracle({k: got[k] for k in ("residual_out", "norm_out")}, want, "none", gamma=g, eps=1e-6)
    assert bits_equal(got["q"], eager.quant_fp8_static(got["norm_out"], scale))
    assert bits_equal(got["q"], want["q"])
    got2 = run_hip(p, r, g, 1e-6, "fp8_static", static_scale=scale, write_norm=False)
    assert bits_equal(got2["q"], got["q"])


@pytest.mark.parametrize("dtype,gscale,scale", [(torch.float32, 1e30, 1e-9), (torch.bfloat16, 1e30, 1e-9), (torch.float32, 1e25, 3e-17)])
def test_static_scale_quotient_beyond_fp32_range(cuda_device, dtype, gscale, scale):
    """Normed values around 1e30 (or 1e25) divided by a static scale of 1e-9 (3e-17) leave the fp32 range: the codes
    must saturate with the value's own sign (0x7E / 0xFE), exactly as the oracle's clamp does."""
    p, r, g = eager.make_inputs(4, 9, 1024, torch.float32, 1.0, seed=43)
    p, r, g = p.to(dtype), r.to(dtype), (g * gscale).to(dtype)
    want = eager.reduce_rms(p, r, g, 1e-6, "fp8_static", static_scale=scale)
    got = run_hip(p, r, g, 1e-6, "fp8_static", static_scale=scale)
    assert bits_equal(got["norm_out"], want["norm_out"])
    assert bits_equal(got["q"], want["q"])
    codes = got["q"].view(torch.uint8)
    nonzero = want["norm_out"].float() != 0
    assert bool(((codes[nonzero] & 0x7F) == 0x7E).all())
    assert bool(((codes >> 7).bool() == (want["norm_out"].float() < 0))[nonzero].all())


def test_static_scale_is_validated(cuda_device):
    p, r, g = eager.make_inputs(2, 4, 256, torch.bfloat16, 1.0, seed=42)
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(_capi.TdeError) as e:
            run_hip(p, r, g, 1e-6, "fp8_static", static_scale=bad)
        assert e.value.status == _capi.EQUANT


def test_first_large_lds_launch_inside_a_capture(cuda_device):
    """The first launch of a kernel with more than 64 KiB of dynamic LDS raises that kernel's ceiling (a function
    attribute, not a stream operation).  No other test launches this instantiation (fp32, 2 partials, int8) with such a
    size, so here that happens while the stream is being captured; the graph must still be valid and right."""
    dev = cuda_device
    n, t, h = 2, 64, 2048
    cp, cr, cg = eager.make_inputs(n, t, h, torch.float32, 1.0, seed=5)
    parts = [p.to(dev) for p in cp]
    res, gamma = cr.to(dev), cg.to(dev)
    res_out = torch.empty_like(res)
    q = torch.empty((t, h), dtype=torch.uint8, device=dev)
    sc = torch.empty((t,), dtype=torch.float32, device=dev)
    prob = _capi.make_problem(_capi.F32, n, t, h, 1e-6, quant=_capi.QUANT_INT8_TOKEN, workgroups_per_cu=1)
    assert _capi.plan(prob).lds_bytes > 64 * 1024
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _capi.reduce_rms(prob, [p.data_ptr() for p in parts], res.data_ptr(), res_out.data_ptr(), gamma.data_ptr(),
                         q_out=q.data_ptr(), scale_out=sc.data_ptr(), stream=torch.cuda.current_stream().cuda_stream)
    want = eager.reduce_rms(cp, cr, cg, 1e-6, "int8_token")
    for _ in range(2):
        for v in (res_out, q, sc):
            v.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = {"residual_out": res_out.cpu(), "q": q.cpu().view(torch.int8), "scale": sc.cpu()}
        check_against_oracle(got, want, "int8_token", gamma=cg, eps=1e-6)


def test_hip_graph_replays_with_a_workgroup_limit(cuda_device):
    """A launch limited to two workgroups per CU asks for 79 KiB of dynamic LDS (the kernel's ceiling is raised by the
    eager warm-up call, before the capture): the captured launch keeps that size and replays with new inputs match the oracle."""
    dev = cuda_device
    n, t, h = 4, 96, 7168
    parts = [torch.empty((t, h), dtype=torch.float16, device=dev) for _ in range(n)]
    res = torch.empty((t, h), dtype=torch.float16, device=dev)
    gamma = torch.empty((h,), dtype=torch.float16, device=dev)
    res_out = torch.empty_like(res)
    q = torch.empty((t, h), dtype=torch.uint8, device=dev)
    sc = torch.empty((t, h // 128), dtype=torch.float32, device=dev)
    prob = _capi.make_problem(_capi.F16, n, t, h, 1e-6, quant=_capi.QUANT_FP8_GROUP, workgroups_per_cu=2)
    assert _capi.plan(prob).lds_bytes > 64 * 1024

    def launch(stream):
        _capi.reduce_rms(prob, [p.data_ptr() for p in parts], res.data_ptr(), res_out.data_ptr(), gamma.data_ptr(),
                         q_out=q.data_ptr(), scale_out=sc.data_ptr(), stream=stream)

    def fill(seed):
        cp, cr, cg = eager.make_inputs(n, t, h, torch.float16, 1.0, seed=seed)
        for i in range(n):
            parts[i].copy_(cp[i])
        res.copy_(cr)
        gamma.copy_(cg)
        return cp, cr, cg

    fill(41)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(torch.cuda.current_stream().cuda_stream)
    for seed in (42, 43, 44):
        cp, cr, cg = fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = {"residual_out": res_out.cpu(), "q": q.cpu().view(torch.float8_e4m3fn), "scale": sc.cpu()}
        for v in (res_out, q, sc):
            v.zero_()                        # eager work between replays
        torch.cuda.synchronize()
        check_against_oracle(got, eager.reduce_rms(cp, cr, cg, 1e-6, "fp8_group"), "fp8_group", gamma=cg, eps=1e-6)


@pytest.mark.parametrize("algo", [_capi.ALGO_FUSED, _capi.ALGO_STAGED, _capi.ALGO_STAGED_OWNED])
def test_hip_graph_replays_match_eager(cuda_device, algo):
    """The launch allocates nothing and synchronizes nothing, so it can be captured (the staged algorithms:
    both launches in one graph).  Replays are checked against eager launches, with new input contents and
    eager work between the replays."""
    dev = cuda_device
    n, t, h = 8, 128, 4096
    stage = torch.empty((t, h), dtype=torch.bfloat16, device=dev) if algo != _capi.ALGO_FUSED else None
    parts = [torch.empty((t, h), dtype=torch.bfloat16, device=dev) for _ in range(n)]
    res = torch.empty((t, h), dtype=torch.bfloat16, device=dev)
    gamma = torch.empty((h,), dtype=torch.bfloat16, device=dev)
    outs = {k: torch.empty((t, h), dtype=torch.bfloat16, device=dev) for k in ("res_out", "norm")}
    q = torch.empty((t, h), dtype=torch.uint8, device=dev)
    sc = torch.empty((t,), dtype=torch.float32, device=dev)
    prob = _capi.make_problem(_capi.BF16, n, t, h, 1e-5, quant=_capi.QUANT_FP8_TOKEN, write_norm=1, algo=algo)

    def launch(stream):
        if algo == _capi.ALGO_STAGED_OWNED:       # all N ranks' shares, then the norm: the whole two-shot
            for k in range(n):
                pk = _capi.make_problem(_capi.BF16, n, t, h, 1e-5, quant=_capi.QUANT_FP8_TOKEN, write_norm=1, algo=algo, rank=k)
                _capi.reduce_rms(pk, [p.data_ptr() for p in parts], None, None, None, stage=stage.data_ptr(), stream=stream,
                                 phases=("reduce",))
            _capi.reduce_rms(prob, [None] * n, res.data_ptr(), outs["res_out"].data_ptr(), gamma.data_ptr(),
                             norm_out=outs["norm"].data_ptr(), q_out=q.data_ptr(), scale_out=sc.data_ptr(),
                             stage=stage.data_ptr(), stream=stream, phases=("norm",))
            return
        _capi.reduce_rms(prob, [p.data_ptr() for p in parts], res.data_ptr(), outs["res_out"].data_ptr(), gamma.data_ptr(),
                         norm_out=outs["norm"].data_ptr(), q_out=q.data_ptr(), scale_out=sc.data_ptr(),
                         stage=stage.data_ptr() if stage is not None else None, stream=stream)

    def fill(seed):
        cp, cr, cg = eager.make_inputs(n, t, h, torch.bfloat16, 0.5, seed=seed)
        for i in range(n):
            parts[i].copy_(cp[i])
        res.copy_(cr)
        gamma.copy_(cg)
        return cp, cr, cg

    fill(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(side.cuda_stream)            # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(torch.cuda.current_stream().cuda_stream)
    for seed in (2, 3, 4):
        cp, cr, cg = fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = {"residual_out": outs["res_out"].cpu(), "norm_out": outs["norm"].cpu(),
               "q": q.cpu().view(torch.float8_e4m3fn), "scale": sc.cpu()}
        for v in (outs["res_out"], outs["norm"], q, sc):
            v.zero_()                        # eager work between replays
        launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert bits_equal(outs["res_out"].cpu(), got["residual_out"]) and bits_equal(outs["norm"].cpu(), got["norm_out"])
        assert bits_equal(q.cpu(), got["q"].view(torch.uint8)) and bits_equal(sc.cpu(), got["scale"])
        check_against_oracle(got, eager.reduce_rms(cp, cr, cg, 1e-5, "fp8_token"), "fp8_token", gamma=cg, eps=1e-5)


@pytest.mark.parametrize("quant", ["none", "fp8_token", "fp8_group", "int8_token"])
@pytest.mark.parametrize("dtype,hidden", [(torch.float16, 8192), (torch.float32, 4096), (torch.bfloat16, 7168), (torch.float32, 3584)])
@pytest.mark.parametrize("n", [2, 4, 8])
def test_long_rows_every_dtype(cuda_device, dtype, hidden, quant, n):
    """Rows of 896..1024 vectors take the 4-vectors-per-thread kernels once there are many rows; cover them
    for every dtype, mode and number of partials (forced here, the input has few rows): with four and eight
    partials these are the kernels that sum rank by rank while the loads arrive."""
    p, r, g = eager.make_inputs(n, 19, hidden, dtype, 1.0, seed=hidden + 3 + n)
    code = {torch.float16: _capi.F16, torch.float32: _capi.F32, torch.bfloat16: _capi.BF16}[dtype]
    assert _capi.plan(_capi.make_problem(code, n, 4096, hidden, 1e-6)).vecs_per_thread == 4
    assert _capi.plan(_capi.make_problem(code, n, 19, hidden, 1e-6)).vecs_per_thread == 1
    _case("long-rows", p, r, g, 1e-6, quant, vecs_per_thread=4)


def test_randomized_shapes_and_modes(cuda_device):
    """Seeded sweep over random (dtype, N, tokens, hidden, mode) combinations, small enough for the CPU oracle:
    exercises row packing, partly filled wavefronts and every kernel family in one go."""
    rng = torch.Generator().manual_seed(2024)
    dtypes = [torch.bfloat16, torch.float16, torch.float32]
    modes = ["none", "fp8_token", "fp8_group", "int8_token"]
    done = 0
    for _ in range(64):
        dtype = dtypes[int(torch.randint(0, 3, (1,), generator=rng))]
        n = [2, 4, 8][int(torch.randint(0, 3, (1,), generator=rng))]
        tokens = int(torch.randint(1, 70, (1,), generator=rng))
        vec = 4 if dtype == torch.float32 else 8
        nvec = int(torch.randint(1, 1025, (1,), generator=rng))
        quant = modes[int(torch.randint(0, 4, (1,), generator=rng))]
        hidden = nvec * vec
        if quant == "fp8_group":
            hidden = max(128, hidden // 128 * 128)
        p, r, g = eager.make_inputs(n, tokens, hidden, dtype, 1.0, seed=1000 + done)
        _case("fuzz%d" % done, p, r, g, 1e-6, quant)
        done += 1
    assert done == 64


def test_randomized_launch_geometries(cuda_device):
    """The same kind of sweep with the launch forced at random as well: vectors per thread, rows per workgroup, the
    limit on workgroups per CU (with and without more than 64 KiB of LDS), the algorithm and the extra normed output."""
    rng = torch.Generator().manual_seed(77)

    def pick(seq):
        return seq[int(torch.randint(0, len(seq), (1,), generator=rng))]

    for k in range(48):
        dtype = pick([torch.bfloat16, torch.float16, torch.float32])
        n = pick([2, 4, 8])
        tokens = int(torch.randint(1, 50, (1,), generator=rng))
        vec = 4 if dtype == torch.float32 else 8
        quant = pick(["none", "fp8_token", "fp8_group", "int8_token"])
        hidden = int(torch.randint(1, 1025, (1,), generator=rng)) * vec
        if quant == "fp8_group":
            hidden = max(128, hidden // 128 * 128)
        kw = dict(vecs_per_thread=pick([0, 1, 2, 4]), rows_per_block=pick([0, 0, 1, 2, 4]),
                  workgroups_per_cu=pick([0, -1, 1, 2, 3, 5, 8]), algo=pick([_capi.ALGO_AUTO, _capi.ALGO_AUTO, _capi.ALGO_STAGED]),
                  write_norm=pick([True, False]))
        p, r, g = eager.make_inputs(n, tokens, hidden, dtype, 1.0, seed=2000 + k)
        print("geometry fuzz", k, dtype, n, tokens, hidden, quant, kw, flush=True)
        _case("geofuzz%d" % k, p, r, g, 1e-6, quant, **kw)


@pytest.mark.parametrize("quant", ["none", "fp8_token", "fp8_group", "int8_token", "fp8_static"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hidden,vpt", [(256, 0), (2048, 1), (8192, 4), (4096, 2)])
def test_nonfinite_rows(cuda_device, dtype, quant, hidden, vpt):
    """NaN, +inf and -inf in a partial, in the residual and in gamma: the eager composition (test/test_all_reduce_fusion.py:
    23-28,75) is made of NaN-propagating torch ops, and so are amax and clamp in the quantizer.  A NaN anywhere in a row
    makes the whole normed row NaN and its scale NaN; an infinity makes the reciprocal RMS zero, the infinite elements
    NaN and the rest zero; gamma's NaN and infinities reach only their own columns (and their group's or row's scale).
    The kernel's outputs must be the oracle's with NaN matching NaN."""
    if dtype == torch.float32 and hidden > 4096:
        hidden = 4096
    p, r, g = eager.make_inputs(4, 12, hidden, dtype, 0.5, seed=401 + hidden)
    last = hidden - 1
    p[1, 0, 5] = float("nan")          # one NaN in the first wavefront's part of the row
    p[2, 1, last - 3] = float("inf")   # +inf in the last wavefront's part
    p[0, 2, hidden // 2] = float("-inf")
    r[3, 11] = float("nan")
    r[4, 3] = float("inf")
    p[3, 5, 7] = float("inf")
    p[1, 5, 7] = float("-inf")         # inf - inf in the reduction
    p[0, 6, 130 % hidden] = float("inf")
    r[6, 130 % hidden] = float("-inf")  # inf - inf in the residual add
    # rows 7.. stay finite
    for gamma_case in ("finite", "special"):
        gamma = g.clone()
        if gamma_case == "special":
            gamma[100] = float("nan")
            gamma[hidden - 126] = float("inf")
            gamma[hidden - 60] = float("-inf")
            gamma[17] = -1.0
        static_scale = 0.0123 if quant == "fp8_static" else None
        want = eager.reduce_rms(p, r, gamma, 1e-5, quant, static_scale=static_scale)
        got = run_hip(p, r, gamma, 1e-5, quant, vecs_per_thread=vpt, static_scale=static_scale or 0.0)
        check_nonfinite(got, want, quant)
        # the finite rows with finite gamma are ordinary rows: bit for bit, no NaN anywhere
        if gamma_case == "finite":
            assert not torch.isnan(got["norm_out"][7:].float()).any()
            assert bits_equal(got["norm_out"][7:], want["norm_out"][7:])
            assert torch.isnan(got["norm_out"][:7].float()).any(dim=1).all()


@pytest.mark.parametrize("quant", ["fp8_token", "fp8_group", "int8_token", "fp8_static"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_negative_gamma_and_the_sign_of_zero(cuda_device, dtype, quant):
    """Negative gamma on a zero element gives a normed -0, whose e4m3 code is 0x80, not 0x00: the quotient has to
    keep the sign of a zero numerator.  Also rows that are zero throughout with mixed-sign gamma."""
    p, r, g = eager.make_inputs(4, 9, 1024, dtype, 0.5, seed=77)
    g[::3] = -g[::3]
    p[:, :, 40:48] = 0.0
    r[:, 40:48] = 0.0       # zero elements under both signs of gamma (columns 42 and 45 are negative)
    p[:, 4] = 0.0
    r[4] = 0.0              # an all-zero row: scale 0, codes +-0
    static_scale = 0.05 if quant == "fp8_static" else None
    want = eager.reduce_rms(p, r, g, 1e-5, quant, static_scale=static_scale)
    got = run_hip(p, r, g, 1e-5, quant, static_scale=static_scale or 0.0)
    assert bits_equal(got["norm_out"], want["norm_out"])
    assert (want["norm_out"].view(torch.int16 if dtype != torch.float32 else torch.int32)[:, 42] < 0).any()   # a -0 is there
    assert bits_equal(got["q"], want["q"]), "codes differ (sign of zero?)"
    if quant != "fp8_static":
        assert bits_equal(got["scale"].reshape(-1), want["scale"].reshape(-1))
    if quant.startswith("fp8"):
        assert (got["q"].view(torch.uint8) == 0x80).any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("scale", [1e-30, 3e-39, 1e-6, 1e4])
def test_extreme_magnitudes(cuda_device, dtype, scale):
    """Very small (down to fp32 subnormals) and large inputs: the reduce and the residual add stay bit-exact,
    i.e. the kernel neither flushes subnormals nor rounds differently near the ends of the range."""
    if dtype == torch.float16 and scale < 1e-6:
        scale = 6e-8 * (1 if scale < 1e-30 else 40)     # fp16 subnormal range
    if dtype == torch.float16 and scale > 100:
        scale = 2000.0                                    # sums reach past 65504: rounds to inf in both
    p, r, g = eager.make_inputs(4, 9, 512, torch.float32, 1.0, seed=61)
    p, r = (p * scale).to(dtype), (r * scale).to(dtype)
    g = g.to(dtype)
    want = eager.reduce_rms(p, r, g, 1e-6)
    got = run_hip(p, r, g, 1e-6, "none")
    assert bits_equal(got["residual_out"], want["residual_out"])
    finite = torch.isfinite(want["norm_out"].float()) & torch.isfinite(got["norm_out"].float())
    assert bool((torch.isfinite(want["norm_out"].float()) == torch.isfinite(got["norm_out"].float())).all())
    from helpers import ulp_distance as _ud
    d = _ud(got["norm_out"], want["norm_out"])[finite]
    assert d.numel() == 0 or int(d.max()) <= (8 if dtype == torch.float32 else 2)


@pytest.mark.parametrize("quant", ["fp8_token", "fp8_group", "int8_token"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("gscale", [1e-30, 1e25])
def test_quant_with_scales_outside_the_fast_division_range(cuda_device, dtype, quant, gscale):
    """gamma of 1e-30 / 1e25 pushes the dynamic scale below 2^-60 / above 2^60, where the kernel leaves its
    reciprocal-based quotient for a plain division: codes and scales must still be the oracle's, bit for bit."""
    p, r, g = eager.make_inputs(4, 11, 1024, torch.float32, 1.0, seed=71)
    p, r, g = p.to(dtype), r.to(dtype), (g * gscale).to(dtype)
    _case("tiny-scale", p, r, g, 1e-6, quant)


@pytest.mark.parametrize("key", ["c2", "c3", "c4", "c5@4096"])
def test_full_size_outputs_match_committed_digests(cuda_device, key):
    """Every output is bit-exact: the SHA-256 of residual_out, norm_out, codes and scales at full size must equal
    the digests the CPU oracle produced when tests/golden/digests.json was written (inputs regenerate from
    their seeds; the case is skipped if this host's torch generates different inputs)."""
    import hashlib
    import json
    with open(os.path.join(os.path.dirname(__file__), "golden", "digests.json")) as f:
        want = json.load(f)[key]
    name, _, tok = key.partition("@")
    p, r, g, eps, quant = eager.make_config(name, tokens=int(tok) if tok else None)

    def sha(*ts):
        h = hashlib.sha256()
        for t in ts:
            h.update(t.contiguous().view(torch.uint8).numpy().tobytes())
        return h.hexdigest()
    if sha(p, r, g) != want["inputs"]:
        pytest.skip("this host's torch generates different inputs from the same seeds")
    out = run_hip(p, r, g, eps, quant)
    assert sha(out["residual_out"]) == want["residual_out"]
    assert sha(out["norm_out"]) == want["norm_out"]
    if quant != "none":
        assert sha(out["q"]) == want["q"]
        assert sha(out["scale"]) == want["scale"]


def test_device_info(cuda_device):
    info = _capi.device_info()
    assert info.compute_units == torch.cuda.get_device_properties(0).multi_processor_count
    assert info.total_memory_bytes == torch.cuda.get_device_properties(0).total_memory
    assert info.memory_clock_khz >= 0 and info.memory_bus_bits >= 0


@pytest.mark.parametrize("n,tokens,hidden,dtype,quant,write_norm", [
    (8, 70, 4096, torch.bfloat16, "fp8_token", False), (4, 33, 1024, torch.float16, "none", True),
    (2, 300, 8192, torch.bfloat16, "int8_token", True), (4, 19, 508, torch.float32, "fp8_token", False),
])
def test_traffic_skeleton_touches_every_byte_once(cuda_device, n, tokens, hidden, dtype, quant, write_norm):
    """tde_probe_rows reads every input vector and writes every output vector: its outputs are the
    exclusive-or of all N+1 input rows (16 bytes at a time), folded to 8 or 4 bytes for the code rows."""
    p, r, g = eager.make_inputs(n, tokens, hidden, dtype, 1.0, seed=77)
    out = run_hip(p, r, g, 1e-6, quant, write_norm=write_norm, calls=[(("traffic",), 0)])
    words = lambda t: t.contiguous().view(torch.int32).reshape(tokens, -1, 4)
    x = words(r).clone()
    for k in range(n):
        x ^= words(p[k])
    assert torch.equal(words(out["residual_out"]), x)
    if write_norm or quant == "none":
        assert torch.equal(words(out["norm_out"]), x)
    if quant != "none":
        q = out["q"].contiguous().view(torch.uint8).view(torch.int32)
        if dtype == torch.float32:
            assert torch.equal(q.reshape(tokens, -1), x[..., 0] ^ x[..., 1] ^ x[..., 2] ^ x[..., 3])
        else:
            assert torch.equal(q.reshape(tokens, -1, 2), torch.stack([x[..., 0] ^ x[..., 2], x[..., 1] ^ x[..., 3]], dim=-1))


@pytest.mark.parametrize("n,tokens,hidden", [(2, 33, 1024), (4, 129, 2048), (8, 7, 258), (8, 300, 2), (4, 1000, 1536)])
def test_doubles(cuda_device, n, tokens, hidden):
    """double rows (the reference's dtype macro admits them, src/ops/all_reduce_fusion.cpp:29-33): the sum,
    the residual add and the scaling are done in double as eager does for double tensors; only the mean of
    squares is fp32 (test/test_all_reduce_fusion.py:25).  residual_out bit-exact, normed rows bit-identical
    to the composition for a reciprocal RMS within 4 fp32 ulps."""
    p, r, g = eager.make_inputs(n, tokens, hidden, torch.float64, 1.0, seed=600 + n)
    assert p.dtype == torch.float64 and (p.view(torch.int64) & 0xFFFFFFF).ne(0).any()   # real doubles, not widened floats
    _case("f64", p, r, g, 1e-6, "none")
    _case("f64 table", p, r, g, 1e-6, "none", use_table=True, rank=1)


@pytest.mark.parametrize("n,tokens,hidden", [(2, 33, 1024), (4, 129, 2048), (8, 7, 258), (4, 1000, 1536)])
def test_doubles_through_the_staged_algorithms(cuda_device, n, tokens, hidden):
    """The reference sends doubles through either of its kernels (src/ops/all_reduce_fusion.cpp:29-33,
    all_reduce_fusion_impl.h:491): the two-launch structure for doubles -- all rows staged, this rank's rows staged
    with the others delivered, and the N + 1 phase calls -- against the oracle, and bit-identical to the fused kernel."""
    p, r, g = eager.make_inputs(n, tokens, hidden, torch.float64, 1.0, seed=650 + n)
    fused, want, _ = _case("f64 fused", p, r, g, 1e-6, "none")
    staged, _, _ = _case("f64 staged", p, r, g, 1e-6, "none", algo=_capi.ALGO_STAGED)
    sums = torch.zeros((tokens, hidden), dtype=torch.float64)
    for k in range(n):
        sums = sums + p[k]
    init = sums.clone()
    init[1::n] = float("nan")
    owned = run_hip(p, r, g, 1e-6, "none", algo=_capi.ALGO_STAGED_OWNED, rank=1, stage_init=init)
    assert bits_equal(owned.pop("stage"), sums)
    calls = [(("reduce",), k) for k in range(n)] + [(("norm",), 0)]
    phased = run_hip(p, r, g, 1e-6, "none", algo=_capi.ALGO_STAGED_OWNED, calls=calls,
                     stage_init=torch.full((tokens, hidden), float("nan"), dtype=torch.float64))
    assert bits_equal(phased.pop("stage"), sums)
    for other in (staged, owned, phased):
        for k in fused:
            assert bits_equal(fused[k], other[k]), k


def test_doubles_limits(cuda_device):
    p, r, g = eager.make_inputs(2, 4, 256, torch.float64, 1.0, seed=1)
    with pytest.raises(_capi.TdeError) as ei:
        run_hip(p, r, g, 1e-6, "fp8_token")
    assert ei.value.status == _capi.EQUANT
    with pytest.raises(_capi.TdeError) as ei:
        run_hip(p, r, g, 1e-6, "none", calls=[(("traffic",), 0)])
    assert ei.value.status == _capi.EDTYPE


@pytest.mark.parametrize("tokens", [1, 7, 63, 64, 65, 127, 128, 129, 255, 257, 1000, 1029])
@pytest.mark.parametrize("n", [4, 8])
def test_row_mapping_covers_every_row_once(cuda_device, n, tokens):
    """Workgroups take row groups in XCD-sized chunks (groups of 64 or 128 workgroups, launch order in the
    tail): with every grid size around those group sizes, and with one and several rows per workgroup, each
    row is produced exactly once (outputs start as NaN bytes; the traffic skeleton's exclusive-or output is
    checked the same way)."""
    p, r, g = eager.make_inputs(n, tokens, 512, torch.bfloat16, 1.0, seed=tokens)
    want = eager.reduce_rms(p, r, g, 1e-6, "fp8_token")
    for rows_per_block in (0, 1, 4):
        got = run_hip(p, r, g, 1e-6, "fp8_token", rows_per_block=rows_per_block)
        sk = run_hip(p, r, g, 1e-6, "fp8_token", write_norm=False, calls=[(("traffic",), 0)], rows_per_block=rows_per_block)
        check_against_oracle(got, want, "fp8_token", gamma=g, eps=1e-6)
        x = r.contiguous().view(torch.int32).clone()
        for k in range(n):
            x ^= p[k].contiguous().view(torch.int32)
        assert torch.equal(sk["residual_out"].view(torch.int32), x)


def test_stream_probe(cuda_device):
    n = 1 << 20
    src = torch.empty(n + 16, dtype=torch.uint8, device=cuda_device).random_(0, 255)
    dst = torch.zeros(n + 16, dtype=torch.uint8, device=cuda_device)
    st = torch.cuda.current_stream().cuda_stream
    _capi.probe_stream(dst.data_ptr(), src.data_ptr(), n - 48, 2, st)          # copy, ragged last workgroup
    torch.cuda.synchronize()
    assert torch.equal(dst[:n - 48], src[:n - 48]) and int(dst[n - 48:].sum()) == 0
    dst.zero_()
    _capi.probe_stream(dst.data_ptr(), src.data_ptr(), n, 0, st)               # read only: nothing written
    torch.cuda.synchronize()
    assert int(dst.sum()) == 0
    _capi.probe_stream(dst.data_ptr(), src.data_ptr(), n, 1, st)               # write only: every vector written
    torch.cuda.synchronize()
    words = dst[:n].view(torch.int32).view(-1, 4)
    assert bool((words[:, 2] == 0x9e3779b9 - (1 << 32)).all()) and int(dst[n:].sum()) == 0
    with pytest.raises(_capi.TdeError):
        _capi.probe_stream(dst.data_ptr(), src.data_ptr(), n, 3, st)


GOLDEN_SHA256 = "e826e121639af71fc57b0b02599d943982c2f8cf9e32c75497e5af8e639b1997"


@pytest.mark.parametrize("name", ["c1", "q_fp8_token", "q_fp8_group", "q_int8_token"])
def test_committed_golden_fixtures_through_the_kernel(cuda_device, name):
    """tests/golden/golden.npz (inputs and the oracle's outputs, committed) fed through tde_reduce_rms: every stored
    output must come back bit for bit.  The file itself is pinned by its SHA-256, so an edited fixture fails here
    rather than redefining the expected values."""
    import hashlib
    import numpy as np
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden.npz")
    with open(path, "rb") as f:
        assert hashlib.sha256(f.read()).hexdigest() == GOLDEN_SHA256, "tests/golden/golden.npz was altered"
    d = np.load(path)
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16}[str(d[name + "/dtype"])]
    quant, eps = str(d[name + "/quant"]), float(d[name + "/eps"])

    def t16(a):
        return torch.from_numpy(a.view(np.int16).copy()).view(dtype)

    parts, residual, gamma = t16(d[name + "/parts"]), t16(d[name + "/residual"]), t16(d[name + "/gamma"])
    print("golden case", name, tuple(parts.shape), dtype, quant, flush=True)
    got = run_hip(parts, residual, gamma, eps, quant)
    assert bits_equal(got["residual_out"], t16(d[name + "/residual_out"]))
    assert bits_equal(got["norm_out"], t16(d[name + "/norm_out"]))
    if quant != "none":
        assert np.array_equal(got["q"].view(torch.uint8).numpy(), d[name + "/q"])
        assert np.array_equal(got["scale"].numpy().view(np.uint32), d[name + "/scale"].view(np.uint32))


def test_more_than_2_to_the_31_elements_per_buffer(cuda_device):
    """270 000 rows of 8192 bf16 are 2.2e9 elements and 4.4 GB per buffer: byte offsets and element counts beyond
    32 bits (the reference indexes with int, src/common/all_reduce_fusion_impl.h:304).  The rows at the start, around
    element 2^31 (row 262 144) and at the end must equal what the same kernel computes for those rows alone, which in
    turn is checked against the oracle."""
    n, t, h, eps = 2, 270000, 8192, 1e-5
    dev = cuda_device
    gen = torch.Generator(device=dev).manual_seed(5)
    parts = []
    for _ in range(n):
        p = torch.empty((t, h), dtype=torch.bfloat16, device=dev)
        for lo in range(0, t, 30000):       # in pieces: no fp32 copy of the whole buffer
            hi = min(t, lo + 30000)
            p[lo:hi] = (torch.randn((hi - lo, h), generator=gen, device=dev) * 0.5).to(torch.bfloat16)
        parts.append(p)
    res = torch.empty((t, h), dtype=torch.bfloat16, device=dev)
    for lo in range(0, t, 30000):
        hi = min(t, lo + 30000)
        res[lo:hi] = torch.randn((hi - lo, h), generator=gen, device=dev).to(torch.bfloat16)
    gamma = (torch.rand((h,), generator=gen, device=dev) + 0.5).to(torch.bfloat16)
    res_out = torch.empty_like(res)
    q = torch.empty((t, h), dtype=torch.uint8, device=dev)
    scale = torch.empty((t,), dtype=torch.float32, device=dev)
    for buf in (res_out, q, scale):
        buf.view(torch.uint8).fill_(0xFF)
    stream = torch.cuda.current_stream(dev).cuda_stream
    prob = _capi.make_problem(_capi.BF16, n, t, h, eps, quant=_capi.QUANT_FP8_TOKEN, write_norm=0)
    assert _capi.plan(prob).grid_blocks == t
    print("case 2^31 elements", t, h, flush=True)
    _capi.reduce_rms(prob, [p.data_ptr() for p in parts], res.data_ptr(), res_out.data_ptr(), gamma.data_ptr(),
                     q_out=q.data_ptr(), scale_out=scale.data_ptr(), stream=stream)
    torch.cuda.synchronize(dev)
    boundary = (1 << 31) // h
    for lo, hi in ((0, 40), (boundary - 20, boundary + 20), (t - 40, t)):
        cp = torch.stack([p[lo:hi] for p in parts]).cpu()
        want = eager.reduce_rms(cp, res[lo:hi].cpu(), gamma.cpu(), eps, "fp8_token")
        assert bits_equal(res_out[lo:hi].cpu(), want["residual_out"]), (lo, hi)
        assert bits_equal(q[lo:hi].cpu(), want["q"]), (lo, hi)
        assert bits_equal(scale[lo:hi].cpu(), want["scale"]), (lo, hi)
    # every row was written (no 0xFF fill left in the scales) and rows far apart differ
    assert bool(torch.isfinite(scale).all()) and bool((scale > 0).all())


SUM_ORDER_HIDDEN = {
    # vectors of 8 floats V = hidden // 8: left-over vectors V % 4, left-over scalars hidden % 8, a last block shorter
    # than 16 steps ((V // 4) % 16), no full step at all (V < 4), fewer than 8 floats
    torch.bfloat16: [8, 16, 24, 32, 40, 72, 120, 128, 136, 264, 504, 520, 1032, 2040, 2056, 4104, 6152, 8184],
    torch.float16: [8, 56, 520, 4088],
    torch.float32: [4, 8, 12, 20, 28, 36, 100, 132, 516, 1028, 2052, 4092],
    torch.float64: [2, 4, 6, 8, 10, 14, 18, 66, 130, 1026, 2046],
}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.float64])
def test_sum_of_squares_order_at_every_row_shape(cuda_device, dtype):
    """The kernel's sum of squares follows torch's CPU reduction through every branch of it: left-over vectors and
    scalars, a short last block, rows without a full step, rows shorter than one vector.  Normed rows (and int8 codes
    and scales where the type has them) must be bit-identical to the oracle's at each of these row lengths, with one,
    several and many rows per workgroup."""
    for hidden in SUM_ORDER_HIDDEN[dtype]:
        for rows_per_block in (0, 1):
            p, r, g = eager.make_inputs(2, 37, hidden, dtype, 1.0, seed=hidden)
            quant = "int8_token" if dtype in (torch.bfloat16, torch.float16, torch.float32) else "none"
            print("case sum-order", dtype, hidden, rows_per_block, flush=True)
            want = eager.reduce_rms(p, r, g, 1e-6, quant)
            got = run_hip(p, r, g, 1e-6, quant, rows_per_block=rows_per_block)
            check_against_oracle(got, want, quant, gamma=g, eps=1e-6)


@pytest.mark.parametrize("vecs_per_thread", [0, 1, 2, 4])
def test_fp16_product_is_rounded_twice_like_the_eager_composition(cuda_device, vecs_per_thread):
    """T(x * rs) is an fp32 product rounded to fp32 and then to fp16.  An instruction that multiplies and converts in one
    step rounds the exact product once, which differs where the fp32 product falls on an fp16 rounding boundary.  The
    inputs hold such elements (counted here with an exact float64 product), and the kernel must still match the oracle
    bit for bit."""
    import numpy as np
    p, r, g = eager.make_inputs(4, 192, 5120, torch.float16, 1.0, seed=77)
    want = eager.reduce_rms(p, r, g, 1e-6, "none")
    x = want["residual_out"].float()
    rs = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)
    twice = (x * rs).to(torch.float16)
    once = torch.from_numpy((x.double().numpy() * rs.double().numpy()).astype(np.float16))
    sensitive = int((twice.view(torch.int16) != once.view(torch.int16)).sum())
    print("case fp16 double rounding: %d of %d elements tell the two apart" % (sensitive, x.numel()), flush=True)
    assert sensitive >= 8
    got = run_hip(p, r, g, 1e-6, "none", vecs_per_thread=vecs_per_thread)
    check_against_oracle(got, want, "none", gamma=g, eps=1e-6)


def test_calls_on_two_streams_at_once(cuda_device):
    """The launch keeps no state between calls, so calls on different streams with different outputs may overlap: two
    problems of different shape and mode are launched alternately on two streams, several times over without
    synchronizing in between, and each is then checked against the oracle."""
    dev = cuda_device
    jobs = []
    for seed, (n, t, h, dtype, dcode, quant, qm) in enumerate([
            (8, 512, 8192, torch.bfloat16, _capi.BF16, "fp8_token", _capi.QUANT_FP8_TOKEN),
            (4, 700, 5120, torch.float16, _capi.F16, "int8_token", _capi.QUANT_INT8_TOKEN)]):
        cp, cr, cg = eager.make_inputs(n, t, h, dtype, 0.5, seed=90 + seed)
        d = dict(cp=cp, cr=cr, cg=cg, quant=quant, parts=[p.contiguous().to(dev) for p in cp], res=cr.to(dev), gamma=cg.to(dev),
                 res_out=torch.empty((t, h), dtype=dtype, device=dev), q=torch.empty((t, h), dtype=torch.uint8, device=dev),
                 sc=torch.empty((t,), dtype=torch.float32, device=dev), prob=_capi.make_problem(dcode, n, t, h, 1e-5, quant=qm),
                 stream=torch.cuda.Stream())
        jobs.append(d)
    torch.cuda.synchronize()
    for _ in range(6):
        for d in jobs:
            _capi.reduce_rms(d["prob"], [p.data_ptr() for p in d["parts"]], d["res"].data_ptr(), d["res_out"].data_ptr(),
                             d["gamma"].data_ptr(), q_out=d["q"].data_ptr(), scale_out=d["sc"].data_ptr(),
                             stream=d["stream"].cuda_stream)
    torch.cuda.synchronize()
    for d in jobs:
        q = d["q"].cpu()
        got = {"residual_out": d["res_out"].cpu(), "scale": d["sc"].cpu(),
               "q": q.view(torch.float8_e4m3fn) if d["quant"] == "fp8_token" else q.view(torch.int8)}
        check_against_oracle(got, eager.reduce_rms(d["cp"], d["cr"], d["cg"], 1e-5, d["quant"]), d["quant"], gamma=d["cg"], eps=1e-5)
