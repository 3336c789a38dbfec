"""tde_reduce_rms_static_stage: the staged algorithm with the stage buffer inside the library's device
image, for callers that cannot allocate.  Checked bit for bit against tde_reduce_rms with TDE_ALGO_STAGED
(the existing entry point it is a variant of) on two calls in a row, the second smaller, and against the
oracle; a run of calls leaves the device's free memory unchanged."""
import ctypes

import pytest
import torch

from helpers import bits_equal, check_against_oracle, run_hip
from oracle import eager
from torch_dist_ext_amd import _capi

pytestmark = pytest.mark.gpu

CASES = [
    # first call fills most of the 32 MiB array, the second reuses its beginning with other contents
    (8, 1536, 8192, torch.bfloat16, 0.5, 1e-5, "fp8_token", 21),
    (4, 37, 1024, torch.float16, 1.0, 1e-6, "int8_token", 22),
    (2, 19, 2048, torch.float64, 1.0, 1e-6, "none", 24),      # doubles go through the staged launches as well
]


def test_static_stage_equals_staged_on_two_calls_in_a_row(cuda_device):
    for n, tokens, hidden, dtype, sigma, eps, quant, seed in CASES:
        parts, residual, gamma = eager.make_inputs(n, tokens, hidden, dtype, sigma, seed=seed)
        print("static stage case", n, tokens, hidden, dtype, quant, flush=True)
        want = run_hip(parts, residual, gamma, eps, quant, algo=_capi.ALGO_STAGED)
        got = run_hip(parts, residual, gamma, eps, quant, calls=[(("static_stage",), 0)])
        assert set(got) == set(want)
        for key in want:
            assert bits_equal(got[key], want[key]), key
        oracle = eager.reduce_rms(parts, residual, gamma, eps, quant)
        check_against_oracle(got, oracle, quant, gamma=gamma, eps=eps)


def test_static_stage_calls_leave_free_memory_unchanged(cuda_device):
    n, tokens, hidden = 4, 256, 4096
    parts, residual, gamma = eager.make_inputs(n, tokens, hidden, torch.bfloat16, 1.0, seed=23)
    dev = cuda_device
    d_parts = [p.contiguous().to(dev) for p in parts]
    d_res, d_gamma = residual.to(dev), gamma.to(dev)
    d_res_out, d_norm = torch.empty_like(d_res), torch.empty_like(d_res)
    prob = _capi.make_problem(_capi.BF16, n, tokens, hidden, 1e-6)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def call():
        _capi.reduce_rms(prob, [p.data_ptr() for p in d_parts], d_res.data_ptr(), d_res_out.data_ptr(), d_gamma.data_ptr(),
                         norm_out=d_norm.data_ptr(), stream=stream, phases=("static_stage",))

    call()   # the first call on a device looks the array's address up
    torch.cuda.synchronize(dev)
    free_before, _ = torch.cuda.mem_get_info(dev)
    for _ in range(20):
        call()
    torch.cuda.synchronize(dev)
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before
    want = eager.reduce_rms(parts, residual, gamma, 1e-6, "none")
    assert bits_equal(d_res_out.cpu(), want["residual_out"])


def test_static_stage_limits(cuda_device):
    lib = _capi.load()
    b = _capi.Buffers()
    # one row more than fits: 2049 x 8192 bf16 = 32 MiB + 16 KiB
    prob = _capi.make_problem(_capi.BF16, 8, 2049, 8192, 1e-6)
    assert lib.tde_reduce_rms_static_stage(ctypes.byref(prob), ctypes.byref(b), None) == _capi.ETOOBIG
    assert "static stage" in _capi.status_string(_capi.ETOOBIG)
    for algo in (_capi.ALGO_FUSED, _capi.ALGO_STAGED_OWNED):
        prob = _capi.make_problem(_capi.BF16, 8, 16, 1024, 1e-6, algo=algo)
        assert lib.tde_reduce_rms_static_stage(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EALGO


def test_static_stage_inside_a_hip_graph(cuda_device):
    """What the entry point is for: captured in a HIP graph (after one eager call on the device, which looks the
    array's address up), replayed with new inputs and eager work in between, every replay checked against the oracle."""
    dev = cuda_device
    n, t, h = 8, 96, 4096
    parts = [torch.empty((t, h), dtype=torch.bfloat16, device=dev) for _ in range(n)]
    res, gamma = torch.empty((t, h), dtype=torch.bfloat16, device=dev), torch.empty((h,), dtype=torch.bfloat16, device=dev)
    res_out = torch.empty_like(res)
    q = torch.empty((t, h), dtype=torch.uint8, device=dev)
    sc = torch.empty((t,), dtype=torch.float32, device=dev)
    prob = _capi.make_problem(_capi.BF16, n, t, h, 1e-5, quant=_capi.QUANT_FP8_TOKEN)

    def launch(stream):
        _capi.reduce_rms(prob, [p.data_ptr() for p in parts], res.data_ptr(), res_out.data_ptr(), gamma.data_ptr(),
                         q_out=q.data_ptr(), scale_out=sc.data_ptr(), stream=stream, phases=("static_stage",))

    def fill(seed):
        cp, cr, cg = eager.make_inputs(n, t, h, torch.bfloat16, 0.5, seed=seed)
        for i in range(n):
            parts[i].copy_(cp[i])
        res.copy_(cr)
        gamma.copy_(cg)
        return cp, cr, cg

    fill(31)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(torch.cuda.current_stream().cuda_stream)
    for seed in (32, 33, 34):
        cp, cr, cg = fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = {"residual_out": res_out.cpu(), "q": q.cpu().view(torch.float8_e4m3fn), "scale": sc.cpu()}
        for v in (res_out, q, sc):
            v.zero_()                        # eager work between replays
        torch.cuda.synchronize()
        check_against_oracle(got, eager.reduce_rms(cp, cr, cg, 1e-5, "fp8_token"), "fp8_token", gamma=cg, eps=1e-5)
