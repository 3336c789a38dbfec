"""Shared pieces of the parity tests: bit-level distances and the C-ABI call on device tensors."""
import torch

from torch_dist_ext_amd import _capi

DTYPE_CODE = {torch.bfloat16: _capi.BF16, torch.float16: _capi.F16, torch.float32: _capi.F32}
QUANT_CODE = {"none": _capi.QUANT_NONE, "fp8_token": _capi.QUANT_FP8_TOKEN, "fp8_group": _capi.QUANT_FP8_GROUP,
              "int8_token": _capi.QUANT_INT8_TOKEN}


def ordered_bits(t: torch.Tensor) -> torch.Tensor:
    """Map a float tensor (bf16/fp16/fp32/fp8) to int64 keys that are monotonic in value, so that
    |key(a)-key(b)| is the distance in units in the last place (+0 and -0 coincide)."""
    if t.element_size() == 1:
        raw = t.view(torch.uint8).to(torch.int64)
        sign, mag = raw >> 7, raw & 0x7F
    elif t.element_size() == 2:
        raw = t.view(torch.int16).to(torch.int64) & 0xFFFF
        sign, mag = raw >> 15, raw & 0x7FFF
    else:
        raw = t.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
        sign, mag = raw >> 31, raw & 0x7FFFFFFF
    return torch.where(sign == 1, -mag, mag)


def ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (ordered_bits(a) - ordered_bits(b)).abs()


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    va = a.contiguous().view(torch.uint8)
    vb = b.contiguous().view(torch.uint8)
    return va.shape == vb.shape and bool(torch.equal(va, vb))


def run_hip(parts, residual, gamma, eps, quant="none", algo=_capi.ALGO_AUTO, write_norm=None, use_table=False,
            rank=0, device="cuda:0"):
    """Run the HIP path through the C ABI (tde_reduce_rms) on CPU inputs; returns CPU outputs.
    parts: [N,T,H] tensor or list of N [T,H] tensors."""
    dev = torch.device(device)
    n = len(parts)
    T, H = residual.shape
    dtype = residual.dtype
    # N separate device allocations, as the N peer buffers
    d_parts = [parts[r].contiguous().to(dev) for r in range(n)]
    d_res = residual.contiguous().to(dev)
    d_gamma = gamma.contiguous().to(dev)
    d_res_out = torch.empty_like(d_res)
    qm = QUANT_CODE[quant]
    if write_norm is None:
        write_norm = True
    d_norm = torch.empty_like(d_res) if (write_norm or qm == 0) else None
    d_q = d_scale = None
    if qm:
        d_q = torch.empty((T, H), dtype=torch.uint8, device=dev)
        nscale = T * (H // 128) if quant == "fp8_group" else T
        d_scale = torch.empty((nscale,), dtype=torch.float32, device=dev)
    d_stage = torch.empty_like(d_res) if algo == _capi.ALGO_STAGED else None
    prob = _capi.make_problem(DTYPE_CODE[dtype], n, T, H, eps, quant=qm, algo=algo, write_norm=int(bool(write_norm)),
                              rank=rank)
    ptrs = [p.data_ptr() for p in d_parts]
    table = None
    d_table = None
    if use_table:
        d_table = torch.tensor(ptrs, dtype=torch.int64, device=dev)
        table = d_table.data_ptr()
        ptrs = [p if r == rank else None for r, p in enumerate(ptrs)]
    stream = torch.cuda.current_stream(dev).cuda_stream
    _capi.reduce_rms(prob, ptrs, d_res.data_ptr(), d_res_out.data_ptr(), d_gamma.data_ptr(),
                     norm_out=d_norm.data_ptr() if d_norm is not None else None,
                     q_out=d_q.data_ptr() if d_q is not None else None,
                     scale_out=d_scale.data_ptr() if d_scale is not None else None,
                     stage=d_stage.data_ptr() if d_stage is not None else None,
                     partial_table=table, stream=stream)
    torch.cuda.synchronize(dev)
    out = {"residual_out": d_res_out.cpu()}
    if d_norm is not None:
        out["norm_out"] = d_norm.cpu()
    if qm:
        q = d_q.cpu()
        out["q"] = q.view(torch.int8) if quant == "int8_token" else q.view(torch.float8_e4m3fn)
        sc = d_scale.cpu()
        out["scale"] = sc.view(T, H // 128) if quant == "fp8_group" else sc
    return out


def check_against_oracle(got, want, quant, norm_ulp=1, scale_rtol=1e-6, allow_scale_outliers=0):
    """The parity bar: residual bit-exact, normed within norm_ulp units in the last place, codes within
    one quant step, scales within scale_rtol relative.  Returns a dict of mismatch statistics."""
    stats = {}
    assert bits_equal(got["residual_out"], want["residual_out"]), "residual_out is not bit-exact"
    if "norm_out" in got:
        d = ulp_distance(got["norm_out"], want["norm_out"])
        stats["norm_max_ulp"] = int(d.max()) if d.numel() else 0
        stats["norm_mismatch_frac"] = float((d > 0).float().mean()) if d.numel() else 0.0
        assert stats["norm_max_ulp"] <= norm_ulp, "norm_out off by %d ulp" % stats["norm_max_ulp"]
        assert not torch.isnan(got["norm_out"].float()).any()
    if quant != "none":
        gs, ws = got["scale"].double().flatten(), want["scale"].double().flatten()
        rel = (gs - ws).abs() / ws.abs().clamp_min(1e-30)
        rel = torch.where((gs == 0) & (ws == 0), torch.zeros_like(rel), rel)
        bad = int((rel > scale_rtol).sum())
        stats["scale_max_rel"] = float(rel.max()) if rel.numel() else 0.0
        stats["scale_bad"] = bad
        assert bad <= allow_scale_outliers, "%d scales differ by more than %g relative (max %g)" % (
            bad, scale_rtol, stats["scale_max_rel"])
        if quant == "int8_token":
            dq = (got["q"].to(torch.int32) - want["q"].to(torch.int32)).abs()
        else:
            dq = ulp_distance(got["q"], want["q"])
        stats["q_max_step"] = int(dq.max()) if dq.numel() else 0
        stats["q_mismatch_frac"] = float((dq > 0).float().mean()) if dq.numel() else 0.0
        assert stats["q_max_step"] <= 1, "codes off by %d quant steps" % stats["q_max_step"]
    return stats
