"""ORACLE — TEST INFRASTRUCTURE ONLY.  Nothing under torch_dist_ext_amd/ may import this package;
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do, and only as the checker.

CPU restatement (torch eager, no GPU) of what the reference's own test computes for one rank's
stage of `allreduce_rms`:

  reduce + residual   test/test_all_reduce_fusion.py:75      allreduce_in.sum(dim=0) + residual_in
                      (kernel statement of the same order: src/common/all_reduce_fusion_impl.h:271-298)
  RMSNorm             test/test_all_reduce_fusion.py:23-28   fp32 variance, x*rsqrt(var+eps) -> .to(T) -> weight*x

The arithmetic lives in torch's CPU kernels (third-party; the reference pins no torch version, the
image has torch 2.10.0).  The reference has no quantization code (FP8_E4M3_MAX and scale_factor at
all_reduce_fusion_impl.h:26,313 are unused) and its tests assert nothing, so:

  pinned   reduce_residual, rmsnorm : checked in tests/test_oracle.py against closed forms, an
           order-sensitivity vector, an integer-arithmetic RNE restatement (oracle/tde_oracle.c),
           the reference's fp64 CPU check (test/unit_test.cpp:175-217, restated) and, where it
           builds, oracle/_ref (that function compiled from the reference's own file).
  PARITY UNPINNED by the reference: quant_fp8 / quant_int8 / quant_fp8_static.  Their definition is this build's own
           (scale = amax/448 resp. amax/127, RNE codes, clamp); they are pinned only against the
           mathematics: a textbook e4m3 encoder over all codes and midpoints, max-code and
           half-step dequantization properties, ties-to-even for int8; quant_fp8_static through
           power-of-two scales (exact quotients -> the textbook encoder), saturation at +-448*scale and
           bit equality with quant_fp8 when given a row's own dynamic scale.
"""
import torch

FP8_E4M3_MAX = 448.0
INT8_MAX = 127.0
GROUP = 128


def reduce_residual(parts: torch.Tensor, residual_in: torch.Tensor) -> torch.Tensor:
    """parts [N,T,H], residual_in [T,H], both dtype T.

    test_all_reduce_fusion.py:75 writes `allreduce_in.sum(dim=0) + residual_in`.  The sum is restated as
    what the kernel contract fixes (all_reduce_fusion_impl.h:280-298): fp32 accumulation in rank order
    0..N-1, one rounding to T.  torch's CPU `sum(dim=0)` is bit-identical to this wherever it runs its
    vectorized path; only the last few elements of the flattened tensor (the scalar tail when T*H is
    not a multiple of its vector chunk) are added in a different, host-ISA-dependent order
    (tests/test_oracle.py::test_torch_sum_dim0_is_rank_order_except_flat_tail)."""
    acc_type = torch.float64 if parts.dtype == torch.float64 else torch.float32   # doubles are summed as doubles
    acc = torch.zeros(parts.shape[1:], dtype=acc_type)
    for r in range(parts.shape[0]):
        acc = acc + parts[r].to(acc_type)
    return acc.to(parts.dtype) + residual_in


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """test_all_reduce_fusion.py:23-28 (RMSNorm.forward), statement for statement."""
    input_dtype = x.dtype
    variance = x.float().pow(2).mean(-1, keepdim=True)
    x = x * torch.rsqrt(variance + eps)
    x = x.to(input_dtype)
    return weight * x


def _scales_and_scaled(y: torch.Tensor, qmax: float, group):
    yf = y.float()
    T, H = yf.shape
    g = H if group is None else group
    yg = yf.view(T, H // g, g)
    amax = yg.abs().amax(dim=-1, keepdim=True)
    scale = amax / qmax
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    scaled = (yg / safe).clamp(-qmax, qmax)
    return scale.squeeze(-1), scaled.view(T, H)


def quant_fp8(y: torch.Tensor, group=None):
    """Dynamic OCP e4m3 quantization of the normed rows.  group=None: one scale per row ([T]);
    group=128: one per [row, 128 columns] ([T, H/128]).  Returns (codes float8_e4m3fn [T,H], scales fp32)."""
    scale, scaled = _scales_and_scaled(y, FP8_E4M3_MAX, group)
    if group is None:
        scale = scale.view(-1)
    return scaled.to(torch.float8_e4m3fn), scale


def quant_fp8_static(y: torch.Tensor, scale: float):
    """OCP e4m3 codes with a caller-given per-tensor scale (fp32): e4m3(clamp(float(y)/scale, +-448))."""
    s = torch.tensor(scale, dtype=torch.float32)
    return (y.float() / s).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)


def quant_int8(y: torch.Tensor):
    """Dynamic symmetric int8 per row: scale = amax/127, code = clamp(round_half_even(y/scale), +-127)."""
    scale, scaled = _scales_and_scaled(y, INT8_MAX, None)
    return torch.round(scaled).to(torch.int8), scale.view(-1)


def reduce_rms(parts, residual_in, gamma, eps, quant="none", static_scale=None):
    """The whole stage.  quant in {"none", "fp8_token", "fp8_group", "int8_token", "fp8_static"}.
    Returns dict(residual_out, norm_out[, q, scale])."""
    residual_out = reduce_residual(parts, residual_in)
    norm_out = rmsnorm(residual_out, gamma, eps)
    out = {"residual_out": residual_out, "norm_out": norm_out}
    if quant == "fp8_token":
        out["q"], out["scale"] = quant_fp8(norm_out, None)
    elif quant == "fp8_group":
        out["q"], out["scale"] = quant_fp8(norm_out, GROUP)
    elif quant == "int8_token":
        out["q"], out["scale"] = quant_int8(norm_out)
    elif quant == "fp8_static":
        out["q"] = quant_fp8_static(norm_out, static_scale)
    elif quant != "none":
        raise ValueError(quant)
    return out


# ---- seeded synthetic inputs shared by tests, smoke and bench --------------------------------------

CONFIGS = {
    # name: (N, T, H, dtype, sigma_partials, eps, quant, seed)
    "c1": (2, 16, 1024, torch.bfloat16, 1.0, 1e-6, "none", 0),
    "c2": (8, 128, 4096, torch.bfloat16, 0.5, 1e-5, "none", 2),
    "c3": (8, 2048, 8192, torch.bfloat16, 0.5, 1e-5, "fp8_token", 3),
    "c4": (4, 8192, 7168, torch.bfloat16, 1.0, 1e-6, "fp8_group", 4),
}
C5_TOKENS = (1, 64, 512, 4096, 32768)


def make_inputs(N, T, H, dtype, sigma=1.0, seed=0, outlier_channels=0, outlier_scale=100.0):
    """CPU tensors: parts [N,T,H], residual [T,H], gamma [H] in `dtype`.
    partials ~ N(0, sigma), residual ~ N(0,1), gamma ~ U(0.5,1.5); optional fixed seeded set of
    `outlier_channels` columns multiplied by outlier_scale in every partial before the cast."""
    g = torch.Generator().manual_seed(seed)
    wide = torch.float64 if dtype == torch.float64 else torch.float32   # doubles get all their mantissa bits
    parts = torch.randn((N, T, H), generator=g, dtype=wide) * sigma
    if outlier_channels:
        cols = torch.randperm(H, generator=g)[:outlier_channels]
        parts[:, :, cols] *= outlier_scale
    residual = torch.randn((T, H), generator=g, dtype=wide)
    gamma = torch.rand((H,), generator=g, dtype=wide) + 0.5
    return parts.to(dtype), residual.to(dtype), gamma.to(dtype)


def make_config(name, tokens=None):
    """Inputs of a named benchmark configuration (c1..c5).  "c5" needs tokens in C5_TOKENS.  Returns
    (parts, residual, gamma, eps, quant)."""
    if name == "c5":
        assert tokens is not None
        p, r, g = make_inputs(4, tokens, 5120, torch.float16, 1.0, seed=5, outlier_channels=5)
        return p, r, g, 1e-6, "int8_token"
    N, T, H, dtype, sigma, eps, quant, seed = CONFIGS[name]
    if tokens is not None:
        T = tokens
    p, r, g = make_inputs(N, T, H, dtype, sigma, seed)
    return p, r, g, eps, quant
