"""MI355X-native drop-in for the fused path of the reference package `torch_dist_ext`.

Public names, argument order and meaning follow the reference's torch_dist_ext/__init__.py:
`CommWorkspace` (:15), `allreduce_rms_fusion_impl` (:16), `CommProcess` (:19-34), `setup_env` (:41-46),
operators `torch_dist_ext::get_workspace` (:49-61) and `torch_dist_ext::allreduce_rms` (:64-81, registered by the C++
library here), module attribute `allreduce_rms` (:84).

What differs: one GPU plays every rank.  The N peer partial buffers are N local allocations owned
by `CommWorkspace`; `set_peer_partial` / `peer_partial` fill them where the reference's peers would
write through IPC-mapped memory.  No torch.distributed call is made.

The HIP library is required: importing this package without the built shared libraries raises.
"""
import ctypes
import os
import torch

from . import _capi
from ._capi import (ALGO_AUTO, ALGO_FUSED, ALGO_STAGED, ALGO_STAGED_OWNED, QUANT_FP8_GROUP, QUANT_FP8_STATIC, QUANT_FP8_TOKEN, QUANT_INT8_TOKEN,
                    QUANT_NONE, QUANT_GROUP)

this_dir = os.path.dirname(os.path.abspath(__file__))
# where the reference's loader looks (torch_dist_ext/__init__.py:8-12): beside the package directory
filename = os.path.join(os.path.dirname(this_dir), "libtorch_dist_ext.so")
if not (os.path.exists(filename) and os.path.exists(_capi.LIB_PATH)):
    raise ImportError(
        "torch_dist_ext_amd: %s / %s not built. Run `python torch_dist_ext_amd/_build.py` "
        "(there is no CPU fallback)." % (os.path.basename(filename), os.path.basename(_capi.LIB_PATH)))
_capi.load()  # libtde_hip.so first, so the extension resolves against the in-tree copy
torch.ops.load_library(filename)

CommWorkspace = torch.classes.torch_dist_ext.CommWorkspace
allreduce_rms_fusion_impl = torch.ops.torch_dist_ext.allreduce_rms_fusion
allreduce_rms_quant_fusion_impl = torch.ops.torch_dist_ext.allreduce_rms_quant_fusion
reduce_rms_local_impl = torch.ops.torch_dist_ext.reduce_rms_local

QUANT_MODES = {"none": QUANT_NONE, "fp8_token": QUANT_FP8_TOKEN, "fp8_group": QUANT_FP8_GROUP, "int8_token": QUANT_INT8_TOKEN,
               "fp8_static": QUANT_FP8_STATIC}


class CommProcess:
    """Reference: torch_dist_ext/__init__.py:19-34.  The handle exchange that the reference does with
    dist.all_gather_object + two barriers is a local list here: every slot lives in this process."""

    def __init__(self, rank, world_size, size_in_bytes, group=None):
        if rank < torch.cuda.device_count():
            torch.cuda.set_device(rank)
        nblocks = 256
        self.rank = rank
        self.world_size = world_size
        self.comm = CommWorkspace(rank, world_size, nblocks, size_in_bytes)
        handle = self.comm.get_handle()
        handle_list = [handle.clone() for _ in range(world_size)]
        torch.cuda.synchronize()
        self.comm.open_handles(handle_list)
        torch.cuda.synchronize()

    def get_workspace(self, ref):
        return self.comm.get_workspace(ref)


comm = None
world_size_ = None


def setup_env(rank, world_size, max_size_in_bytes=8192 * 16384, group=None):
    """Reference: torch_dist_ext/__init__.py:41-46."""
    global comm
    global world_size_
    comm = CommProcess(rank, world_size, max_size_in_bytes, group)
    comm.comm.make_current()   # the workspace torch_dist_ext::get_workspace hands out from now on
    world_size_ = world_size


def set_peer_partial(r: int, partial: torch.Tensor) -> None:
    """Emulation only: store rank r's partial where that peer's kernel would have written it."""
    assert comm is not None
    comm.comm.set_peer_partial(r, partial)


def peer_partial(r: int, ref: torch.Tensor) -> torch.Tensor:
    """Emulation only: a tensor like `ref` aliasing rank r's slot (fill it in place, no copy)."""
    assert comm is not None
    return comm.comm.peer_partial(r, ref)


# torch_dist_ext::get_workspace (reference: torch_dist_ext/__init__.py:49-53, a Python custom_op over the global `comm`)
# is registered by the C++ library, which keeps the workspace that setup_env made current: 1.5 us per call instead of
# the 7 us a Python custom_op costs.  Its fake implementation stays here, as in the reference (:56-61).
get_workspace = torch.ops.torch_dist_ext.get_workspace


@torch.library.register_fake("torch_dist_ext::get_workspace")
def get_workspace_fake(ref: torch.Tensor) -> torch.Tensor:
    global world_size_
    assert world_size_ is not None
    nbytes = (world_size_ * 3 + 5) * ctypes.sizeof(ctypes.c_void_p)
    return torch.empty(nbytes, dtype=torch.uint8)


# torch_dist_ext::allreduce_rms (reference: torch_dist_ext/__init__.py:64-81, a Python custom_op with a fake
# implementation) and its quantizing form torch_dist_ext::allreduce_rms_quant are registered by the C++ library with
# the same names and schemas, CUDA and Meta kernels: the outputs are allocated in C++ and a call costs the dispatcher
# and one kernel launch, not a Python custom_op's 12 us of host time.  What differs from the reference: hidden_dim >
# 8192 raises RuntimeError where the reference's `assert` raises AssertionError.
#
#   allreduce_rms(rank, nranks, allreduce_in, residual_in, rms_gamma, eps, workspace) -> (norm_out, residual_out)
#   allreduce_rms_quant(rank, nranks, allreduce_in, residual_in, rms_gamma, eps, workspace, quant_mode, write_norm,
#                       static_scale=0.0) -> (codes, scales, residual_out, norm_out)
#     quant_mode is one of QUANT_FP8_TOKEN / QUANT_FP8_GROUP / QUANT_INT8_TOKEN / QUANT_FP8_STATIC; norm_out has zero
#     elements unless write_norm; scales has zero elements for QUANT_FP8_STATIC (static_scale is the scale).
allreduce_rms_quant = torch.ops.torch_dist_ext.allreduce_rms_quant


def _quant_out_shapes(allreduce_in: torch.Tensor, quant_mode: int):
    hidden = allreduce_in.shape[-1]
    lead = tuple(allreduce_in.shape[:-1])
    if quant_mode == QUANT_FP8_GROUP:
        scale_shape = lead + (hidden // QUANT_GROUP,)
    elif quant_mode == QUANT_FP8_STATIC:
        scale_shape = (0,)   # the scale is the caller's; nothing is written
    else:
        scale_shape = lead
    q_dtype = torch.int8 if quant_mode == QUANT_INT8_TOKEN else torch.float8_e4m3fn
    return q_dtype, scale_shape


def reduce_rms(partials, residual_in, rms_gamma, eps, quant_mode=QUANT_NONE, write_norm=None, algo=ALGO_AUTO, stage=None,
               static_scale=0.0):
    """One rank's stage with the N partials passed as a list of N [tokens, hidden] GPU tensors.

    Returns a dict with residual_out and, depending on the mode, norm_out / q / scale."""
    ref = partials[0]
    if write_norm is None:
        write_norm = quant_mode == QUANT_NONE
    out = {"residual_out": torch.empty_like(residual_in)}
    norm_out = torch.empty_like(ref) if (write_norm or quant_mode == QUANT_NONE) else None
    q_out = scale_out = None
    if quant_mode != QUANT_NONE:
        q_dtype, scale_shape = _quant_out_shapes(ref, quant_mode)
        q_out = torch.empty(ref.shape, dtype=q_dtype, device=ref.device)
        out["q"] = q_out
        if quant_mode != QUANT_FP8_STATIC:
            scale_out = torch.empty(scale_shape, dtype=torch.float32, device=ref.device)
            out["scale"] = scale_out
    if algo in (ALGO_STAGED, ALGO_STAGED_OWNED) and stage is None:
        stage = torch.empty_like(ref)
    reduce_rms_local_impl(list(partials), residual_in, rms_gamma, out["residual_out"], norm_out, q_out, scale_out, eps,
                          quant_mode, algo, stage, static_scale)
    if norm_out is not None:
        out["norm_out"] = norm_out
    return out


allreduce_rms = torch.ops.torch_dist_ext.allreduce_rms
