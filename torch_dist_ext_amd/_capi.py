"""ctypes view of the C ABI in include/tde_abi.h (libtde_hip.so).

Only plain pointers and sizes cross this boundary.  Torch is used by callers for device memory
and streams; this module itself does not import it."""
import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtde_hip.so")

MAX_RANKS = 16
QUANT_GROUP = 128

OK, EINVAL, ENRANKS, EDTYPE, ESHAPE, EHIDDEN, EALIGN, EQUANT, EALGO, EHIP, ERANK, ENOMEM, ETOOBIG = range(13)
STATIC_STAGE_BYTES = 32 << 20
BF16, F16, F32, F64 = 0, 1, 2, 3
QUANT_NONE, QUANT_FP8_TOKEN, QUANT_FP8_GROUP, QUANT_INT8_TOKEN, QUANT_FP8_STATIC = 0, 1, 2, 3, 4
ALGO_AUTO, ALGO_FUSED, ALGO_STAGED, ALGO_STAGED_OWNED = 0, 1, 2, 3

# Every symbol include/tde_abi.h declares.
ABI_VERSION = 4   # TDE_ABI_VERSION of include/tde_abi.h

EXPORTS = (
    "tde_abi_version", "tde_status_string", "tde_last_hip_error", "tde_plan", "tde_reduce_rms", "tde_stage_reduce", "tde_stage_norm",
    "tde_reduce_rms_static_stage",
    "tde_probe_copy", "tde_probe_launch", "tde_probe_stream", "tde_probe_rows", "tde_probe_rows_parts", "tde_device_info",
    "tde_workspace_create", "tde_workspace_destroy", "tde_workspace_slot", "tde_workspace_stage",
    "tde_workspace_slot_bytes", "tde_workspace_nranks", "tde_workspace_fill_table",
)


class Problem(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32), ("nranks", ctypes.c_int32), ("rank", ctypes.c_int32), ("quant", ctypes.c_int32),
        ("algo", ctypes.c_int32), ("write_norm", ctypes.c_int32), ("tokens", ctypes.c_int64), ("hidden", ctypes.c_int64),
        ("eps", ctypes.c_float), ("static_scale", ctypes.c_float),
        ("tune_vecs_per_thread", ctypes.c_int32), ("tune_rows_per_block", ctypes.c_int32),
        ("tune_workgroups_per_cu", ctypes.c_int32), ("reserved", ctypes.c_int32),
    ]


class Buffers(ctypes.Structure):
    _fields_ = [
        ("partial", ctypes.c_void_p * MAX_RANKS), ("partial_table", ctypes.c_void_p), ("residual_in", ctypes.c_void_p),
        ("residual_out", ctypes.c_void_p), ("norm_out", ctypes.c_void_p), ("gamma", ctypes.c_void_p),
        ("q_out", ctypes.c_void_p), ("scale_out", ctypes.c_void_p), ("stage", ctypes.c_void_p),
    ]


class PlanOut(ctypes.Structure):
    _fields_ = [
        ("algo", ctypes.c_int32), ("reference_algo", ctypes.c_int32), ("vec_elems", ctypes.c_int32),
        ("block_threads", ctypes.c_int32), ("vecs_per_thread", ctypes.c_int32), ("rows_per_block", ctypes.c_int32),
        ("grid_blocks", ctypes.c_int32), ("xcd_chunk", ctypes.c_int32), ("workgroups_per_cu", ctypes.c_int32),
        ("lds_bytes", ctypes.c_int32), ("algorithmic_bytes", ctypes.c_int64),
        ("scale_elems", ctypes.c_int64),
    ]


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("compute_units", ctypes.c_int32), ("memory_clock_khz", ctypes.c_int32), ("memory_bus_bits", ctypes.c_int32),
        ("reserved", ctypes.c_int32), ("total_memory_bytes", ctypes.c_int64),
    ]


class TdeError(RuntimeError):
    def __init__(self, status, text):
        super().__init__("tde status %d: %s" % (status, text))
        self.status = status


_lib = None


def load():
    """Load libtde_hip.so (once).  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s not built; run `python torch_dist_ext_amd/_build.py`" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    lib.tde_abi_version.restype = ctypes.c_int
    if lib.tde_abi_version() != ABI_VERSION:   # the structures below mirror one version of include/tde_abi.h
        raise ImportError("%s has ABI version %d, this module is written for %d; rebuild it"
                          % (LIB_PATH, lib.tde_abi_version(), ABI_VERSION))
    lib.tde_status_string.restype = ctypes.c_char_p
    lib.tde_status_string.argtypes = [ctypes.c_int]
    lib.tde_last_hip_error.restype = ctypes.c_int
    lib.tde_plan.restype = ctypes.c_int
    lib.tde_plan.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(PlanOut)]
    lib.tde_reduce_rms.restype = ctypes.c_int
    lib.tde_reduce_rms.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(Buffers), ctypes.c_void_p]
    for fn in (lib.tde_stage_reduce, lib.tde_stage_norm, lib.tde_probe_rows, lib.tde_reduce_rms_static_stage):
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(Buffers), ctypes.c_void_p]
    lib.tde_probe_rows_parts.restype = ctypes.c_int
    lib.tde_probe_rows_parts.argtypes = [ctypes.POINTER(Problem), ctypes.POINTER(Buffers), ctypes.c_int32, ctypes.c_void_p]
    lib.tde_probe_launch.restype = ctypes.c_int
    lib.tde_probe_launch.argtypes = [ctypes.c_void_p]
    lib.tde_probe_copy.restype = ctypes.c_int
    lib.tde_probe_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    lib.tde_probe_stream.restype = ctypes.c_int
    lib.tde_probe_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p]
    lib.tde_device_info.restype = ctypes.c_int
    lib.tde_device_info.argtypes = [ctypes.POINTER(DeviceInfo)]
    lib.tde_workspace_create.restype = ctypes.c_int
    lib.tde_workspace_create.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int64, ctypes.POINTER(ctypes.c_void_p)]
    lib.tde_workspace_destroy.restype = ctypes.c_int
    lib.tde_workspace_destroy.argtypes = [ctypes.c_void_p]
    lib.tde_workspace_slot.restype = ctypes.c_void_p
    lib.tde_workspace_slot.argtypes = [ctypes.c_void_p, ctypes.c_int32]
    lib.tde_workspace_stage.restype = ctypes.c_void_p
    lib.tde_workspace_stage.argtypes = [ctypes.c_void_p, ctypes.c_int32]
    lib.tde_workspace_slot_bytes.restype = ctypes.c_int64
    lib.tde_workspace_slot_bytes.argtypes = [ctypes.c_void_p]
    lib.tde_workspace_nranks.restype = ctypes.c_int32
    lib.tde_workspace_nranks.argtypes = [ctypes.c_void_p]
    lib.tde_workspace_fill_table.restype = ctypes.c_int
    lib.tde_workspace_fill_table.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int32]
    _lib = lib
    return lib


def status_string(status):
    return load().tde_status_string(int(status)).decode()


def check(status):
    if status != OK:
        text = status_string(status)
        if status == EHIP:
            text += " (hipError %d)" % load().tde_last_hip_error()
        raise TdeError(status, text)


def make_problem(dtype, nranks, tokens, hidden, eps, quant=QUANT_NONE, algo=ALGO_AUTO, write_norm=0, rank=0,
                 static_scale=0.0, vecs_per_thread=0, rows_per_block=0, workgroups_per_cu=0):
    return Problem(dtype=dtype, nranks=nranks, rank=rank, quant=quant, algo=algo, write_norm=int(write_norm),
                   tokens=tokens, hidden=hidden, eps=eps, static_scale=static_scale,
                   tune_vecs_per_thread=vecs_per_thread, tune_rows_per_block=rows_per_block,
                   tune_workgroups_per_cu=workgroups_per_cu)


def plan(problem):
    """tde_plan -> PlanOut (raises TdeError on a rejected problem)."""
    out = PlanOut()
    check(load().tde_plan(ctypes.byref(problem), ctypes.byref(out)))
    return out


def reduce_rms(problem, partials, residual_in, residual_out, gamma, norm_out=None, q_out=None, scale_out=None,
               stage=None, partial_table=None, stream=None, phases=("reduce", "norm")):
    """tde_reduce_rms with raw device addresses (ints).  `partials` is a sequence of addresses (None
    entries are taken from partial_table).  phases=("reduce",) / ("norm",) calls tde_stage_reduce /
    tde_stage_norm instead, phases=("traffic",) tde_probe_rows, phases=("static_stage",)
    tde_reduce_rms_static_stage.  Raises TdeError on a non-zero status."""
    b = Buffers()
    for r, p in enumerate(partials):
        b.partial[r] = p
    b.partial_table = partial_table
    b.residual_in, b.residual_out, b.norm_out, b.gamma = residual_in, residual_out, norm_out, gamma
    b.q_out, b.scale_out, b.stage = q_out, scale_out, stage
    lib = load()
    fn = {("reduce", "norm"): lib.tde_reduce_rms, ("reduce",): lib.tde_stage_reduce,
          ("norm",): lib.tde_stage_norm, ("traffic",): lib.tde_probe_rows,
          ("static_stage",): lib.tde_reduce_rms_static_stage}[tuple(phases)]
    check(fn(ctypes.byref(problem), ctypes.byref(b), stream))


def device_info():
    """tde_device_info for the current device -> DeviceInfo."""
    out = DeviceInfo()
    check(load().tde_device_info(ctypes.byref(out)))
    return out


def probe_stream(dst, src, nbytes, mode, stream=None):
    """tde_probe_stream: mode 0 read-only, 1 write-only, 2 copy."""
    check(load().tde_probe_stream(dst, src, nbytes, mode, stream))


def probe_copy(dst, src, nbytes, stream=None):
    check(load().tde_probe_copy(dst, src, nbytes, stream))
