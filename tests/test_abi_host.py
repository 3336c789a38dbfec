"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol the header
declares, tde_plan validates like the reference's launcher asserts, algorithmic bytes match the
documented formula, and the torch layer registers the reference's schemas verbatim."""
import ctypes
import os
import re

import pytest
import torch

from torch_dist_ext_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "tde_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tde_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_capi.LIB_PATH)
    declared = _declared_functions()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(_capi.EXPORTS) == declared
    assert _capi.load().tde_abi_version() == _capi.ABI_VERSION == 4


def test_library_exports_nothing_but_the_declared_symbols():
    """Launchers, kernel handles and template instantiations stay inside the library (its link uses an export map),
    so a second copy of the library in one process runs its own kernels; the dynamic symbol table is read with nm."""
    import shutil
    import subprocess
    if shutil.which("nm") is None:
        pytest.skip("no nm on this machine")
    out = subprocess.run(["nm", "-D", "--defined-only", _capi.LIB_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == _declared_functions()


def test_struct_layouts_match_header():
    assert ctypes.sizeof(_capi.Problem) == 64
    assert ctypes.sizeof(_capi.Buffers) == (16 + 8) * 8
    assert ctypes.sizeof(_capi.PlanOut) == 56


def _plan(**kw):
    base = dict(dtype=_capi.BF16, nranks=8, tokens=2048, hidden=8192, eps=1e-5)
    base.update(kw)
    return _capi.plan(_capi.make_problem(**base))


@pytest.mark.parametrize("kw,status", [
    (dict(nranks=3), _capi.ENRANKS), (dict(nranks=16), _capi.ENRANKS), (dict(nranks=1), _capi.ENRANKS),
    (dict(dtype=7), _capi.EDTYPE),
    (dict(hidden=8190), _capi.ESHAPE),      # 8190*2 bytes is not a multiple of 16 (impl.h:480)
    (dict(hidden=0), _capi.ESHAPE), (dict(tokens=-1), _capi.ESHAPE),
    (dict(tokens=1 << 60), _capi.ESHAPE),   # tokens * hidden * 2 overflows 64-bit byte offsets
    (dict(dtype=_capi.F64, hidden=2050), _capi.EHIDDEN), (dict(dtype=_capi.F64, hidden=1025), _capi.ESHAPE),
    (dict(dtype=_capi.F64, quant=_capi.QUANT_FP8_TOKEN), _capi.EQUANT),
    (dict(hidden=8200), _capi.EHIDDEN),     # beyond 1024 vectors per row (the reference asserts hidden <= 8192)
    (dict(dtype=_capi.F32, hidden=4100), _capi.EHIDDEN),
    (dict(quant=9), _capi.EQUANT), (dict(quant=_capi.QUANT_FP8_GROUP, hidden=1032), _capi.EQUANT),
    (dict(quant=_capi.QUANT_FP8_STATIC), _capi.EQUANT), (dict(quant=_capi.QUANT_FP8_STATIC, static_scale=-2.0), _capi.EQUANT),
    (dict(algo=5), _capi.EALGO), (dict(rank=8), _capi.ERANK), (dict(rank=-1), _capi.ERANK),
    (dict(hidden=1 << 40), _capi.EHIDDEN),  # far beyond a row: refused before any size arithmetic
    (dict(vecs_per_thread=3), _capi.EINVAL), (dict(rows_per_block=-1), _capi.EINVAL),   # per-call geometry overrides
])
def test_plan_rejects(kw, status):
    with pytest.raises(_capi.TdeError) as e:
        _plan(**kw)
    assert e.value.status == status
    assert _capi.status_string(status) != "unknown status"


def test_static_stage_entry_point_limits_need_no_gpu():
    lib = _capi.load()
    b = _capi.Buffers()
    prob = _capi.make_problem(_capi.BF16, 8, 2049, 8192, 1e-6)       # one row more than the 32 MiB stage holds
    assert lib.tde_reduce_rms_static_stage(ctypes.byref(prob), ctypes.byref(b), None) == _capi.ETOOBIG
    for algo in (_capi.ALGO_FUSED, _capi.ALGO_STAGED_OWNED):
        prob = _capi.make_problem(_capi.BF16, 8, 16, 1024, 1e-6, algo=algo)
        assert lib.tde_reduce_rms_static_stage(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EALGO
    assert lib.tde_reduce_rms_static_stage(None, None, None) == _capi.EINVAL


def test_plan_geometry_overrides_are_per_call():
    auto = _plan()
    forced = _plan(vecs_per_thread=1)
    assert auto.vecs_per_thread == 4 and forced.vecs_per_thread == 1 and forced.block_threads == 1024
    assert _plan().vecs_per_thread == 4          # nothing sticks between calls
    packed = _plan(hidden=1024, tokens=4096, vecs_per_thread=1, rows_per_block=4)
    assert packed.rows_per_block == 4 and packed.block_threads == 512 and packed.grid_blocks == 1024


def test_plan_null_pointers():
    lib = _capi.load()
    assert lib.tde_plan(None, None) == _capi.EINVAL
    assert lib.tde_reduce_rms(None, None, None) == _capi.EINVAL
    out = _capi.PlanOut()
    assert lib.tde_plan(None, ctypes.byref(out)) == _capi.EINVAL


@pytest.mark.parametrize("cfg,expected", [
    # the five benchmark configurations: bytes = (N+1)*T*H*e + H*e + T*H*e + OUT
    (dict(nranks=2, tokens=16, hidden=1024, quant=_capi.QUANT_NONE), 165888),
    (dict(nranks=8, tokens=128, hidden=4096, quant=_capi.QUANT_NONE), 11542528),
    (dict(nranks=8, tokens=2048, hidden=8192, quant=_capi.QUANT_FP8_TOKEN), 352346112),
    (dict(nranks=4, tokens=8192, hidden=7168, quant=_capi.QUANT_FP8_GROUP), 765212672),
    (dict(dtype=_capi.F16, nranks=4, tokens=32768, hidden=5120, quant=_capi.QUANT_INT8_TOKEN), 66564 * 32768 + 10240),
    (dict(dtype=_capi.F16, nranks=4, tokens=1, hidden=5120, quant=_capi.QUANT_INT8_TOKEN), 66564 + 10240),
])
def test_algorithmic_bytes(cfg, expected):
    assert _plan(**cfg).algorithmic_bytes == expected


def test_plan_geometry_and_reference_threshold():
    p = _plan(tokens=128)
    assert p.reference_algo == 1 and _plan(tokens=129).reference_algo == 2   # kOneShotMaxToken, impl.h:24,491
    assert p.vec_elems == 8 and _plan(dtype=_capi.F32, hidden=1024).vec_elems == 4
    for hidden in (124, 508, 1024, 4096, 5120, 7168, 8192):
        for dt in (_capi.BF16, _capi.F32):
            if (dt == _capi.F32 and hidden > 4096) or (dt == _capi.BF16 and hidden % 8):
                continue
            q = _plan(dtype=dt, hidden=hidden, tokens=777)
            nvec = hidden // q.vec_elems
            assert q.block_threads % 64 == 0 and q.block_threads <= 1024
            per_row = q.block_threads // q.rows_per_block
            assert per_row * q.vecs_per_thread >= nvec                  # every vector of a row has an owner
            assert q.grid_blocks * q.rows_per_block >= 777
    assert _plan(tokens=0).grid_blocks == 0
    assert _plan(algo=_capi.ALGO_STAGED).algo == _capi.ALGO_STAGED and _plan().algo == _capi.ALGO_FUSED
    assert _plan(algo=_capi.ALGO_STAGED_OWNED).algo == _capi.ALGO_STAGED_OWNED
    assert _plan(quant=_capi.QUANT_FP8_GROUP, hidden=7168, nranks=4, tokens=8192).scale_elems == 8192 * 56


def test_reduce_rms_argument_checks_need_no_gpu():
    lib = _capi.load()
    prob = _capi.make_problem(_capi.BF16, 2, 4, 256, 1e-6)
    b = _capi.Buffers()
    assert lib.tde_reduce_rms(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EINVAL      # no partials
    b.partial[0], b.partial[1] = 0x1000, 0x2008                                                   # misaligned
    assert lib.tde_reduce_rms(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EALIGN
    b.partial[1] = 0x2000
    assert lib.tde_reduce_rms(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EINVAL      # no residual/gamma
    b.residual_in = b.residual_out = b.gamma = b.norm_out = 0x3000
    prob.algo = _capi.ALGO_STAGED
    assert lib.tde_reduce_rms(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EALGO       # staged without stage
    prob.algo = _capi.ALGO_AUTO
    prob.quant = _capi.QUANT_FP8_TOKEN
    assert lib.tde_reduce_rms(ctypes.byref(prob), ctypes.byref(b), None) == _capi.EINVAL      # quant without q/scale
    prob.tokens = 0
    assert lib.tde_reduce_rms(ctypes.byref(prob), ctypes.byref(_capi.Buffers()), None) == _capi.OK   # empty input: no launch


def test_workspace_argument_checks_need_no_gpu():
    lib = _capi.load()
    ws = ctypes.c_void_p()
    assert lib.tde_workspace_create(3, 256, 1024, ctypes.byref(ws)) == _capi.ENRANKS
    assert lib.tde_workspace_create(2, 256, 1000, ctypes.byref(ws)) == _capi.ESHAPE
    assert lib.tde_workspace_create(2, 256, 1024, None) == _capi.EINVAL
    assert lib.tde_workspace_create(2, 0, 1024, ctypes.byref(ws)) == _capi.EINVAL      # nblocks sizes the flag regions
    assert lib.tde_workspace_destroy(None) == _capi.OK
    assert lib.tde_workspace_slot(None, 0) is None


# ---- torch layer: the reference's names and schemas (src/register.cpp:4-15, torch_dist_ext/__init__.py) ------

def test_torch_schemas_match_reference():
    import torch_dist_ext_amd as tde
    s = str(torch.ops.torch_dist_ext.allreduce_rms_fusion.default._schema)
    assert s == ("torch_dist_ext::allreduce_rms_fusion(SymInt rank, SymInt nranks, Tensor allreduce_in, Tensor residual_in, "
                 "Tensor rms_gamma, Tensor residual_out, Tensor norm_out, float eps, Tensor workspace) -> ()")
    s = str(torch.ops.torch_dist_ext.allreduce_rms.default._schema)
    assert s == ("torch_dist_ext::allreduce_rms(SymInt rank, SymInt nranks, Tensor allreduce_in, Tensor residual_in, "
                 "Tensor rms_gamma, float eps, Tensor workspace) -> (Tensor, Tensor)") or "int rank, int nranks" in s
    assert "get_workspace(Tensor ref) -> Tensor" in str(torch.ops.torch_dist_ext.get_workspace.default._schema)
    for name in ("CommWorkspace", "allreduce_rms_fusion_impl", "CommProcess", "setup_env", "get_workspace", "allreduce_rms"):
        assert hasattr(tde, name), name
    assert tde.allreduce_rms is torch.ops.torch_dist_ext.allreduce_rms
    import inspect
    assert list(inspect.signature(tde.setup_env).parameters) == ["rank", "world_size", "max_size_in_bytes", "group"]
    assert inspect.signature(tde.setup_env).parameters["max_size_in_bytes"].default == 8192 * 16384


def test_reference_package_name_resolves_to_this_build():
    """A caller written against the reference does `import torch_dist_ext` (test/test_all_reduce_fusion.py:8) and
    the reference loads `<parent of the package>/libtorch_dist_ext.so` (torch_dist_ext/__init__.py:8-12)."""
    import importlib
    import os
    import torch_dist_ext
    import torch_dist_ext_amd
    assert torch_dist_ext is torch_dist_ext_amd
    assert importlib.import_module("torch_dist_ext") is torch_dist_ext_amd
    for name in ("CommWorkspace", "allreduce_rms_fusion_impl", "CommProcess", "setup_env", "get_workspace", "allreduce_rms"):
        assert hasattr(torch_dist_ext, name), name
    assert torch_dist_ext.allreduce_rms is torch.ops.torch_dist_ext.allreduce_rms
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    assert os.path.samefile(torch_dist_ext.filename, os.path.join(root, "libtorch_dist_ext.so"))
    assert os.path.isdir(os.path.join(root, "torch_dist_ext"))   # the directory whose name the loader rule starts from


def test_fake_tensor_shapes():
    import torch_dist_ext_amd as tde
    from torch._subclasses.fake_tensor import FakeTensorMode
    tde.world_size_ = 4
    try:
        with FakeTensorMode():
            x = torch.empty((128, 1024), dtype=torch.bfloat16)
            g = torch.empty((1024,), dtype=torch.bfloat16)
            ws = torch.ops.torch_dist_ext.get_workspace(x)
            assert ws.shape == ((4 * 3 + 5) * 8,) and ws.dtype == torch.uint8
            n, r = torch.ops.torch_dist_ext.allreduce_rms(0, 4, x, x, g, 1e-6, ws)
            assert n.shape == x.shape and r.shape == x.shape and n.dtype == x.dtype
            q, s, r2, n2 = torch.ops.torch_dist_ext.allreduce_rms_quant(0, 4, x, x, g, 1e-6, ws, tde.QUANT_FP8_GROUP, False)
            assert q.dtype == torch.float8_e4m3fn and s.shape == (128, 8) and n2.numel() == 0
            q, s, r2, n2 = torch.ops.torch_dist_ext.allreduce_rms_quant(0, 4, x, x, g, 1e-6, ws, tde.QUANT_INT8_TOKEN, True)
            assert q.dtype == torch.int8 and s.shape == (128,) and n2.shape == x.shape
    finally:
        tde.world_size_ = None


def test_cpu_tensors_are_rejected_not_silently_computed():
    import torch_dist_ext_amd as tde
    x = torch.zeros((4, 256), dtype=torch.bfloat16)
    g = torch.ones((256,), dtype=torch.bfloat16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        tde.allreduce_rms_fusion_impl(0, 2, x, x, g, torch.empty_like(x), torch.empty_like(x), 1e-6,
                                      torch.zeros(88, dtype=torch.uint8))


def test_bench_draws_the_configurations_seeded_inputs():
    """bench.py checks the kernel's outputs for its first input set against the oracle; that set must be the
    configuration's seeded inputs (the same tensors the parity tests use)."""
    import importlib.util
    import os
    from oracle import eager
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("tde_bench", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    got = bench.seeded_cpu_inputs(torch, bench.BENCH_CONFIGS["c2"])
    want = eager.make_config("c2")[:3]
    for g, w in zip(got, want):
        assert torch.equal(g.view(torch.int16), w.view(torch.int16))
    cfg = list(bench.BENCH_CONFIGS["c5"])
    cfg[1] = 64                                    # c5 at 64 rows: the outlier channels and the fp16 cast
    got = bench.seeded_cpu_inputs(torch, tuple(cfg))
    want = eager.make_config("c5", tokens=64)[:3]
    for g, w in zip(got, want):
        assert torch.equal(g.view(torch.int16), w.view(torch.int16))
    assert bench.BENCH_CONFIGS["c3"][:3] == (8, 2048, 8192) and bench.BENCH_CONFIGS["c3"][5] == eager.CONFIGS["c3"][5]
    assert len(bench.kernel_sources_sha256()) == 64


def _needs_256_compute_units():
    """tde_plan sizes the geometry for the visible device's compute units (256 where there is none, as here on the
    CPU): the expectations below are for an unpartitioned MI355X."""
    if torch.cuda.is_available():
        cus = _capi.device_info().compute_units
        if cus != 256:
            pytest.skip("expectations are for 256 compute units, the visible device has %d" % cus)


@pytest.mark.parametrize("kw,vpt,threads", [
    # the benchmark configurations
    (dict(nranks=8, tokens=128, hidden=4096), 1, 512),                               # c2
    (dict(nranks=8, tokens=2048, hidden=8192), 4, 256),                              # c3
    (dict(nranks=4, tokens=8192, hidden=7168), 4, 256),                              # c4
    (dict(dtype=_capi.F16, nranks=4, tokens=32768, hidden=5120), 4, 192),            # c5, 32768 rows
    (dict(dtype=_capi.F16, nranks=4, tokens=4096, hidden=5120), 2, 320),             # c5, 4096 rows
    (dict(dtype=_capi.F16, nranks=4, tokens=512, hidden=5120), 1, 640),              # c5, 512 rows
    # the measured boundaries of the choice
    (dict(nranks=8, tokens=255, hidden=8192), 2, 512), (dict(nranks=8, tokens=127, hidden=8192), 1, 1024),
    (dict(nranks=2, tokens=2048, hidden=8192), 2, 512), (dict(nranks=2, tokens=2049, hidden=8192), 4, 256),
    (dict(nranks=8, tokens=1024, hidden=4096), 4, 128), (dict(nranks=4, tokens=1024, hidden=4096), 1, 512),
    (dict(nranks=8, tokens=2048, hidden=2048), 4, 64), (dict(nranks=8, tokens=2047, hidden=2048), 1, 256),
    (dict(nranks=4, tokens=32767, hidden=2048), 1, 256), (dict(nranks=4, tokens=32768, hidden=2048), 2, 128),
    (dict(nranks=8, tokens=640, hidden=5120), 2, 320), (dict(nranks=8, tokens=2048, hidden=5120), 1, 640),
    (dict(nranks=8, tokens=16383, hidden=5120), 1, 640), (dict(nranks=8, tokens=16384, hidden=5120), 2, 320),
    # long launches of mid-length rows: two vectors per thread
    (dict(nranks=8, tokens=16383, hidden=4096), 4, 128), (dict(nranks=8, tokens=16384, hidden=4096), 2, 256),
    (dict(nranks=8, tokens=32767, hidden=2048), 4, 64), (dict(nranks=8, tokens=32768, hidden=2048), 2, 128),
    (dict(nranks=8, tokens=2047, hidden=6144), 1, 768), (dict(nranks=8, tokens=2048, hidden=6144), 4, 192),
    (dict(nranks=8, tokens=5632, hidden=6144), 1, 768), (dict(nranks=8, tokens=8192, hidden=6144), 2, 384),
    (dict(nranks=4, tokens=1024, hidden=6144), 4, 192), (dict(nranks=4, tokens=2048, hidden=6144), 1, 768),
    (dict(nranks=8, tokens=8191, hidden=3072, quant=_capi.QUANT_FP8_TOKEN), 1, 384), (dict(nranks=8, tokens=8192, hidden=3072, quant=_capi.QUANT_FP8_TOKEN), 4, 128),
    (dict(nranks=8, tokens=32768, hidden=3072, quant=_capi.QUANT_INT8_TOKEN), 2, 192), (dict(nranks=8, tokens=32768, hidden=3072), 1, 384),
    (dict(nranks=8, tokens=4096, hidden=1024), 2, 64), (dict(nranks=8, tokens=8192, hidden=1024), 1, 128),
    (dict(nranks=2, tokens=32768, hidden=5120), 2, 320), (dict(nranks=4, tokens=16384, hidden=5120), 4, 192), (dict(nranks=4, tokens=16383, hidden=5120), 2, 320),
])
def test_plan_vectors_per_thread(kw, vpt, threads):
    """The launch geometry tde_plan chooses where the sweeps put a boundary (threads = one row's share)."""
    _needs_256_compute_units()
    p = _plan(**kw)
    assert (p.vecs_per_thread, p.block_threads // p.rows_per_block) == (vpt, threads)


@pytest.mark.parametrize("kw,limit,lds", [
    # fewer than 6144 workgroups, two partials, the staged algorithms and doubles: no limit, LDS = what the reduction needs
    # (eight partials at 1024 to 6143 workgroups: the kernel for two wavefronts per SIMD, reported as 2, no LDS padding)
    (dict(nranks=8, tokens=1023, hidden=8192), 0, (256 * 4 * 8 + 1024) * 4),
    (dict(nranks=4, tokens=6143, hidden=8192), 0, (256 * 4 * 8 + 1024) * 4),
    (dict(nranks=2, tokens=32768, hidden=8192), 0, (256 * 4 * 8 + 1024) * 4),
    (dict(nranks=8, tokens=32768, hidden=8192, algo=_capi.ALGO_STAGED), 0, (256 * 4 * 8 + 1024) * 4),
    # long launches: about 128 KiB of loads in flight per CU, never fewer than two workgroups or eight wavefronts
    (dict(nranks=8, tokens=6144, hidden=8192), 2, 80896),                                    # 144 KiB per workgroup
    (dict(nranks=4, tokens=32768, hidden=8192), 2, 80896),                                   # 80 KiB per workgroup
    (dict(nranks=4, tokens=32768, hidden=5120, dtype=_capi.F16, quant=_capi.QUANT_INT8_TOKEN), 3, 53504),  # 3 wavefronts each
    (dict(nranks=4, tokens=8192, hidden=7168, quant=_capi.QUANT_FP8_GROUP), 3, 53504),      # twelve wavefronts for group scales
    (dict(nranks=4, tokens=8192, hidden=7168, quant=_capi.QUANT_FP8_TOKEN), 2, 80896),
    (dict(nranks=4, tokens=8191, hidden=7168, quant=_capi.QUANT_FP8_TOKEN), 0, (256 * 4 * 8 + 1024) * 4),   # four partials: from 8192
    (dict(nranks=8, tokens=32768, hidden=1024), 4, 39936),                                   # 2 rows x 18 KiB per workgroup
    (dict(nranks=4, tokens=16384, hidden=2048), 6, 26112),
    (dict(nranks=8, tokens=32768, hidden=2048, dtype=_capi.F64), 0, (1024 * 2 + 1024) * 4),   # doubles: 2 per vector, 1024 threads
    # the per-call override
    (dict(nranks=8, tokens=16, hidden=1024, workgroups_per_cu=1), 1, 162816),
    (dict(nranks=8, tokens=16, hidden=1024, workgroups_per_cu=8), 8, 19456),
    (dict(nranks=8, tokens=32768, hidden=8192, workgroups_per_cu=-1), 0, (256 * 4 * 8 + 1024) * 4),
    # a request beyond what the geometry's own LDS admits: the plan reports what the launch enforces (4, not 8)
    (dict(nranks=8, tokens=32768, hidden=8192, workgroups_per_cu=8), 4, (256 * 4 * 8 + 1024) * 4),
])
def test_plan_workgroups_per_cu(kw, limit, lds):
    """The limit on resident workgroups per compute unit and the dynamic LDS that enforces it."""
    _needs_256_compute_units()
    p = _plan(**kw)
    assert (p.workgroups_per_cu, p.lds_bytes) == (limit, lds)
    if limit:   # `limit` workgroups of this LDS (plus the kernels' 64 static bytes) fit 160 KiB, one more does not
        assert limit * (lds + 64) <= 160 * 1024 < (limit + 1) * (lds + 64)


@pytest.mark.parametrize("kw,limit", [
    (dict(nranks=8, tokens=2048, hidden=8192, quant=_capi.QUANT_FP8_TOKEN), 2),                     # the benchmark's c3
    (dict(nranks=8, tokens=1024, hidden=8192, dtype=_capi.F16, quant=_capi.QUANT_INT8_TOKEN), 2),  # from 4 workgroups per CU
    (dict(nranks=8, tokens=4096, hidden=2048, quant=_capi.QUANT_FP8_TOKEN), 2),                     # 4 rows per workgroup: 1024 workgroups
    (dict(nranks=8, tokens=2048, hidden=8192, quant=_capi.QUANT_FP8_GROUP), 2),
    (dict(nranks=8, tokens=2048, hidden=8192), 2),                                                   # T-typed output
    (dict(nranks=8, tokens=2048, hidden=4096, dtype=_capi.F32, quant=_capi.QUANT_FP8_TOKEN), 2),
    (dict(nranks=8, tokens=1023, hidden=8192, quant=_capi.QUANT_FP8_TOKEN), 0),
    (dict(nranks=8, tokens=2048, hidden=5120, quant=_capi.QUANT_FP8_TOKEN), 0),                     # one vector per thread
    (dict(nranks=8, tokens=2048, hidden=2048, dtype=_capi.F64), 0),
    (dict(nranks=4, tokens=2048, hidden=8192, quant=_capi.QUANT_FP8_TOKEN), 0),
    (dict(nranks=8, tokens=2048, hidden=8192, quant=_capi.QUANT_FP8_TOKEN, workgroups_per_cu=-1), 0),
    (dict(nranks=8, tokens=2048, hidden=8192, quant=_capi.QUANT_FP8_TOKEN, algo=_capi.ALGO_STAGED), 0),
])
def test_plan_picks_the_two_wavefronts_per_simd_kernel(kw, limit):
    """Eight partials, four vectors per thread, 4 to 24 workgroups per CU and no limit asked for: the plan reports two
    workgroups per CU (the kernel's registers) and leaves the LDS as the geometry needs it."""
    _needs_256_compute_units()
    p = _plan(**kw)
    assert p.workgroups_per_cu == limit
    unpadded = dict(kw)
    unpadded["workgroups_per_cu"] = -1
    assert p.lds_bytes == _plan(**unpadded).lds_bytes


@pytest.mark.parametrize("kw", [dict(workgroups_per_cu=9), dict(workgroups_per_cu=-2)])
def test_plan_rejects_workgroup_limits_out_of_range(kw):
    with pytest.raises(_capi.TdeError) as err:
        _plan(**kw)
    assert err.value.status == _capi.EINVAL


def test_plan_rejects_nonzero_reserved_field():
    prob = _capi.make_problem(_capi.BF16, 8, 16, 1024, 1e-6)
    prob.reserved = 1
    assert _capi.load().tde_plan(ctypes.byref(prob), ctypes.byref(_capi.PlanOut())) == _capi.EINVAL

