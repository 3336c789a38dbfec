"""GPU: the reference's own call sequence (test/test_all_reduce_fusion.py:40-61) on one GPU:
setup_env -> get_workspace -> allreduce_rms, with the peers' partials placed into the workspace slots."""
import pytest
import torch

from oracle import eager

from helpers import bits_equal, check_against_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tde(cuda_device):
    import torch_dist_ext_amd as m
    return m


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("tokens", [129, 128])
def test_reference_call_sequence(tde, cuda_device, dtype, tokens):
    world_size, hidden, eps, rank = 4, 1024, 1e-6, 1
    print("case call-sequence", dtype, tokens, flush=True)
    g = torch.Generator().manual_seed(tokens)
    wide = torch.float64 if dtype == torch.float64 else torch.float32
    allreduce_in = torch.randn((world_size, tokens, hidden), generator=g, dtype=wide).to(dtype)
    residual_in = torch.randn((tokens, hidden), generator=g, dtype=wide).to(dtype)
    gamma = torch.randn((hidden,), generator=g, dtype=wide).to(dtype)
    want = eager.reduce_rms(allreduce_in, residual_in, gamma, eps)

    tde.setup_env(rank, world_size)
    local_in = allreduce_in[rank].to(cuda_device)
    for r in range(world_size):
        if r != rank:
            tde.set_peer_partial(r, allreduce_in[r].to(cuda_device))
    workspace = tde.get_workspace(local_in)
    assert workspace.dtype == torch.uint8 and workspace.numel() == (3 * world_size + 5) * 8 and workspace.is_cuda
    norm_out, residual_out = tde.allreduce_rms(rank, world_size, local_in, residual_in.to(cuda_device),
                                               gamma.to(cuda_device), eps, workspace)
    torch.cuda.synchronize()
    got = {"norm_out": norm_out.cpu(), "residual_out": residual_out.cpu()}
    print("  stats", check_against_oracle(got, want, "none", gamma=gamma, eps=eps), flush=True)


@pytest.mark.parametrize("mode,quant", [(1, "fp8_token"), (2, "fp8_group"), (3, "int8_token")])
def test_quant_op_through_workspace(tde, cuda_device, mode, quant):
    world_size, tokens, hidden, eps, rank = 8, 70, 4096, 1e-5, 5
    print("case quant-op", quant, flush=True)
    p, r, g = eager.make_inputs(world_size, tokens, hidden, torch.bfloat16, 0.5, seed=31)
    want = eager.reduce_rms(p, r, g, eps, quant)
    tde.setup_env(rank, world_size, max_size_in_bytes=tokens * hidden * 2)
    for k in range(world_size):
        if k != rank:
            tde.peer_partial(k, p[k].to(cuda_device)).copy_(p[k].to(cuda_device))
    ws = tde.get_workspace(p[rank].to(cuda_device))
    q, s, res_out, norm = torch.ops.torch_dist_ext.allreduce_rms_quant(
        rank, world_size, p[rank].to(cuda_device), r.to(cuda_device), g.to(cuda_device), eps, ws, mode, True)
    torch.cuda.synchronize()
    got = {"q": q.cpu(), "scale": s.cpu(), "residual_out": res_out.cpu(), "norm_out": norm.cpu()}
    print("  stats", check_against_oracle(got, want, quant, gamma=g, eps=eps), flush=True)
    q2, s2, res2, norm2 = torch.ops.torch_dist_ext.allreduce_rms_quant(
        rank, world_size, p[rank].to(cuda_device), r.to(cuda_device), g.to(cuda_device), eps, ws, mode, False)
    assert norm2.numel() == 0 and bits_equal(q2.cpu(), got["q"]) and bits_equal(s2.cpu(), got["scale"])


def test_local_list_op_and_staged(tde, cuda_device):
    p, r, g = eager.make_inputs(4, 50, 2048, torch.float16, 1.0, seed=32)
    want = eager.reduce_rms(p, r, g, 1e-6, "int8_token")
    parts = [p[i].to(cuda_device) for i in range(4)]
    a = tde.reduce_rms(parts, r.to(cuda_device), g.to(cuda_device), 1e-6, tde.QUANT_INT8_TOKEN, write_norm=True)
    b = tde.reduce_rms(parts, r.to(cuda_device), g.to(cuda_device), 1e-6, tde.QUANT_INT8_TOKEN, write_norm=True,
                       algo=tde.ALGO_STAGED)
    torch.cuda.synchronize()
    got = {k: v.cpu() for k, v in a.items()}
    check_against_oracle(got, want, "int8_token", gamma=g, eps=1e-6)
    for k in a:
        assert bits_equal(a[k].cpu(), b[k].cpu()), k


def test_error_paths_raise(tde, cuda_device):
    x = torch.zeros((4, 256), dtype=torch.bfloat16, device=cuda_device)
    g = torch.ones((256,), dtype=torch.bfloat16, device=cuda_device)
    tde.setup_env(0, 2, max_size_in_bytes=4096)
    ws = tde.get_workspace(x)
    with pytest.raises(RuntimeError, match="nranks must be 2, 4 or 8"):
        tde.allreduce_rms_fusion_impl(0, 3, x, x, g, torch.empty_like(x), torch.empty_like(x), 1e-6,
                                      torch.zeros(200, dtype=torch.uint8, device=cuda_device))
    with pytest.raises(RuntimeError, match="dtype"):
        tde.allreduce_rms_fusion_impl(0, 2, x, x.float(), g, torch.empty_like(x), torch.empty_like(x), 1e-6, ws)
    with pytest.raises(RuntimeError, match="exceed the slot size"):
        tde.peer_partial(1, torch.zeros((64, 256), dtype=torch.bfloat16, device=cuda_device))
    with pytest.raises(RuntimeError, match="rank"):
        tde.CommWorkspace(5, 4, 256, 4096)
    # rows that do not fit the workspace slots (4096 bytes here) are refused, not read past the slot
    big = torch.zeros((16, 256), dtype=torch.bfloat16, device=cuda_device)
    with pytest.raises(RuntimeError, match="workspace slots hold 4096"):
        tde.allreduce_rms_fusion_impl(0, 2, big, big, g, torch.empty_like(big), torch.empty_like(big), 1e-6, ws)
    # so is a table that no live workspace handed out
    with pytest.raises(RuntimeError, match="not a pointer table handed out"):
        tde.allreduce_rms_fusion_impl(0, 2, x, x, g, torch.empty_like(x), torch.empty_like(x), 1e-6, ws.clone())
    y = torch.zeros((4, 8200), dtype=torch.bfloat16, device=cuda_device)
    with pytest.raises(RuntimeError, match="hidden_dim <= 8192"):   # the reference asserts (torch_dist_ext/__init__.py:68)
        tde.allreduce_rms(0, 2, y, y, torch.ones(8200, dtype=torch.bfloat16, device=cuda_device), 1e-6, ws)


def test_workspace_table_is_uploaded_once_and_ops_trace(tde, cuda_device):
    """get_workspace hands out one cached device table (no per-call host-to-device copy), and the custom
    ops run under torch.compile (aot_eager: traced through their fake implementations, no code generation)."""
    world_size, tokens, hidden, eps, rank = 2, 16, 1024, 1e-6, 0
    p, r, g = eager.make_inputs(world_size, tokens, hidden, torch.bfloat16, 1.0, seed=51)
    tde.setup_env(rank, world_size, max_size_in_bytes=tokens * hidden * 2)
    tde.set_peer_partial(1, p[1].to(cuda_device))
    x = p[0].to(cuda_device)
    ws1 = tde.get_workspace(x)
    ws2 = tde.get_workspace(x)
    assert ws1.data_ptr() == ws2.data_ptr()
    rd, gd = r.to(cuda_device), g.to(cuda_device)

    def step(x, rd, gd, ws):
        n, ro = torch.ops.torch_dist_ext.allreduce_rms(rank, world_size, x, rd, gd, eps, ws)
        return n * 2, ro

    want = eager.reduce_rms(p, r, g, eps)
    compiled = torch.compile(step, backend="aot_eager", fullgraph=True)
    n2, ro = compiled(x, rd, gd, ws1)
    torch.cuda.synchronize()
    assert bits_equal(ro.cpu(), want["residual_out"])
    assert bits_equal(n2.cpu(), (want["norm_out"] * 2))


def test_static_quant_op(tde, cuda_device):
    p, r, g = eager.make_inputs(4, 20, 1024, torch.bfloat16, 1.0, seed=52)
    parts = [p[i].to(cuda_device) for i in range(4)]
    out = tde.reduce_rms(parts, r.to(cuda_device), g.to(cuda_device), 1e-6, tde.QUANT_FP8_STATIC, write_norm=True,
                         static_scale=0.01)
    torch.cuda.synchronize()
    assert "scale" not in out
    assert bits_equal(out["q"].cpu(), eager.quant_fp8_static(out["norm_out"].cpu(), 0.01))
    tde.setup_env(0, 4, max_size_in_bytes=20 * 1024 * 2)
    for k in range(1, 4):
        tde.set_peer_partial(k, parts[k])
    ws = tde.get_workspace(parts[0])
    q, s, ro, no = torch.ops.torch_dist_ext.allreduce_rms_quant(0, 4, parts[0], r.to(cuda_device), g.to(cuda_device), 1e-6, ws,
                                                               tde.QUANT_FP8_STATIC, False, 0.01)
    torch.cuda.synchronize()
    assert s.numel() == 0 and no.numel() == 0 and bits_equal(q.cpu(), out["q"].cpu())


def test_slot_alias_keeps_the_workspace_alive(tde, cuda_device):
    """A tensor returned by peer_partial/stage aliases workspace memory and must keep it allocated after
    the workspace object itself is dropped; a table whose workspace is gone is refused."""
    import gc
    ref = torch.zeros((8, 512), dtype=torch.bfloat16, device=cuda_device)
    ws = tde.CommWorkspace(0, 2, 256, 8 * 512 * 2)
    table = ws.get_workspace(ref)
    alias = ws.peer_partial(1, ref)
    del ws
    gc.collect()
    alias.fill_(3.0)
    torch.cuda.synchronize()
    assert float(alias.float().sum().item()) == 3.0 * 8 * 512
    g = torch.ones((512,), dtype=torch.bfloat16, device=cuda_device)
    # the alias still owns the workspace, so its table stays valid
    out = torch.empty_like(ref)
    tde.allreduce_rms_fusion_impl(0, 2, ref, ref, g, torch.empty_like(ref), out, 1e-6, table)
    torch.cuda.synchronize()
    del alias
    gc.collect()
    with pytest.raises(RuntimeError, match="not a pointer table handed out"):
        tde.allreduce_rms_fusion_impl(0, 2, ref, ref, g, torch.empty_like(ref), out, 1e-6, table)


def test_ops_under_default_torch_compile(tde, cuda_device):
    """The custom ops inside a graph compiled with torch's default backend, which generates the surrounding
    elementwise code itself (skipped where that backend cannot build on the host)."""
    pytest.importorskip("triton")
    from torch._dynamo.exc import BackendCompilerFailed
    import torch._inductor.config as inductor_config
    inductor_config.compile_threads = 1      # compile in this process: no pool of worker processes
    world_size, tokens, hidden, eps, rank = 2, 16, 1024, 1e-6, 0
    p, r, g = eager.make_inputs(world_size, tokens, hidden, torch.bfloat16, 1.0, seed=52)
    tde.setup_env(rank, world_size, max_size_in_bytes=tokens * hidden * 2)
    tde.set_peer_partial(1, p[1].to(cuda_device))
    x, rd, gd = p[0].to(cuda_device), r.to(cuda_device), g.to(cuda_device)
    ws = tde.get_workspace(x)

    def step(x, rd, gd, ws):
        q, s, ro, _ = torch.ops.torch_dist_ext.allreduce_rms_quant(rank, world_size, x, rd, gd, eps, ws,
                                                                    tde.QUANT_FP8_TOKEN, False)
        return q.float() * s.unsqueeze(-1), ro.float() + 1

    try:
        deq, ro1 = torch.compile(step, fullgraph=True)(x, rd, gd, ws)
    except BackendCompilerFailed as e:   # the code generator, not this library
        pytest.skip("default torch.compile backend unavailable here: %s" % str(e)[:200])
    torch.cuda.synchronize()
    want = eager.reduce_rms(p, r, g, eps, "fp8_token")
    assert torch.equal(ro1.cpu(), want["residual_out"].float() + 1)
    e_deq, e_ro1 = step(x, rd, gd, ws)
    assert torch.equal(deq, e_deq) and torch.equal(ro1, e_ro1)


def test_reference_test_body_under_the_reference_package_name(cuda_device):
    """The body of the reference's worker (test/test_all_reduce_fusion.py:42-61) with its own import line,
    `import torch_dist_ext`, on one GPU: setup_env, get_workspace, allreduce_rms, compared with the eager
    composition of the same file (:17-28, :72-76).  Only the peers' partials are placed by hand."""
    import torch_dist_ext
    world_size, num_tokens, hidden_dim, eps, rank = 4, 129, 1024, 1e-6, 0
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(99)
    allreduce_in = torch.randn((world_size, num_tokens, hidden_dim), generator=g).to(dtype)
    residual_in = torch.randn((num_tokens, hidden_dim), generator=g).to(dtype)
    weight = torch.randn((hidden_dim,), generator=g).to(dtype)
    want = eager.reduce_rms(allreduce_in, residual_in, weight, eps)
    torch_dist_ext.setup_env(rank, world_size)
    for r in range(1, world_size):
        torch_dist_ext.set_peer_partial(r, allreduce_in[r].to(cuda_device))
    local_in = allreduce_in[rank].to(cuda_device)
    workspace = torch_dist_ext.get_workspace(local_in)
    norm_out, residual_out = torch_dist_ext.allreduce_rms(rank, world_size, local_in, residual_in.to(cuda_device),
                                                          weight.to(cuda_device), eps, workspace)
    torch.cuda.synchronize()
    check_against_oracle({"norm_out": norm_out.cpu(), "residual_out": residual_out.cpu()}, want, "none", gamma=weight, eps=eps)


def test_torch_ops_inside_a_hip_graph(tde, cuda_device):
    """get_workspace outside the capture, allreduce_rms and allreduce_rms_quant inside it; the graph is replayed
    with new input contents several times, with eager work and synchronizations in between, and every replay is
    compared with the oracle."""
    world_size, tokens, hidden, eps, rank = 4, 96, 2048, 1e-5, 2
    tde.setup_env(rank, world_size, max_size_in_bytes=tokens * hidden * 2)
    p, r, g = eager.make_inputs(world_size, tokens, hidden, torch.bfloat16, 0.5, seed=41)
    local_in = p[rank].to(cuda_device)
    res_in, gamma = r.to(cuda_device), g.to(cuda_device)
    peers = {k: tde.peer_partial(k, local_in) for k in range(world_size) if k != rank}
    for k, t in peers.items():
        t.copy_(p[k].to(cuda_device))
    ws = tde.get_workspace(local_in)          # uploads the pointer table once, outside the capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):              # warm-up on the capture stream
        tde.allreduce_rms(rank, world_size, local_in, res_in, gamma, eps, ws)
        torch.ops.torch_dist_ext.allreduce_rms_quant(rank, world_size, local_in, res_in, gamma, eps, ws, tde.QUANT_FP8_TOKEN, False)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        norm_out, residual_out = tde.allreduce_rms(rank, world_size, local_in, res_in, gamma, eps, ws)
        q, scale, residual_out2, _ = torch.ops.torch_dist_ext.allreduce_rms_quant(
            rank, world_size, local_in, res_in, gamma, eps, ws, tde.QUANT_FP8_TOKEN, False)
    for replay in range(4):
        p2, r2, _ = eager.make_inputs(world_size, tokens, hidden, torch.bfloat16, 0.5, seed=50 + replay)
        local_in.copy_(p2[rank].to(cuda_device))
        res_in.copy_(r2.to(cuda_device))
        for k, t in peers.items():
            t.copy_(p2[k].to(cuda_device))
        for t in (norm_out, residual_out, residual_out2):
            t.fill_(float("nan"))
        q.view(torch.uint8).fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = eager.reduce_rms(p2, r2, g, eps, "fp8_token")
        check_against_oracle({"norm_out": norm_out.cpu(), "residual_out": residual_out.cpu()}, want, "none", gamma=g, eps=eps)
        assert bits_equal(residual_out2.cpu(), want["residual_out"])
        assert bits_equal(q.cpu(), want["q"]) and bits_equal(scale.cpu(), want["scale"])
        # eager work between replays
        eager_norm, _ = tde.allreduce_rms(rank, world_size, local_in, res_in, gamma, eps, ws)
        assert bits_equal(eager_norm.cpu(), want["norm_out"])

