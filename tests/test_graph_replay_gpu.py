"""The GEMM launches that keep state between calls -- arrival counters that the last workgroup of a
split-K exchange resets, partial-sum workspaces shared by every layer, the persistent int8 tile
kernel's tile stream -- replayed from a captured HIP graph: every replay, with new inputs written
between replays and eager launches of other shapes in between (on the capture stream, so they use the
same workspace), must
give exactly the bits of an eager launch on the same inputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _replay_against_eager(run, inputs, fresh_inputs, between=None, replays=3):
    """run() -> output tensor computed from the tensors in `inputs`; fresh_inputs(i) -> replacement
    values for them.  Everything -- warm-up, capture, replays, the eager launches in between and the
    eager reference -- runs on ONE side stream, so all of it shares that stream's workspace and
    arrival counters (the workspace is keyed by device and stream)."""
    from vllm_gcu_amd.kernels import _runtime as rt
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run()                                        # warm-up: workspaces are allocated outside the capture
        side.synchronize()
        ws_at_capture = rt.workspace(torch.device("cuda", torch.cuda.current_device()), 1).data_ptr()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out = run()
        side.synchronize()
        for i in range(replays):
            for t, v in zip(inputs, fresh_inputs(i)):
                t.copy_(v, non_blocking=False)
            side.synchronize()
            graph.replay()
            side.synchronize()
            got = out.clone()
            if between is not None:
                between()                            # other launches on the same workspace / counters
            want = run()
            side.synchronize()
            assert rt.workspace(torch.device("cuda", torch.cuda.current_device()), 1).data_ptr() == ws_at_capture
            assert torch.isfinite(got).all()
            assert torch.equal(got, want), f"replay {i} differs from the eager launch"
    torch.cuda.synchronize()


@pytest.mark.parametrize("M", [16, 32, 128, 512])
def test_w4a16_split_k_launches_replay(M):
    """K = 14336, N = 4096 (the down projection): split-K exchange between workgroups for up to 32
    rows, narrow tiles with a reduction kernel at 128, wide tiles with one at 512."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    K, N, g = 14336, 4096, 128
    gen = torch.Generator(device="cpu").manual_seed(M)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=gen).cuda()
    zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, generator=gen).cuda()
    sc = (torch.rand(K // g, N, generator=gen) * 0.009 + 0.001).half().cuda()
    x = torch.randn(M, K, generator=gen).half().cuda()
    other_x = torch.randn(48, 4096, generator=gen).half().cuda()
    other_qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (4096 // 8, 6144), dtype=torch.int32, generator=gen).cuda()
    other_zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (4096 // g, 6144 // 8), dtype=torch.int32, generator=gen).cuda()
    other_sc = (torch.rand(4096 // g, 6144, generator=gen) * 0.009 + 0.001).half().cuda()
    print(f"case graph replay w4a16 down M={M}", flush=True)
    _replay_against_eager(
        lambda: ops.w4a16_gemm(x, qw, sc, zp, None, g),
        [x], lambda i: [torch.randn(M, K, generator=gen).half()],
        between=lambda: ops.w4a16_gemm(other_x, other_qw, other_sc, other_zp, None, g))


def test_replay_survives_a_larger_eager_plan_on_the_capture_stream():
    """A graph captured at a decode size holds the workspace's address for its partial tiles and arrival
    counters.  An eager prefill-sized launch on the same stream afterwards needs a far larger plan; the
    workspace must neither move nor be freed, and the replays must still equal eager."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    K, N, g = 14336, 4096, 128
    gen = torch.Generator(device="cpu").manual_seed(77)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=gen).cuda()
    zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, generator=gen).cuda()
    sc = (torch.rand(K // g, N, generator=gen) * 0.009 + 0.001).half().cuda()
    x = torch.randn(16, K, generator=gen).half().cuda()
    big = torch.randn(1100, K, generator=gen).half().cuda()       # wide tiles, K split three ways: 54 MB of partials
    print("case graph replay w4a16 decode graph, prefill eager in between", flush=True)
    _replay_against_eager(
        lambda: ops.w4a16_gemm(x, qw, sc, zp, None, g),
        [x], lambda i: [torch.randn(16, K, generator=gen).half()],
        between=lambda: ops.w4a16_gemm(big, qw, sc, zp, None, g))


@pytest.mark.parametrize("M,K,N", [(300, 4096, 7168), (1024, 512, 16384)])
def test_bf16_rows_staged_in_the_workspace_replay(M, K, N):
    """bf16 prefill stages its rows as fp16 in the stream's workspace (64-row tiles at 300 rows, the
    512-column ring workgroups with their scale maxima at 1024 x 16384).  Between the replays another bf16
    launch of another height overwrites the staging area and a split-K launch the partial tiles before it."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    g = 128
    gen = torch.Generator(device="cpu").manual_seed(M)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 8, N), dtype=torch.int32, generator=gen).cuda()
    zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // g, N // 8), dtype=torch.int32, generator=gen).cuda()
    sc = (torch.rand(K // g, N, generator=gen) * 0.009 + 0.001).bfloat16().cuda()
    x = torch.randn(M, K, generator=gen).bfloat16().cuda()
    other = (torch.randn(777, K, generator=gen) * 1000.0).bfloat16().cuda()
    small = torch.randn(128, K, generator=gen).bfloat16().cuda()
    print(f"case graph replay w4a16 bf16 staged M={M} K={K} N={N}", flush=True)

    def between():
        ops.w4a16_gemm(other, qw, sc, zp, None, g)
        ops.w4a16_gemm(small, qw, sc, zp, None, g)
    _replay_against_eager(
        lambda: ops.w4a16_gemm(x, qw, sc, zp, None, g),
        [x], lambda i: [(torch.randn(M, K, generator=gen) * (4.0 ** i)).bfloat16()],
        between=between)


def test_workspace_refuses_to_allocate_under_capture(monkeypatch):
    from vllm_gcu_amd.kernels import _runtime as rt
    dev = torch.device("cuda", torch.cuda.current_device())
    rt.workspace(dev, 1)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    held = rt.workspace(dev, 1)                                   # already there: fine under capture
    with pytest.raises(RuntimeError, match="before capturing"):
        rt.workspace(dev, held.numel() + 1)


def test_grouped_w4a16_split_k_replay():
    """Grouped W4A16 GEMM with a long K and few column tiles (the second GEMM of a Mixtral layer at a
    reduced width): K split over the grid, partial sums in the operator's workspace, routing weights
    applied by the reduction."""
    from vllm_gcu_amd.kernels import fused_moe
    E, K, N, g, slots = 8, 14336, 1024, 128, 512
    gen = torch.Generator(device="cpu").manual_seed(5)
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (E, K // 8, N), dtype=torch.int32, generator=gen).cuda()
    zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (E, K // g, N // 8), dtype=torch.int32, generator=gen).cuda()
    sc = (torch.rand(E, K // g, N, generator=gen) * 0.009 + 0.001).half().cuda()
    a = torch.randn(slots, K, generator=gen).half().cuda()
    ids = torch.randint(0, E, (slots, 1), dtype=torch.int32, generator=gen).cuda()
    tw = (torch.rand(slots, 1, generator=gen) * 0.9 + 0.1).float().cuda()
    sorted_ids, expert_ids, npp = fused_moe.moe_align_block_size(ids, 64, E)
    out = torch.empty(slots, 1, N, dtype=torch.float16, device="cuda")
    kw = dict(use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=True, block_shape=[0, g])

    def run():
        fused_moe.invoke_fused_moe_kernel(a, qw, out, None, sc, zp, tw, ids, sorted_ids, expert_ids, npp, True, 1,
                                          {"BLOCK_SIZE_M": 64}, **kw)
        return out

    print("case graph replay grouped w4a16 split-K", flush=True)
    _replay_against_eager(run, [a], lambda i: [torch.randn(slots, K, generator=gen).half()])


def test_w8a8_int8_tile_and_streaming_kernels_replay():
    """Persistent int8 tile kernel (300 rows) and the weight-streaming int8 kernel (16 rows)."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    K, N = 1024, 1792
    gen = torch.Generator(device="cpu").manual_seed(9)
    w = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=gen).cuda()
    ws = (torch.rand(N, generator=gen) * 0.019 + 0.001).float().cuda()
    for M in (300, 16):
        x = torch.randn(M, K, generator=gen).half().cuda()

        def run():
            xq, xs, _ = ops.scaled_int8_quant(x)
            return ops.cutlass_scaled_mm(xq, w.t(), xs, ws, torch.float16, None)

        print(f"case graph replay w8a8 M={M}", flush=True)
        _replay_against_eager(run, [x], lambda i: [torch.randn(M, K, generator=gen).half()])


def _moe_layer(mode):
    from vllm_gcu_amd.kernels.modular_experts import TritonExpertsPad
    from vllm_gcu_amd.kernels.modular_kernel import FusedMoEModularKernel
    from vllm_gcu_amd.kernels.prepare_finalize import MoEPrepareAndFinalizeNoEP
    if mode == "w4a16":
        fe = TritonExpertsPad(use_int4_w4a16=True, block_shape=[0, 128])
    else:
        fe = TritonExpertsPad(use_fp8_w8a8=True, block_shape=[128, 128])
    return FusedMoEModularKernel(MoEPrepareAndFinalizeNoEP(), fe)


@pytest.mark.parametrize("tokens", [16, 200])
def test_fused_moe_w4a16_layer_replays_with_new_routing(tokens):
    """A whole W4A16 expert layer (routing, align, two grouped GEMMs, gate, sum) captured once and replayed
    with new activations and new router logits: the routing -- which blocks exist, which experts they
    belong to, how many slots are valid -- is read on the device, so every replay must equal eager."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    E, T, H, I, g = 8, 2, 512, 1024, 128
    gen = torch.Generator(device="cpu").manual_seed(tokens)

    def rnd(*shape):
        return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, dtype=torch.int32, generator=gen).cuda()

    w13, z13 = rnd(E, H // 8, 2 * I), rnd(E, H // g, 2 * I // 8)
    w2, z2 = rnd(E, I // 8, H), rnd(E, I // g, H // 8)
    s13 = (torch.rand(E, H // g, 2 * I, generator=gen) * 0.009 + 0.001).half().cuda()
    s2 = (torch.rand(E, I // g, H, generator=gen) * 0.009 + 0.001).half().cuda()
    x = torch.randn(tokens, H, generator=gen).half().cuda()
    logits = torch.randn(tokens, E, generator=gen).cuda()
    moe = _moe_layer("w4a16")

    def run():
        tw, ids = ops.fused_topk(x, logits, T, True)
        return moe(x, w13, w2, tw, ids, w1_scale=s13, w2_scale=s2, w1_zp=z13, w2_zp=z2)

    print(f"case graph replay fused moe w4a16 tokens={tokens}", flush=True)
    _replay_against_eager(run, [x, logits],
                          lambda i: [torch.randn(tokens, H, generator=gen).half(), torch.randn(tokens, E, generator=gen) * (1 + 3 * i)])


def test_fused_moe_fp8_block_layer_replays_with_new_routing():
    """The same for a block-scaled fp8 layer with grouped routing (quantisers, K-contiguous grouped GEMMs)."""
    from vllm_gcu_amd.kernels import fused_moe
    E, T, H, I, tokens = 32, 4, 512, 256, 48
    gen = torch.Generator(device="cpu").manual_seed(7)

    def rnd_fp8(*shape):
        b = torch.randint(0, 256, shape, dtype=torch.uint8, generator=gen)
        b[(b & 0x7f) == 0x7f] = 0                       # no NaN codes
        return b.cuda().view(torch.float8_e4m3fn)

    w13, w2 = rnd_fp8(E, 2 * I, H), rnd_fp8(E, H, I)
    s13 = (torch.rand(E, 2 * I // 128, H // 128, generator=gen) * 1e-3 + 1e-4).cuda()
    s2 = (torch.rand(E, H // 128, I // 128, generator=gen) * 1e-3 + 1e-4).cuda()
    x = torch.randn(tokens, H, generator=gen).to(torch.bfloat16).cuda()
    logits = torch.randn(tokens, E, generator=gen).cuda()
    moe = _moe_layer("fp8")

    def run():
        tw, ids = fused_moe.grouped_topk(x, logits, T, True, 4, 2, "softmax", None)
        return moe(x, w13, w2, tw, ids, w1_scale=s13, w2_scale=s2)

    print("case graph replay fused moe fp8", flush=True)
    _replay_against_eager(run, [x, logits],
                          lambda i: [torch.randn(tokens, H, generator=gen).to(torch.bfloat16), torch.randn(tokens, E, generator=gen) * (1 + 2 * i)])
