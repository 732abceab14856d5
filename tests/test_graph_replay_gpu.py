"""The GEMM launches that keep state between calls -- arrival counters that the last workgroup of a
split-K exchange resets, partial-sum workspaces shared by every layer, the persistent int8 tile
kernel's tile stream -- replayed from a captured HIP graph: every replay, with new inputs written
between replays and eager launches of other shapes in between (they use the same workspace), must
give exactly the bits of an eager launch on the same inputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _replay_against_eager(run, inputs, fresh_inputs, between=None, replays=3):
    """run() -> output tensor computed from the tensors in `inputs`; fresh_inputs(i) -> replacement
    values for them."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run()                                        # warm-up: workspaces are allocated outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out = run()
    torch.cuda.synchronize()
    for i in range(replays):
        for t, v in zip(inputs, fresh_inputs(i)):
            t.copy_(v)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        if between is not None:
            between()                                # other launches on the same workspace / counters
        want = run()
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), f"replay {i} differs from the eager launch"


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
