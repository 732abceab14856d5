"""``mi355q_w4a16_gemm_noalloc`` -- the W4A16 GEMM for callers that cannot allocate -- against
``mi355q_w4a16_gemm`` through the C ABI: bit-identical outputs (same kernels, same split-K plan),
within rtol = atol = 1e-2 of the CPU oracle, on calls in a row that share the fixed scratch array,
each smaller than the one before, and a clear error for a shape whose plan does not fit the array."""
import numpy as np
import pytest
import torch

from oracle import w4 as ow4

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _case(seed, M, K, N, g=128):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    return q, z, s, x


def _both(lib, _lib, rt, rearrange, q, z, s, x, g=128):
    M, K = x.shape
    N = q.shape[1]
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    xd, sd = dev(x), dev(s)
    ws_bytes = lib.mi355q_w4a16_workspace_bytes(M, K, N)
    ws = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    ref = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    st = rt.stream_ptr()
    _lib.check(lib.mi355q_w4a16_gemm(ref.data_ptr(), xd.data_ptr(), w.data_ptr(), sd.data_ptr(), zp.data_ptr(),
                                     _lib.ZP_PACKED, None, M, K, N, g, _lib.F16, ws.data_ptr(), ws.numel(), st),
               "w4a16_gemm")
    _lib.check(lib.mi355q_w4a16_gemm_noalloc(got.data_ptr(), xd.data_ptr(), w.data_ptr(), sd.data_ptr(),
                                             zp.data_ptr(), _lib.ZP_PACKED, None, M, K, N, g, _lib.F16, st),
               "w4a16_gemm_noalloc")
    torch.cuda.synchronize()
    return ref, got


def test_noalloc_entry_point_matches_the_workspace_one_on_calls_in_a_row():
    from vllm_gcu_amd import _lib
    from vllm_gcu_amd.kernels import _runtime as rt
    from vllm_gcu_amd.kernels.quantization import rearrange
    lib = _lib.load()
    assert lib.mi355q_w4a16_noalloc_scratch_bytes() == 32 << 20
    # largest first: cross-workgroup split-K of the streaming kernel (arrival counters + partial
    # tiles in the scratch array), then the MFMA kernel's split-K partials, then smaller launches that
    # find the earlier calls' contents in the array
    shapes = [(16, 14336, 4096), (128, 4096, 4096), (16, 8192, 2048), (8, 4096, 1024), (1, 2048, 512)]
    for i, (M, K, N) in enumerate(shapes):
        print(f"case noalloc M={M} K={K} N={N}", flush=True)
        q, z, s, x = _case(100 + i, M, K, N)
        ref, got = _both(lib, _lib, rt, rearrange, q, z, s, x)
        assert torch.isfinite(got).all()
        assert torch.equal(ref.view(torch.int16), got.view(torch.int16)), (M, K, N)
        want = ow4.w4a16_gemm(x.astype(np.float32), q, z, s.astype(np.float32), 128)
        np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # the same shape twice more: the kernels must have left the counters at zero
    q, z, s, x = _case(7, 16, 14336, 4096)
    a, b = _both(lib, _lib, rt, rearrange, q, z, s, x)
    c, d = _both(lib, _lib, rt, rearrange, q, z, s, x)
    assert torch.equal(a.view(torch.int16), b.view(torch.int16)) and torch.equal(b.view(torch.int16), d.view(torch.int16))


def test_noalloc_entry_point_in_a_captured_graph_replays_with_new_inputs():
    """After one eager call (which looks the scratch array up), the entry point is captured into a HIP
    graph on a side stream and replayed with new activations each time; other eager no-alloc calls run
    on the same stream between the replays and leave their contents in the shared array."""
    from vllm_gcu_amd import _lib
    from vllm_gcu_amd.kernels import _runtime as rt
    from vllm_gcu_amd.kernels.quantization import rearrange
    lib = _lib.load()
    M, K, N, g = 16, 14336, 4096, 128                       # cross-workgroup split-K: counters + partial tiles
    q, z, s, x = _case(21, M, K, N)
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    xd, sd = dev(x), dev(s)
    q2, z2, s2, x2 = _case(22, 8, 8192, 2048)
    w2, zp2 = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q2)), dev(ow4.gptq_pack_zeros(z2)))
    x2d, s2d = dev(x2), dev(s2)
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    out2 = torch.empty((8, 2048), dtype=torch.float16, device="cuda")
    ws = torch.zeros(max(lib.mi355q_w4a16_workspace_bytes(M, K, N), 16), dtype=torch.uint8, device="cuda")
    ref = torch.empty_like(out)

    def noalloc(o, xx, ww, ss, zz, m, k, n):
        _lib.check(lib.mi355q_w4a16_gemm_noalloc(o.data_ptr(), xx.data_ptr(), ww.data_ptr(), ss.data_ptr(),
                                                 zz.data_ptr(), _lib.ZP_PACKED, None, m, k, n, g, _lib.F16,
                                                 rt.stream_ptr()), "w4a16_gemm_noalloc")

    print("case noalloc captured graph", flush=True)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        noalloc(out, xd, w, sd, zp, M, K, N)                # warm-up outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            noalloc(out, xd, w, sd, zp, M, K, N)
        side.synchronize()
        rng = np.random.default_rng(23)
        for i in range(3):
            xd.copy_(dev(rng.standard_normal((M, K)).astype(np.float16)))
            out.fill_(float("nan"))
            side.synchronize()
            graph.replay()
            side.synchronize()
            got = out.clone()
            noalloc(out2, x2d, w2, s2d, zp2, 8, 8192, 2048)  # another shape through the same array
            _lib.check(lib.mi355q_w4a16_gemm(ref.data_ptr(), xd.data_ptr(), w.data_ptr(), sd.data_ptr(),
                                             zp.data_ptr(), _lib.ZP_PACKED, None, M, K, N, g, _lib.F16,
                                             ws.data_ptr(), ws.numel(), rt.stream_ptr()), "w4a16_gemm")
            side.synchronize()
            assert torch.isfinite(got).all()
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"replay {i}"
    torch.cuda.synchronize()


def test_noalloc_entry_point_rejects_what_does_not_fit():
    from vllm_gcu_amd import _lib
    from vllm_gcu_amd.kernels import _runtime as rt
    lib = _lib.load()
    # 128 rows x 16384 columns: the MFMA kernel's plan splits K four ways -> 33.5 MB of partial tiles
    M, K, N = 128, 4096, 16384
    out = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    x = torch.zeros((M, K), dtype=torch.float16, device="cuda")
    w = torch.zeros((K // 8, N), dtype=torch.int32, device="cuda")
    s = torch.zeros((K // 128, N), dtype=torch.float16, device="cuda")
    rc = lib.mi355q_w4a16_gemm_noalloc(out.data_ptr(), x.data_ptr(), w.data_ptr(), s.data_ptr(), None, _lib.ZP_NONE,
                                       None, M, K, N, 128, _lib.F16, rt.stream_ptr())
    assert rc != 0
    msg = lib.mi355q_last_error().decode()
    assert "scratch" in msg and "mi355q_w4a16_gemm" in msg
    torch.cuda.synchronize()
