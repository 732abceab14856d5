"""GPU parity of the W8A8 int8 path: quantisers and int32 accumulators are
bit-exact against the CPU oracle; scaled fp16/bf16 outputs within rtol 1e-2 /
atol 1e-2."""
import numpy as np
import pytest
import torch

from oracle import w8a8 as o8

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


@pytest.fixture(scope="module")
def ops():
    from vllm_gcu_amd.kernels import _custom_ops
    return _custom_ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 128), (37, 1000), (64, 8192)])
def test_dynamic_int8_quant_bit_exact(ops, dtype, M, K):
    print(f"case dyn-quant {M}x{K} {dtype}", flush=True)
    rng = np.random.default_rng(M * K)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    if M > 1:
        x[1] = 0                       # all-zero row: scale 0, q 0
        x[2, 5] = 40.0                 # outlier
    q, s, azp = ops.scaled_int8_quant(x.cuda())
    assert azp is None and q.dtype == torch.int8 and s.shape == (M, 1) and s.dtype == torch.float32
    qo, so = o8.dynamic_scaled_int8_quant(x.float().numpy())
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.array_equal(q.cpu().numpy(), qo)


def test_dynamic_int8_quant_3d_input(ops):
    x = torch.randn(3, 5, 256, dtype=torch.float16)
    q, s, _ = ops.scaled_int8_quant(x.cuda())
    qo, so = o8.dynamic_scaled_int8_quant(x.float().numpy().reshape(15, 256))
    assert q.shape == x.shape and s.shape == (15, 1)
    assert np.array_equal(q.cpu().numpy().reshape(15, 256), qo) and np.array_equal(s.cpu().numpy(), so)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_static_int8_quant_bit_exact(ops, dtype):
    rng = np.random.default_rng(1)
    x = torch.from_numpy((rng.standard_normal((33, 512)) * 3).astype(np.float32)).to(dtype)
    x[0, 0] = 1000.0
    x[0, 1] = -1000.0
    np_x = x.numpy() if dtype == torch.float32 else x.numpy().astype(np.float16)
    scale = torch.tensor(0.037, dtype=torch.float32)
    q, s, _ = ops.scaled_int8_quant(x.cuda(), scale.cuda())
    assert np.array_equal(q.cpu().numpy(), o8.static_scaled_int8_quant(np_x, scale.numpy()))
    ch = torch.from_numpy(rng.uniform(0.01, 0.1, 512).astype(np.float32))
    q, _, _ = ops.scaled_int8_quant(x.cuda(), ch.cuda())
    assert np.array_equal(q.cpu().numpy(), o8.static_scaled_int8_quant(np_x, ch.numpy()))


@pytest.mark.parametrize("M,K,N", [(1, 128, 4), (7, 256, 36), (300, 1024, 520), (256, 512, 256), (513, 2048, 1028)])
def test_int8_gemm_accumulators_bit_exact_both_layouts(ops, M, K, N):
    print(f"case i8 acc {M}x{K}x{N}", flush=True)
    rng = np.random.default_rng(M + K + N)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    x[0, :] = -128
    w_nk[0, :] = -127
    want = o8.int8_gemm_i32(x, np.ascontiguousarray(w_nk.T))
    # [K, N] view of an [N, K] checkpoint tensor (compressed-tensors path)
    acc = ops.int8_gemm_accumulators(dev(x), dev(w_nk).t())
    assert acc.dtype == torch.int32 and np.array_equal(acc.cpu().numpy(), want)
    # physically [K, N] weight (w8a8_gcu path, w8a8.py:152-155)
    acc2 = ops.int8_gemm_accumulators(dev(x), dev(np.ascontiguousarray(w_nk.T)))
    assert np.array_equal(acc2.cpu().numpy(), want)


@pytest.mark.parametrize("M,K,N", [(1, 128, 64), (33, 384, 320), (300, 1024, 448), (513, 2048, 1024)])
def test_int8_gemm_kslab_weights(ops, M, K, N):
    """Weights re-ordered by rearrange.to_kslab: the MFMA tile kernel reads them in place (raw
    accumulators bit-exact), and up to 64 rows the operator switches to the weight-streaming kernel,
    whose outputs must equal the tile kernel's on row-major weights bit for bit."""
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case i8 kslab {M}x{K}x{N}", flush=True)
    rng = np.random.default_rng(M * 7 + K + N)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    wk = rearrange.to_kslab(dev(w_nk))
    assert rearrange.is_kslab(wk.t())                      # the flag survives the view the operators receive
    want = o8.int8_gemm_i32(x, np.ascontiguousarray(w_nk.T))
    acc = ops.int8_gemm_accumulators(dev(x), wk.t())
    assert np.array_equal(acc.cpu().numpy(), want)
    xs = rng.uniform(0.001, 0.01, size=(M, 1)).astype(np.float32)
    ws = rng.uniform(0.001, 0.02, N).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.float16).cuda()
    for b in (None, bias):
        a = ops.cutlass_scaled_mm(dev(x), wk.t(), dev(xs), dev(ws), torch.float16, b)
        r = ops.cutlass_scaled_mm(dev(x), dev(w_nk).t(), dev(xs), dev(ws), torch.float16, b)
        assert torch.equal(a, r)
        wantf = o8.scaled_mm_epilogue(want, xs, ws, None if b is None else b.float().cpu().numpy())
        np.testing.assert_allclose(a.float().cpu().numpy(), wantf, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("N", [1536, 7168, 16384])
@pytest.mark.parametrize("M", [1, 16, 17, 32, 33, 64])
def test_int8_streaming_kernel_16_32_and_64_columns_per_workgroup(ops, M, N, monkeypatch):
    """The weight-streaming kernel gives a layer of few columns 16 (N = 1536) or 32 (N = 7168) columns
    per workgroup instead of 64 (N = 16384), so that about every CU streams a share of the weights.
    Kslab and row-major weights, every row-tile count: against the exact integer oracle through the
    epilogue, and bit for bit equal to the MFMA tile kernel on the same operands."""
    from vllm_gcu_amd.kernels import _custom_ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case i8 streaming narrow groups M={M} N={N}", flush=True)
    K = 1024
    rng = np.random.default_rng(M + N)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    xs = rng.uniform(0.001, 0.01, size=(M, 1)).astype(np.float32)
    ws = rng.uniform(0.001, 0.02, N).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.float16).cuda()
    want = o8.scaled_mm_epilogue(o8.int8_gemm_i32(x, np.ascontiguousarray(w_nk.T)), xs, ws, bias.float().cpu().numpy())
    wk = rearrange.to_kslab(dev(w_nk))
    monkeypatch.setattr(_custom_ops, "_INT8_STREAM_MAX_M", 1 << 20)           # the streaming kernel whatever the shape
    got = ops.cutlass_scaled_mm(dev(x), wk.t(), dev(xs), dev(ws), torch.float16, bias)
    row_major = ops.cutlass_scaled_mm(dev(x), dev(w_nk).t(), dev(xs), dev(ws), torch.float16, bias)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    monkeypatch.setattr(_custom_ops, "_INT8_STREAM_MAX_M", 0)                 # the tile kernel
    tile = ops.cutlass_scaled_mm(dev(x), wk.t(), dev(xs), dev(ws), torch.float16, bias)
    assert torch.equal(got, tile) and torch.equal(got, row_major)


@pytest.mark.parametrize("M,K,N,splits", [(128, 4096, 1024, 4), (200, 8192, 512, 8), (700, 2048, 1024, 2),
                                            (64, 14336, 4096, 8), (1000, 3072, 768, 3),
                                            # several row tiles on a layer of few columns: K ranges of 256 x 256 tiles
                                            (520, 8192, 5632, 2)])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_int8_gemm_split_k_is_bit_identical(ops, M, K, N, splits, out_dtype):
    """Few output tiles behind a long K: the operator cuts K into ranges that run side by side (int32
    partial sums in the stream's workspace, a second launch adds them and applies scales and bias).
    Integer sums: outputs and raw accumulators equal those of the entry point without workspace bit
    for bit, and the accumulators equal the oracle's."""
    from vllm_gcu_amd import _lib
    from vllm_gcu_amd.kernels import _runtime as rt
    print(f"case i8 split K {M}x{K}x{N} {out_dtype}", flush=True)
    lib = _lib.load()
    need = lib.mi355q_w8a8_int8_workspace_bytes(M, N, K)
    assert need == (1 << 20) + splits * M * N * 4              # the plan this test was written for
    rng = np.random.default_rng(M + K + N)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    xs = rng.uniform(0.001, 0.01, size=(M, 1)).astype(np.float32)
    ws = rng.uniform(0.001, 0.02, N).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(out_dtype).cuda()
    xd, wd, xsd, wsd = dev(x), dev(w_nk), dev(xs).reshape(-1), dev(ws)
    got = ops.cutlass_scaled_mm(xd, wd.t(), dev(xs), wsd, out_dtype, bias)
    acc = ops.int8_gemm_accumulators(xd, wd.t())
    assert np.array_equal(acc.cpu().numpy(), o8.int8_gemm_i32(x, np.ascontiguousarray(w_nk.T)))
    ref = torch.empty(M, N, dtype=out_dtype, device="cuda")
    ref_acc = torch.empty(M, N, dtype=torch.int32, device="cuda")
    with torch.cuda.device(0):
        _lib.call("mi355q_w8a8_int8_gemm", ref.data_ptr(), ref_acc.data_ptr(), xd.data_ptr(), wd.data_ptr(),
                  xsd.data_ptr(), 1, wsd.data_ptr(), 1, bias.data_ptr(), 0, M, N, K, K, K, N,
                  rt.dtype_code(out_dtype), rt.stream_ptr())
    torch.cuda.synchronize()
    assert torch.equal(acc, ref_acc)
    assert torch.equal(got, ref)
    assert torch.equal(got, ops.cutlass_scaled_mm(xd, wd.t(), dev(xs), wsd, out_dtype, bias))


@pytest.mark.parametrize("M,N", [(2305, 2048), (4200, 1792), (2049, 4096)])
def test_int8_gemm_more_than_eight_row_tiles(ops, M, N):
    # above 2048 rows the XCD-aware tile order walks the row tiles in chunks of eight (with a
    # shorter last chunk): every output tile must still be visited exactly once
    print(f"case i8 many row tiles {M}x{N}", flush=True)
    K = 128
    rng = np.random.default_rng(M + N)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    acc = ops.int8_gemm_accumulators(dev(x), dev(w_nk).t())
    assert np.array_equal(acc.cpu().numpy(), o8.int8_gemm_i32(x, np.ascontiguousarray(w_nk.T)))


@pytest.mark.parametrize("M", [16, 64, 200])
def test_int8_full_size_layer_three_kernels_agree_bit_for_bit(ops, M):
    """K = 8192, N = 28672 (the Llama-3-70B MLP layer of the config): the weight-streaming kernel
    (kslab weights, M <= 64), the MFMA tile kernel on kslab weights and the MFMA tile kernel on
    row-major weights are three independent paths over the same int32 sums and epilogue; their
    outputs must be identical, and sampled entries must match the oracle."""
    from vllm_gcu_amd.kernels import _custom_ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case i8 full size M={M}", flush=True)
    K, N = 8192, 28672
    g = torch.Generator(device="cuda").manual_seed(M)
    w = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    x = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda", generator=g)
    xs = torch.rand(M, 1, device="cuda", generator=g) * 0.01 + 0.001
    ws = torch.rand(N, device="cuda", generator=g) * 0.02 + 0.001
    wk = rearrange.to_kslab(w)
    a = ops.cutlass_scaled_mm(x, wk.t(), xs, ws, torch.float16, None)          # streaming kernel up to 64 rows
    r = ops.cutlass_scaled_mm(x, w.t(), xs, ws, torch.float16, None)           # tile kernel, row-major
    limit = _custom_ops._INT8_STREAM_MAX_M
    try:
        _custom_ops._INT8_STREAM_MAX_M = 0
        t = ops.cutlass_scaled_mm(x, wk.t(), xs, ws, torch.float16, None)      # tile kernel, kslab
    finally:
        _custom_ops._INT8_STREAM_MAX_M = limit
    assert torch.equal(a, r) and torch.equal(t, r)
    rows = np.array([0, M // 2, M - 1])
    cols = np.random.default_rng(M).integers(0, N, size=64)
    acc = x[rows].cpu().numpy().astype(np.int64) @ w[cols].cpu().numpy().astype(np.int64).T
    want = (acc.astype(np.float32) * xs[rows].cpu().numpy()) * ws[cols].cpu().numpy()[None, :]
    got = r[rows][:, cols].float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_cutlass_scaled_mm_epilogue(ops, dtype):
    rng = np.random.default_rng(3)
    M, K, N = 130, 512, 260
    xf = rng.standard_normal((M, K)).astype(np.float16)
    xq, xs = o8.dynamic_scaled_int8_quant(xf)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    ws = rng.uniform(0.001, 0.02, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    acc = o8.int8_gemm_i32(xq, np.ascontiguousarray(w_nk.T))
    for b, sa, sb in [(None, dev(xs), dev(ws)), (torch.from_numpy(bias).to(dtype).cuda(), dev(xs), dev(ws).reshape(N, 1)),
                      (None, dev(xs[:1, 0]).reshape(()), dev(ws[:1]))]:
        out = ops.cutlass_scaled_mm(dev(xq), dev(w_nk).t(), sa, sb, dtype, b)
        want = o8.scaled_mm_epilogue(acc, sa.cpu().numpy(), sb.cpu().numpy(),
                                     None if b is None else b.float().cpu().numpy())
        assert out.dtype == dtype and out.shape == (M, N)
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("N", [264, 488, 28672 // 8])
def test_scaled_mm_wide_and_narrow_output_stores_agree(ops, dtype, N):
    """16-bit outputs leave the tile kernel in 16-byte pieces when N, the output row stride and its address
    allow, in 8-byte pieces otherwise; both orders of the same values, so the results are the same bits."""
    rng = np.random.default_rng(11)
    M, K = 300, 256
    xq = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    xs = rng.uniform(0.5, 1.5, (M, 1)).astype(np.float32)
    ws = rng.uniform(0.001, 0.02, N).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(dtype).cuda()
    want = o8.scaled_mm_epilogue(o8.int8_gemm_i32(xq, np.ascontiguousarray(w_nk.T)), xs, ws, bias.float().cpu().numpy())
    wide = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    torch.ops._C.cutlass_scaled_mm(wide, dev(xq), dev(w_nk).t(), dev(xs), dev(ws), bias)
    np.testing.assert_allclose(wide.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # a row stride of N + 4 elements and a base 8 bytes into the buffer: neither allows 16-byte stores
    for buf, view in ((torch.full((M, N + 4), float("nan"), dtype=dtype, device="cuda"), lambda b: b[:, :N]),
                      (torch.full((M * N + 4,), float("nan"), dtype=dtype, device="cuda"), lambda b: b[4:].view(M, N))):
        narrow = view(buf)
        torch.ops._C.cutlass_scaled_mm(narrow, dev(xq), dev(w_nk).t(), dev(xs), dev(ws), bias)
        assert torch.equal(narrow, wide)
    if N > 300:
        assert bool(torch.isnan(buf[:4]).all())          # nothing written in front of the shifted base


def test_dot_bias_quant_single_scale(ops):
    rng = np.random.default_rng(4)
    M, K, N = 20, 256, 132
    xq = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_kn = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    sc = rng.uniform(1e-4, 1e-3, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float16)
    out = torch.empty(M, N, dtype=torch.float16, device="cuda")
    ops.dot_bias_quant(out, dev(xq), dev(w_kn), dev(sc), dev(bias))
    want = o8.scaled_mm_epilogue(o8.int8_gemm_i32(xq, w_kn), 1.0, sc, bias.astype(np.float32))
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    ops.cutlass_scaled_mm(torch.empty(0, K, dtype=torch.int8, device="cuda"), dev(w_kn), dev(sc[:1]), dev(sc), torch.float16)


def test_config2_full_size_sampled_rows(ops):
    # benchmark configuration 2: x f16 [2048, 8192] -> per-token int8; W int8 [8192, 28672];
    # int32 accumulate bit-exact.  The oracle checks 96 rows spread over every
    # 256-row tile, all 28672 columns.
    M, K, N = 2048, 8192, 28672
    print("case config2", flush=True)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(M, K, generator=g).to(torch.float16)
    w_nk = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g)
    ws = (torch.rand(N, generator=g) * 0.019 + 0.001).float()
    xq, xs, _ = ops.scaled_int8_quant(x.cuda())
    wd = w_nk.cuda()
    acc = ops.int8_gemm_accumulators(xq, wd.t())
    out = ops.cutlass_scaled_mm(xq, wd.t(), xs, ws.cuda(), torch.float16)
    rows = np.unique(np.concatenate([np.arange(0, M, 256), np.arange(255, M, 256),
                                     np.random.default_rng(0).integers(0, M, 80)]))
    xq_o, xs_o = o8.dynamic_scaled_int8_quant(x[rows].float().numpy())
    assert np.array_equal(xq[rows].cpu().numpy(), xq_o)
    want_acc = o8.int8_gemm_i32(xq_o, np.ascontiguousarray(w_nk.numpy().T))
    assert np.array_equal(acc[rows].cpu().numpy(), want_acc)
    want = o8.scaled_mm_epilogue(want_acc, xs_o, ws.numpy())
    np.testing.assert_allclose(out[rows].float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # size-independent property on the full result: linearity in the weights'
    # sign (negating W negates every accumulator exactly)
    acc_neg = ops.int8_gemm_accumulators(xq, (-wd).t())
    assert torch.equal(acc_neg, -acc)
