"""fp8-e4m3fn GEMM with per-token x per-channel (or per-tensor) scales -- ``cutlass_scaled_mm`` on fp8
operands (csrc/src/cutlass_scaled_mm.cpp:12-36; the non-block branch of
vllm_gcu/kernels/quantization/fp8.py:68-69) -- against the CPU oracle: dequantised codes, float32
matmul, ``(acc * x_scale) * w_scale (+ bias)``.  Outputs within rtol = atol = 1e-2."""
import numpy as np
import pytest
import torch

from oracle import fp8 as of8

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _operands(rng, M, K, N):
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    ws = rng.uniform(0.001, 0.02, size=N).astype(np.float32)
    xq, xs = of8.per_token_quant_fp8(rng.standard_normal((M, K)).astype(np.float32))
    return xq, xs.reshape(-1), w, ws


@pytest.mark.parametrize("M", [1, 16, 33, 64, 100, 128])
@pytest.mark.parametrize("kslab", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_streaming_kernel_per_token_per_channel(M, kslab, dtype):
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    K, N = 512, 384
    print(f"case fp8 scaled mm stream M={M} kslab={kslab} {dtype}", flush=True)
    rng = np.random.default_rng(1000 + M)
    xq, xs, w, ws = _operands(rng, M, K, N)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(dtype)
    wd = dev(w).view(torch.float8_e4m3fn)
    if kslab:
        wd = rearrange.to_kslab(wd)
    out = ops.cutlass_scaled_mm(dev(xq).view(torch.float8_e4m3fn), wd.t(), dev(xs).reshape(M, 1), dev(ws).reshape(N, 1),
                                dtype, bias.cuda())
    want = of8.scaled_fp8_mm(xq, xs, w, ws, bias.float().numpy())
    assert out.dtype == dtype and out.shape == (M, N)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("M,K,N", [(65, 384, 256), (129, 128, 128), (300, 512, 384), (513, 1024, 256), (2305, 128, 1024)])
@pytest.mark.parametrize("kslab", [False, True])
def test_tile_kernel_per_token_per_channel(M, K, N, kslab):
    """Activations with a padded row stride cannot take the weight-streaming kernel, so the call runs the MFMA
    tile kernel whatever the shape; checked against the oracle and, for dense activations of few rows, bit for
    bit against nothing else -- the two kernels add in different orders -- but within fp32 accuracy of each other."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case fp8 scaled mm tile M={M} K={K} N={N} kslab={kslab}", flush=True)
    rng = np.random.default_rng(M + K + N)
    xq, xs, w, ws = _operands(rng, M, K, N)
    wd = dev(w).view(torch.float8_e4m3fn)
    if kslab:
        wd = rearrange.to_kslab(wd)
    xpad = torch.zeros((M, K + 64), dtype=torch.uint8, device="cuda")
    xpad[:, :K] = dev(xq)
    xv = xpad.view(torch.float8_e4m3fn)[:, :K]                   # row stride K + 64
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.cutlass_scaled_mm(out, xv, wd.t(), dev(xs), dev(ws), None)
    want = of8.scaled_fp8_mm(xq, xs, w, ws)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # dense activations of the same values: the streaming kernel (fewer than 64 output tiles); same sums
    # up to the order of the fp32 additions
    dense = ops.cutlass_scaled_mm(dev(xq).view(torch.float8_e4m3fn), wd.t(), dev(xs), dev(ws), torch.bfloat16, None)
    d = (dense.float() - out.float()).abs().max().item()
    assert d <= 2 ** -7 * max(1.0, float(np.abs(want).max()))


@pytest.mark.parametrize("x_per_row,w_per_col", [(False, False), (True, False), (False, True)])
def test_per_tensor_scales_and_scale_shapes(x_per_row, w_per_col):
    from vllm_gcu_amd.kernels import _custom_ops as ops
    print(f"case fp8 scaled mm scalar scales x_per_row={x_per_row} w_per_col={w_per_col}", flush=True)
    rng = np.random.default_rng(5)
    for M, K, N, pad in ((24, 256, 192, 0), (200, 256, 256, 16)):
        xq, xs, w, ws = _operands(rng, M, K, N)
        xs_arg = xs if x_per_row else np.float32(0.03)
        ws_arg = ws if w_per_col else np.float32(0.007)
        xpad = torch.zeros((M, K + pad), dtype=torch.uint8, device="cuda")
        xpad[:, :K] = dev(xq)
        xv = xpad.view(torch.float8_e4m3fn)[:, :K]
        xs_t = dev(xs).reshape(M, 1) if x_per_row else torch.tensor(0.03, device="cuda")       # 0-d, as upstream passes it
        ws_t = dev(ws).reshape(N, 1) if w_per_col else torch.tensor([0.007], device="cuda")
        out = ops.cutlass_scaled_mm(xv, dev(w).view(torch.float8_e4m3fn).t(), xs_t, ws_t, torch.float16, None)
        want = of8.scaled_fp8_mm(xq, xs_arg, w, ws_arg)
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_equals_block_scaled_gemm_when_block_scales_are_constant():
    """Block scales that do not vary along K and channel scales that do not vary inside a 128-column block
    describe the same product: ``linear_quant`` and ``cutlass_scaled_mm`` must agree (powers of two: exactly up to
    the order of the fp32 additions)."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    print("case fp8 scaled mm == block scaled", flush=True)
    rng = np.random.default_rng(8)
    for M in (16, 300):
        K, N = 1024, 512
        xq, _, w, _ = _operands(rng, M, K, N)
        xs = (2.0 ** rng.integers(-6, -1, size=M)).astype(np.float32)
        wsb = (2.0 ** rng.integers(-8, -4, size=N // 128)).astype(np.float32)
        blk = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        torch.ops._C.linear_quant(blk, dev(xq).view(torch.float8_e4m3fn), dev(w).view(torch.float8_e4m3fn), None,
                                  dev(np.repeat(xs[:, None], K // 128, 1)), dev(np.repeat(wsb[:, None], K // 128, 1)))
        pc = ops.cutlass_scaled_mm(dev(xq).view(torch.float8_e4m3fn), dev(w).view(torch.float8_e4m3fn).t(), dev(xs),
                                   dev(np.repeat(wsb, 128)), torch.bfloat16, None)
        want = of8.scaled_fp8_mm(xq, xs, w, np.repeat(wsb, 128))
        np.testing.assert_allclose(pc.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
        assert (pc.float() - blk.float()).abs().max().item() <= 2 ** -7 * max(1.0, float(np.abs(want).max()))


@pytest.mark.parametrize("M,K,N", [(128, 4096, 1024), (300, 8192, 512), (700, 2048, 1024), (65, 7168, 1536),
                                   (33, 7168, 1536), (33, 7168, 4096), (25, 14336, 1024)])
@pytest.mark.parametrize("kslab", [False, True])
def test_few_tiles_behind_a_long_k_are_split_into_k_ranges(M, K, N, kslab):
    """Both fp8 tile kernels on layers with few 256 x 128 tiles: K ranges run side by side, their fp32 sums
    go through the stream's workspace and a second launch adds them in range order and applies bias and
    scales.  Against the oracle, run-to-run identical, and within fp32 accuracy of the entry points
    without workspace (same products, another order of additions)."""
    from vllm_gcu_amd import _lib
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels import _runtime as rt
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case fp8 split K M={M} K={K} N={N} kslab={kslab}", flush=True)
    lib = _lib.load()
    assert lib.mi355q_fp8_gemm_workspace_bytes(M, N, K) > (1 << 20)        # a split plan exists for this shape
    if M < 64:                                                              # ... and none one row below its first height
        assert lib.mi355q_fp8_gemm_workspace_bytes(M - 1, N, K) == 0
    rng = np.random.default_rng(M + K + N)
    xq, xs, w, ws = _operands(rng, M, K, N)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.bfloat16).cuda()
    xd = dev(xq).view(torch.float8_e4m3fn)
    wd = dev(w).view(torch.float8_e4m3fn)
    wk = rearrange.to_kslab(wd) if kslab else wd
    # per-token x per-channel scales
    got = ops.cutlass_scaled_mm(xd, wk.t(), dev(xs).reshape(M, 1), dev(ws).reshape(N, 1), torch.bfloat16, bias)
    assert torch.equal(got, ops.cutlass_scaled_mm(xd, wk.t(), dev(xs).reshape(M, 1), dev(ws).reshape(N, 1), torch.bfloat16, bias))
    want = of8.scaled_fp8_mm(xq, xs, w, ws, bias.float().cpu().numpy())
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    ref = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    xsd, wsd = dev(xs), dev(ws)
    with torch.cuda.device(0):
        _lib.call("mi355q_fp8_scaled_gemm", ref.data_ptr(), xd.data_ptr(), wk.data_ptr(), xsd.data_ptr(), 1,
                  wsd.data_ptr(), 1, bias.data_ptr(), M, N, K, K, 0 if kslab else K, N, rt.dtype_code(torch.bfloat16),
                  rt.stream_ptr())
    torch.cuda.synchronize()
    assert (got.float() - ref.float()).abs().max().item() <= 2 ** -7 * max(1.0, float(np.abs(want).max()))
    # 128 x 128 block scales
    xsb = rng.uniform(0.01, 0.05, size=(M, K // 128)).astype(np.float32)
    wsb = rng.uniform(0.01, 0.05, size=(N // 128, K // 128)).astype(np.float32)
    blk = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(blk, xd, wk, bias, dev(xsb), dev(wsb))
    blk2 = torch.empty_like(blk)
    torch.ops._C.linear_quant(blk2, xd, wk, bias, dev(xsb), dev(wsb))
    assert torch.equal(blk, blk2)
    wantb = of8.block_fp8_gemm(xq, xsb, w, wsb, bias=bias.float().cpu().numpy())
    np.testing.assert_allclose(blk.float().cpu().numpy(), wantb, rtol=RTOL, atol=RTOL * max(1.0, float(np.abs(wantb).max())))


@pytest.mark.parametrize("M,K,N", [(300, 256, 16384), (200, 2048, 16384), (1300, 384, 9728), (70, 512, 16512)])
@pytest.mark.parametrize("kslab", [False, True])
def test_block_scales_of_the_activations_staged_k_block_major(M, K, N, kslab, monkeypatch):
    """On a layer of many column tiles the block-scaled tile kernel first re-orders the activation scales K block
    major in the workspace (a workgroup's 256 scales of a K block side by side): the same numbers from another
    address, so the output equals the unstaged launch bit for bit -- unsplit, with K ranges side by side (the
    second shape), with a ragged last row tile -- and meets the oracle."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case fp8 block scales staged M={M} K={K} N={N} kslab={kslab}", flush=True)
    rng = np.random.default_rng(M + K + N + 7)
    xq, _, w, _ = _operands(rng, M, K, N)
    xsb = rng.uniform(0.01, 0.05, size=(M, K // 128)).astype(np.float32)
    wsb = rng.uniform(0.01, 0.05, size=(N // 128, K // 128)).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.bfloat16).cuda()
    xd = dev(xq).view(torch.float8_e4m3fn)
    wd = dev(w).view(torch.float8_e4m3fn)
    wk = rearrange.to_kslab(wd) if kslab else wd
    staged = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(staged, xd, wk, bias, dev(xsb), dev(wsb))
    monkeypatch.setattr(ops, "_FP8_STAGE_SCALES", False)
    plain = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(plain, xd, wk, bias, dev(xsb), dev(wsb))
    torch.cuda.synchronize()
    assert torch.equal(staged, plain)
    want = of8.block_fp8_gemm(xq, xsb, w, wsb, bias=bias.float().cpu().numpy())
    np.testing.assert_allclose(staged.float().cpu().numpy(), want, rtol=RTOL, atol=RTOL * max(1.0, float(np.abs(want).max())))


@pytest.mark.parametrize("M", [1, 16, 128, 2048])
def test_full_size_layer_sampled(M):
    """K = 8192, N = 28672 (one Llama-3-70B MLP projection): sampled rows and columns against the oracle, the whole
    output finite, and run-to-run identical."""
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    print(f"case fp8 scaled mm full size M={M}", flush=True)
    K, N = 8192, 28672
    g = torch.Generator(device="cuda").manual_seed(M)
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.5).to(torch.float8_e4m3fn)
    ws = torch.rand(N, device="cuda", generator=g) * 0.019 + 0.001
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
    xq, xs = ops.scaled_fp8_quant(x, None, use_per_token_if_dynamic=True)
    wk = rearrange.to_kslab(w)
    out = ops.cutlass_scaled_mm(xq, wk.t(), xs, ws.reshape(N, 1), torch.float16, None)
    again = ops.cutlass_scaled_mm(xq, wk.t(), xs, ws.reshape(N, 1), torch.float16, None)
    assert torch.isfinite(out).all() and torch.equal(out, again)
    rows = np.unique(np.array([0, M // 3, M // 2, M - 1]))
    cols = np.random.default_rng(M).integers(0, N, size=256)
    want = of8.scaled_fp8_mm(xq.view(torch.uint8)[rows].cpu().numpy(), xs.reshape(-1)[rows].cpu().numpy(),
                             w.view(torch.uint8)[cols].cpu().numpy(), ws[cols].cpu().numpy())
    got = out[rows][:, cols].float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    # row-major weights give the same bits as the kslab order (same kernel, same order of additions)
    if M in (16, 2048):
        rm = ops.cutlass_scaled_mm(xq, w.t(), xs, ws.reshape(N, 1), torch.float16, None)
        assert torch.equal(rm, out)


@pytest.mark.parametrize("scheme", ["dynamic", "static"])
def test_fp8_linear_method_without_block_scales(scheme):
    """A checkpoint without ``weight_block_size``: merged projection of three shards, one weight scale each
    (upstream Fp8LinearMethod.create_weights, which the reference inherits, fp8.py:49-70); the method keeps every
    shard's own scale as per-channel scales and calls the fp8 ``cutlass_scaled_mm``."""
    from vllm_gcu_amd.kernels.quantization.fp8 import Fp8GCUConfig
    print(f"case fp8 method per tensor {scheme}", flush=True)
    rng = np.random.default_rng(17)
    M, K, widths = 40, 512, [256, 64, 64]
    N = sum(widths)
    cfg = Fp8GCUConfig.from_config({"quant_method": "fp8", "activation_scheme": scheme})
    assert cfg.weight_block_size is None
    method = cfg.get_quant_method()
    layer = torch.nn.Module()
    method.create_weights(layer, K, widths, K, N, torch.bfloat16)
    assert layer.weight.shape == (N, K) and layer.weight_scale.shape == (3,)
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    shard_scales = np.array([0.004, 0.011, 0.002], np.float32)
    layer.weight = torch.nn.Parameter(dev(w).view(torch.float8_e4m3fn), requires_grad=False)
    layer.weight_scale = torch.nn.Parameter(dev(shard_scales), requires_grad=False)
    if scheme == "static":
        assert layer.input_scale.shape == (3,)
        layer.input_scale = torch.nn.Parameter(dev(np.array([0.01, 0.02, 0.015], np.float32)), requires_grad=False)
    method.process_weights_after_loading(layer)
    assert layer.weight_scale.shape == (N,) and getattr(layer.weight, "_mi355q_kslab", False)
    x = torch.from_numpy(rng.standard_normal((2, M // 2, K)).astype(np.float32)).to(torch.bfloat16)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.bfloat16)
    out = method.apply(layer, x.cuda(), bias.cuda())
    assert out.shape == (2, M // 2, N) and out.dtype == torch.bfloat16
    xf = x.float().numpy().reshape(M, K)
    if scheme == "static":
        s = np.float32(0.02)                                      # the largest of the shards' input scales
        xq = of8.to_e4m3fn(np.clip(xf / s, -448, 448).astype(np.float32))
        xs = s
    else:
        xq, xs = of8.per_token_quant_fp8(xf)
        xs = xs.reshape(-1)
    want = of8.scaled_fp8_mm(xq, xs, w, np.repeat(shard_scales, widths), bias.float().numpy())
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(M, N), want, rtol=RTOL, atol=ATOL)


def test_argument_errors():
    from vllm_gcu_amd.kernels import _custom_ops as ops
    x = torch.zeros((4, 256), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    w = torch.zeros((128, 256), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    one = torch.ones(1, device="cuda")
    with pytest.raises(RuntimeError, match="x_scale has 3 entries"):
        ops.cutlass_scaled_mm(x, w.t(), torch.ones(3, device="cuda"), one, torch.float16, None)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        ops.cutlass_scaled_mm(x, w.t(), one, one, torch.float32, None)
    with pytest.raises(RuntimeError, match="float8_e4m3fn weight"):
        ops.cutlass_scaled_mm(x, w.view(torch.int8).t(), one, one, torch.float16, None)
    assert ops.cutlass_scaled_mm(x[:0], w.t(), one, one, torch.float16, None).shape == (0, 128)
