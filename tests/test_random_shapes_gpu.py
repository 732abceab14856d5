"""Seeded random shapes through the dense and grouped operators: every kernel family, row count and ragged
edge that the routing inside the operators can pick, checked against the oracle.  Outputs are
handed over full of NaN, so a tile that no workgroup writes shows up as NaN instead of as a stale
correct value."""
import numpy as np
import pytest
import torch

from oracle import fp8 as of8
from oracle import w4 as ow4
from oracle import w8a8 as o8

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2        # fp16 / bf16 outputs of fp32 accumulation


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def draw_rows(rng):
    # decode sizes, the 16/32/64/128/256-row boundaries of the kernels, and prefill sizes
    kind = rng.integers(0, 4)
    if kind == 0:
        return int(rng.integers(1, 18))
    if kind == 1:
        return int(rng.choice([31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257]))
    if kind == 2:
        return int(rng.integers(18, 300))
    return int(rng.integers(300, 1200))


@pytest.mark.parametrize("seed", range(24))
def test_w4a16_random_shapes(seed):
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    rng = np.random.default_rng(1000 + seed)
    M = draw_rows(rng)
    K = 128 * int(rng.integers(1, 25))
    N = 128 * int(rng.integers(1, 13))
    g = int(rng.choice([32, 64, 128, 128, 128, -1]))
    if g == -1 and K > 1024:
        g = 128
    dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
    with_bias = bool(rng.integers(0, 2))
    sym = bool(rng.integers(0, 4) == 0)
    print(f"case w4a16 random seed={seed} M={M} K={K} N={N} g={g} {dtype} bias={with_bias} sym={sym}", flush=True)
    G = 1 if g == -1 else K // g
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = np.full((G, N), 8, dtype=np.uint8) if sym else rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    s = torch.from_numpy(rng.uniform(0.001, 0.01, size=(G, N)).astype(np.float32)).to(dtype)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(dtype) if with_bias else None
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(ow4.gptq_pack_weight(q)), dev(ow4.gptq_pack_zeros(z)))
    out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    ops.w4a16_gemm(x.cuda(), w, s.cuda(), None if sym else zp, None if bias is None else bias.cuda(), g, out=out)
    torch.cuda.synchronize()
    want = ow4.w4a16_gemm(x.float().numpy(), q, z, s.float().numpy(), g,
                          bias=None if bias is None else bias.float().numpy())
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", range(24))
def test_w8a8_int8_random_shapes(seed):
    from vllm_gcu_amd.kernels.quantization import rearrange
    rng = np.random.default_rng(2000 + seed)
    M = draw_rows(rng)
    K = 128 * int(rng.integers(1, 17))
    kslab = bool(rng.integers(0, 2))
    N = 64 * int(rng.integers(1, 20)) if kslab else 4 * int(rng.integers(1, 300))
    dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
    with_bias = bool(rng.integers(0, 2))
    per_row = bool(rng.integers(0, 4) != 0)
    print(f"case w8a8 random seed={seed} M={M} K={K} N={N} kslab={kslab} {dtype} bias={with_bias} "
          f"per_row={per_row}", flush=True)
    x = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    w_nk = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    xs = rng.uniform(0.001, 0.01, size=(M, 1) if per_row else (1, 1)).astype(np.float32)
    ws = rng.uniform(0.001, 0.02, N).astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(dtype) if with_bias else None
    wd = dev(w_nk)
    if kslab:
        wd = rearrange.to_kslab(wd)
    out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    torch.ops._C.cutlass_scaled_mm(out, dev(x), wd.t(), dev(xs), dev(ws), None if bias is None else bias.cuda())
    torch.cuda.synchronize()
    acc = o8.int8_gemm_i32(x, np.ascontiguousarray(w_nk.T))
    want = o8.scaled_mm_epilogue(acc, xs, ws, None if bias is None else bias.float().numpy())
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", range(24))
def test_fp8_block_random_shapes(seed, monkeypatch):
    from vllm_gcu_amd.kernels import _custom_ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    if seed % 3:
        # shapes this small would all go to the weight-streaming kernel: send two thirds of them (above
        # 64 rows) to the MFMA tile kernel
        monkeypatch.setattr(_custom_ops, "_FP8_TILE_MIN_TILES", 1)
    rng = np.random.default_rng(3000 + seed)
    M = draw_rows(rng)
    K = 128 * int(rng.integers(1, 13))
    N = 128 * int(rng.integers(1, 10))
    kslab = bool(rng.integers(0, 2))
    with_bias = bool(rng.integers(0, 2))
    print(f"case fp8 block random seed={seed} M={M} K={K} N={N} kslab={kslab} bias={with_bias}", flush=True)
    w = of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    ws = rng.uniform(0.02, 0.1, size=(N // 128, K // 128)).astype(np.float32)
    xq, xs = of8.per_token_group_quant_fp8(rng.standard_normal((M, K)).astype(np.float32), 128)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(torch.bfloat16) if with_bias else None
    wd = dev(w).view(torch.float8_e4m3fn)
    if kslab:
        wd = rearrange.to_kslab(wd)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.ops._C.linear_quant(out, dev(xq).view(torch.float8_e4m3fn), wd, None if bias is None else bias.cuda(),
                              dev(xs), dev(ws))
    torch.cuda.synchronize()
    want = of8.block_fp8_gemm(xq, xs, w, ws)
    if bias is not None:
        want = want + bias.float().numpy()
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL,
                               atol=ATOL)


@pytest.mark.parametrize("seed", range(16))
def test_grouped_w4a16_random_shapes(seed):
    """Both GEMM forms of the fused-MoE W4A16 layer over random token counts, expert counts, top-k
    and block sizes, with a routing skewed so that some experts receive nothing."""
    from oracle import moe as om
    from vllm_gcu_amd.kernels import fused_moe as fmoe
    from vllm_gcu_amd.kernels.quantization import rearrange
    rng = np.random.default_rng(4000 + seed)
    M = int(rng.choice([1, 2, 7, 16, 33, 100, 257]))
    E = int(rng.choice([2, 4, 8, 16]))
    T = int(rng.integers(1, min(E, 4) + 1))
    K = 128 * int(rng.integers(1, 7))
    N = 128 * int(rng.integers(1, 6))
    block = int(rng.choice([16, 32, 64, 128]))
    dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
    print(f"case grouped w4a16 random seed={seed} M={M} E={E} T={T} K={K} N={N} block={block} {dtype}", flush=True)
    q = rng.integers(0, 16, size=(E, K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(E, K // 128, N), dtype=np.uint8)
    sd = torch.from_numpy(rng.uniform(0.001, 0.01, size=(E, K // 128, N)).astype(np.float32)).to(dtype)
    qw = np.stack([ow4.gptq_pack_weight(q[e]) for e in range(E)])
    qz = np.stack([ow4.gptq_pack_zeros(z[e]) for e in range(E)])
    w, zp = rearrange.rearrange_uint4_int32_gptq(dev(qw), dev(qz))
    logits = rng.standard_normal((M, E)).astype(np.float32)
    logits[:, : max(1, E // 2)] += 4.0                      # the upper half of the experts is rarely chosen
    tw, ids, _ = om.topk_softmax(logits, T, True)
    wf = lambda e: ow4.dequantize(q[e], z[e], sd[e].float().numpy(), 128)

    def run(A, C, mul, topk):
        s, e, n = fmoe.moe_align_block_size(dev(ids), block, E)
        fmoe.invoke_fused_moe_kernel(A, w, C, None, sd.cuda(), zp, dev(tw), dev(ids), s, e, n, mul, topk,
                                     {"BLOCK_SIZE_M": block}, use_fp8_w8a8=False, use_int8_w8a8=False,
                                     use_int8_w8a16=False, use_int4_w4a16=True, block_shape=[0, 128])
        torch.cuda.synchronize()

    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    C = torch.full((M, T, N), float("nan"), dtype=dtype, device="cuda")
    run(x.cuda(), C, False, T)
    want = om.fused_moe_gemm(x.float().numpy(), wf, ids, T)
    np.testing.assert_allclose(C.view(-1, N).float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    x2 = torch.from_numpy(rng.standard_normal((M * T, K)).astype(np.float32)).to(dtype)
    C2 = torch.full((M, T, N), float("nan"), dtype=dtype, device="cuda")
    run(x2.cuda(), C2, True, 1)
    want2 = om.fused_moe_gemm(x2.float().numpy(), wf, ids, 1, tw, True)
    np.testing.assert_allclose(C2.view(-1, N).float().cpu().numpy(), want2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", range(16))
def test_grouped_fp8_and_int8_random_shapes(seed):
    """The K-contiguous grouped GEMM (fp8 block-scaled and int8 per-token x per-channel experts),
    row-major and kslab weights, random routing with idle experts, all block sizes."""
    from oracle import moe as om
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels import fused_moe as fmoe
    from vllm_gcu_amd.kernels.quantization import rearrange
    rng = np.random.default_rng(5000 + seed)
    M = int(rng.choice([1, 3, 16, 40, 130, 300]))
    E = int(rng.choice([2, 4, 8, 32]))
    T = int(rng.integers(1, min(E, 4) + 1))
    K = 128 * int(rng.integers(1, 7))
    N = 128 * int(rng.integers(1, 5))
    block = int(rng.choice([16, 32, 64, 128]))
    kslab = bool(rng.integers(0, 2))
    mul = bool(rng.integers(0, 2))
    fp8 = bool(seed % 2)
    print(f"case grouped {'fp8' if fp8 else 'int8'} random seed={seed} M={M} E={E} T={T} K={K} N={N} "
          f"block={block} kslab={kslab} mul={mul}", flush=True)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    logits[:, : max(1, E // 2)] += 3.0
    tw, ids, _ = om.topk_softmax(logits, T, True)
    flat = ids.reshape(-1)
    s, e, n = fmoe.moe_align_block_size(dev(ids), block, E)
    want = np.zeros((M * T, N), dtype=np.float32)
    if fp8:
        wq = np.stack([of8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 2, -448, 448).astype(np.float32))
                       for _ in range(E)])
        ws = rng.uniform(0.005, 0.02, size=(E, N // 128, K // 128)).astype(np.float32)
        x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16)
        xq, xs = ops.per_token_group_quant_fp8(x.cuda(), 128)
        wd = dev(wq).view(torch.float8_e4m3fn)
        if kslab:
            wd = rearrange.to_kslab(wd)
        C = torch.full((M, T, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        fmoe.invoke_fused_moe_kernel(xq, wd, C, xs, dev(ws), None, dev(tw), dev(ids), s, e, n, mul, T,
                                     {"BLOCK_SIZE_M": block}, use_fp8_w8a8=True, use_int8_w8a8=False,
                                     use_int8_w8a16=False, use_int4_w4a16=False, block_shape=[128, 128])
        xq_c, xs_c = xq.view(torch.uint8).cpu().numpy(), xs.cpu().numpy()
        for t in range(M * T):
            want[t] = of8.block_fp8_gemm(xq_c[t // T:t // T + 1], xs_c[t // T:t // T + 1], wq[flat[t]], ws[flat[t]])[0]
    else:
        x = rng.standard_normal((M, K)).astype(np.float16)
        xq, xs = o8.dynamic_scaled_int8_quant(x)
        wq = rng.integers(-127, 128, size=(E, N, K), dtype=np.int8)
        ws = rng.uniform(0.001, 0.02, size=(E, N, 1)).astype(np.float32)
        wd = dev(wq)
        if kslab:
            wd = rearrange.to_kslab(wd)
        C = torch.full((M, T, N), float("nan"), dtype=torch.float16, device="cuda")
        fmoe.invoke_fused_moe_kernel(dev(xq), wd, C, dev(xs), dev(ws), None, dev(tw), dev(ids), s, e, n, mul, T,
                                     {"BLOCK_SIZE_M": block}, use_fp8_w8a8=False, use_int8_w8a8=True,
                                     use_int8_w8a16=False, use_int4_w4a16=False)
        for t in range(M * T):
            acc = o8.int8_gemm_i32(xq[t // T:t // T + 1], np.ascontiguousarray(wq[flat[t]].T))
            want[t] = o8.scaled_mm_epilogue(acc, xs[t // T], ws[flat[t], :, 0])[0]
    torch.cuda.synchronize()
    if mul:
        want = want * tw.reshape(-1, 1)
    got = C.view(-1, N).float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
