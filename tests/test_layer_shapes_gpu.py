"""Layer-sized shapes (Llama-, Qwen-, DeepSeek- and Mixtral-like K x N, expert counts and token counts on and
around every row boundary of the dispatch rules) through the dense and grouped operators with no kernel forced:
what the small random shapes cannot reach -- K splits, ring and wide-tile plans, staged bf16 rows, staged fp8
scales, blocks of 128 / 256 slots.  The weights are drawn and dequantised on the device; sampled rows / slots are
compared with a plain fp32 (int8: fp64) torch matmul of the unpacked arrays, outputs pre-filled with NaN."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = [(4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096), (8192, 10240), (8192, 8192), (8192, 57344),
          (28672, 8192), (3584, 4608), (3584, 37888), (18944, 3584), (5120, 13824), (2048, 11008), (7168, 1536),
          (7168, 4096), (16384, 7168), (2048, 7168), (1536, 24576), (11008, 4096), (4096, 22016), (1024, 1024), (6144, 2048)]
ROWS = list(range(1, 18)) + [24, 31, 32, 33, 40, 48, 49, 63, 64, 65, 96, 127, 128, 129, 192, 255, 256, 257, 384, 511, 512, 513, 520,
                             700, 768, 1000, 1024, 1025, 1536, 2047, 2048, 2049, 3000, 4096, 5000]
GSHAPES = [(8, 4096, 2048), (8, 4096, 7168), (8, 2048, 4096), (16, 2048, 2816), (60, 2048, 1408 * 2), (64, 2048, 1024),
           (8, 14336, 4096), (32, 7168, 4096), (32, 2048, 7168), (4, 1024, 512), (128, 1024, 768 * 2)]   # (E, K, N)
TOKENS = [1, 2, 5, 8, 16, 17, 33, 64, 100, 128, 200, 256, 400, 512, 700, 1024, 1500, 2048, 3000]
WHICH = ("w4", "int8", "fp8", "fp8pc")


def check(name, got, want, rtol=1e-2, atol=1e-2):
    got = got.float()
    bad = ~(torch.isfinite(got)) | ((got - want).abs() > atol + rtol * want.abs())
    n = int(bad.sum())
    if n:
        i = torch.nonzero(bad)[0].tolist()
        raise AssertionError(f"{name}: {n} of {got.numel()} outside tolerance, first at {i}: got {float(got[tuple(i)])} "
                             f"want {float(want[tuple(i)])}")


def pick_rows(rng, M, dev):
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, size=min(M, 40))]))
    return torch.from_numpy(rows).to(dev)


def pack8(v):
    """uint8 nibbles [..., 8] -> int32, nibble i at bits 4 i"""
    acc = torch.zeros(v.shape[:-1], dtype=torch.int64, device=v.device)
    for i in range(8):
        acc |= v[..., i].to(torch.int64) << (4 * i)
    return torch.where(acc >= 2**31, acc - 2**32, acc).to(torch.int32)


def dense_case(seed):
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels.quantization import rearrange
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(50000 + seed)
    K, N = SHAPES[int(rng.integers(0, len(SHAPES)))]
    M = int(ROWS[int(rng.integers(0, len(ROWS)))])
    gen = torch.Generator(device=dev).manual_seed(seed)
    if "w4" in WHICH:
        g = int(rng.choice([128, 128, 128, 64, 32])) if K <= 8192 else 128
        dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
        zkind = int(rng.integers(0, 3))        # 0 packed, 1 none, 2 pre-scaled
        with_bias = bool(rng.integers(0, 2))
        print(f"case w4 seed={seed} M={M} K={K} N={N} g={g} {dtype} zkind={zkind} bias={with_bias}", flush=True)
        G = K // g
        q = torch.randint(0, 16, (K, N), dtype=torch.uint8, device=dev, generator=gen)
        z = torch.randint(0, 16, (G, N), dtype=torch.uint8, device=dev, generator=gen)
        s = (torch.rand(G, N, device=dev, generator=gen) * 0.009 + 0.001).to(dtype)
        x = torch.randn(M, K, device=dev, generator=gen).to(dtype)
        bias = torch.randn(N, device=dev, generator=gen).to(dtype) if with_bias else None
        # pack on the device: GPTQ int32 [K/8, N], nibble i of row k8 = q[8 k8 + i]
        q32 = q.view(K // 8, 8, N).to(torch.int64)
        packed = torch.zeros(K // 8, N, dtype=torch.int64, device=dev)
        for i in range(8):
            packed |= q32[:, i, :] << (4 * i)
        packed = (packed & 0xffffffff)
        packed = torch.where(packed >= 2**31, packed - 2**32, packed).to(torch.int32)
        z32 = z.view(G, N // 8, 8).to(torch.int64)
        zp = torch.zeros(G, N // 8, dtype=torch.int64, device=dev)
        for i in range(8):
            zp |= z32[:, :, i] << (4 * i)
        zp = torch.where(zp >= 2**31, zp - 2**32, zp).to(torch.int32)
        # gptq stores z - 1
        zm1 = ((z.to(torch.int64) - 1) & 15).view(G, N // 8, 8)
        zpg = torch.zeros(G, N // 8, dtype=torch.int64, device=dev)
        for i in range(8):
            zpg |= zm1[:, :, i] << (4 * i)
        zpg = torch.where(zpg >= 2**31, zpg - 2**32, zpg).to(torch.int32)
        w, zdev = rearrange.rearrange_uint4_int32_gptq(packed, zpg)
        sf = s.float()
        if zkind == 0:
            zeros, zf = zdev, z.float()
            W = (q.float().view(G, g, N) - zf[:, None, :]) * sf[:, None, :]
        elif zkind == 1:
            zeros = None
            W = (q.float().view(G, g, N) - 8.0) * sf[:, None, :]
        else:
            # the reference loader's form: integer z times scale, rounded to the activation type (the operator layer
            # turns it back into the packed integers: w = (q - z) s, the reading of every kernel)
            zeros = (z.float() * sf).to(dtype)
            W = (q.float().view(G, g, N) - z.float()[:, None, :]) * sf[:, None, :]
        W = W.view(K, N)
        out = torch.full((M, N), float("nan"), dtype=dtype, device=dev)
        ops.w4a16_gemm(x, w, s, zeros, bias, g, out=out)
        torch.cuda.synchronize()
        rows = pick_rows(rng, M, dev)
        want = x[rows].float() @ W
        if bias is not None:
            want = want + bias.float()
        check(f"w4 seed={seed}", out[rows], want)
        del q, z, s, x, W, w, out, packed, q32
    if "int8" in WHICH and K % 128 == 0:
        dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
        kslab = bool(rng.integers(0, 2)) and N % 64 == 0
        per_row = bool(rng.integers(0, 4) != 0)
        with_bias = bool(rng.integers(0, 2))
        print(f"case int8 seed={seed} M={M} K={K} N={N} kslab={kslab} {dtype} per_row={per_row} bias={with_bias}", flush=True)
        x = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=dev, generator=gen)
        wnk = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=gen)
        xs = (torch.rand((M, 1) if per_row else (1, 1), device=dev, generator=gen) * 0.009 + 0.001)
        ws = (torch.rand(N, device=dev, generator=gen) * 0.019 + 0.001)
        bias = torch.randn(N, device=dev, generator=gen).to(dtype) if with_bias else None
        wd = rearrange.to_kslab(wnk) if kslab else wnk
        out = torch.full((M, N), float("nan"), dtype=dtype, device=dev)
        torch.ops._C.cutlass_scaled_mm(out, x, wd.t(), xs, ws, bias)
        torch.cuda.synchronize()
        rows = pick_rows(rng, M, dev)
        acc = (x[rows].double() @ wnk.double().t())
        want = (acc * (xs[rows] if per_row else xs).double() * ws.double()).float()
        if bias is not None:
            want = want + bias.float()
        check(f"int8 seed={seed}", out[rows], want)
        del x, wnk, wd, out, acc
    if ("fp8" in WHICH or "fp8pc" in WHICH) and K % 128 == 0 and N % 128 == 0:
        kslab = bool(rng.integers(0, 2))
        with_bias = bool(rng.integers(0, 2))
        wb = torch.randint(0, 256, (N, K), dtype=torch.uint8, device=dev, generator=gen)
        wb = torch.where((wb & 0x7f) == 0x7f, wb & 0xf0, wb)          # no NaN codes
        xb = torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=gen)
        xb = torch.where((xb & 0x7f) == 0x7f, xb & 0xf0, xb)
        # keep magnitudes moderate: clear the top exponent bit
        wb, xb = wb & 0xbf, xb & 0xbf
        wq, xq = wb.view(torch.float8_e4m3fn), xb.view(torch.float8_e4m3fn)
        wd = rearrange.to_kslab(wq) if kslab else wq
        bias = torch.randn(N, device=dev, generator=gen).to(torch.bfloat16) if with_bias else None
        rows = pick_rows(rng, M, dev)
        if "fp8" in WHICH:
            print(f"case fp8 block seed={seed} M={M} K={K} N={N} kslab={kslab} bias={with_bias}", flush=True)
            ws = torch.rand(N // 128, K // 128, device=dev, generator=gen) * 0.08 + 0.02
            xs = torch.rand(M, K // 128, device=dev, generator=gen) * 0.08 + 0.02
            out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
            torch.ops._C.linear_quant(out, xq, wd, bias, xs, ws)
            torch.cuda.synchronize()
            xf = xq[rows].float() * xs[rows].repeat_interleave(128, dim=1)
            wf = wq.float() * ws.repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
            want = xf @ wf.t()
            if bias is not None:
                want = want + bias.float()
            check(f"fp8 block seed={seed}", out[rows], want, rtol=1.5e-2, atol=1.5e-2 * float(want.abs().mean()) + 1e-2)
            del wf, xf, out
        if "fp8pc" in WHICH:
            print(f"case fp8 pc seed={seed} M={M} K={K} N={N} kslab={kslab} bias={with_bias}", flush=True)
            xs1 = torch.rand(M, 1, device=dev, generator=gen) * 0.008 + 0.002
            ws1 = torch.rand(N, 1, device=dev, generator=gen) * 0.008 + 0.002
            out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
            torch.ops._C.cutlass_scaled_mm(out, xq, wd.t(), xs1, ws1, bias)
            torch.cuda.synchronize()
            want = (xq[rows].float() @ wq.float().t()) * xs1[rows] * ws1.t()
            if bias is not None:
                want = want + bias.float()
            check(f"fp8 pc seed={seed}", out[rows], want, rtol=1.5e-2, atol=1.5e-2 * float(want.abs().mean()) + 1e-2)
            del out
        del wb, xb, wq, xq, wd
    torch.cuda.empty_cache()


def grouped_case(seed):
    from vllm_gcu_amd.kernels import _custom_ops as ops
    from vllm_gcu_amd.kernels import fused_moe as fmoe
    from vllm_gcu_amd.kernels.quantization import rearrange
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(70000 + seed)
    E, K, N = GSHAPES[int(rng.integers(0, len(GSHAPES)))]
    M = int(TOKENS[int(rng.integers(0, len(TOKENS)))])
    T = int(rng.choice([1, 2, 2, 4, 6]))
    T = min(T, E)
    mode = str(rng.choice(["w4", "w4", "fp8", "int8", "h16", "w8a16"]))
    dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
    second_form = bool(rng.integers(0, 2))          # one activation row per slot, routing weights applied
    gen = torch.Generator(device=dev).manual_seed(seed)
    logits = torch.randn(M, E, device=dev, generator=gen)
    if rng.integers(0, 3) == 0:
        logits[:, : max(1, E // 4)] += 3.0          # skewed routing
    tw, ids = ops.fused_topk(torch.empty(M, 8, device=dev, dtype=dtype), logits, T, True)
    cfgdt = {"int8": "int8_w8a8", "h16": "w16a16"}.get(mode)
    cfg = fmoe.get_default_config(M=M, E=E, N=N, K=K, topk=T, dtype=cfgdt, is_marlin=False,
                                  block_shape=[128, 128] if mode == "fp8" else None)
    if rng.integers(0, 3) == 0:
        cfg = dict(cfg, BLOCK_SIZE_M=int(rng.choice([16, 32, 64, 128] + ([256] if mode in ("fp8", "int8", "h16") else []))))
    blk = cfg["BLOCK_SIZE_M"]
    print(f"case grouped seed={seed} mode={mode} E={E} K={K} N={N} M={M} T={T} blk={blk} {dtype} second={second_form}", flush=True)
    rows_a = M * T if second_form else M
    topk_arg = 1 if second_form else T
    flat = ids.reshape(-1).long()
    slots = torch.unique(torch.cat([torch.tensor([0, M * T - 1], device=dev),
                                    torch.randint(0, M * T, (min(M * T, 48),), device=dev, generator=gen)]))
    arow = slots if second_form else slots // T
    s_, e_, n_ = fmoe.moe_align_block_size(ids, blk, E)
    C = torch.full((M, T, N), float("nan"), dtype=dtype if mode != "fp8" else torch.bfloat16, device=dev)
    kw = dict(use_fp8_w8a8=False, use_int8_w8a8=False, use_int8_w8a16=False, use_int4_w4a16=False)
    if mode == "w4":
        g = int(rng.choice([128, 128, 64, 32]))
        G = K // g
        q = torch.randint(0, 16, (E, K, N), dtype=torch.uint8, device=dev, generator=gen)
        z = torch.randint(0, 16, (E, G, N), dtype=torch.uint8, device=dev, generator=gen)
        s = (torch.rand(E, G, N, device=dev, generator=gen) * 0.009 + 0.001).to(dtype)
        x = torch.randn(rows_a, K, device=dev, generator=gen).to(dtype)
        qw = pack8(q.view(E, K // 8, 8, N).permute(0, 1, 3, 2))
        qz = pack8(((z.to(torch.int64) - 1) & 15).view(E, G, N // 8, 8))
        w, zp = rearrange.rearrange_uint4_int32_gptq(qw, qz)
        fmoe.invoke_fused_moe_kernel(x, w, C, None, s, zp, tw, ids, s_, e_, n_, second_form, topk_arg, cfg,
                                     **dict(kw, use_int4_w4a16=True), block_shape=[0, g])
        torch.cuda.synchronize()
        want = torch.empty(slots.numel(), N, device=dev)
        for i, t in enumerate(slots.tolist()):
            e = int(flat[t])
            W = ((q[e].float().view(G, g, N) - z[e].float()[:, None, :]) * s[e].float()[:, None, :]).view(K, N)
            want[i] = x[arow[i]].float() @ W
        del q, z, s, w, qw
    elif mode == "fp8":
        wb = torch.randint(0, 256, (E, N, K), dtype=torch.uint8, device=dev, generator=gen)
        wb = torch.where((wb & 0x7f) == 0x7f, wb & 0xf0, wb) & 0xbf
        xb = torch.randint(0, 256, (rows_a, K), dtype=torch.uint8, device=dev, generator=gen)
        xb = torch.where((xb & 0x7f) == 0x7f, xb & 0xf0, xb) & 0xbf
        wq, x = wb.view(torch.float8_e4m3fn), xb.view(torch.float8_e4m3fn)
        ws = torch.rand(E, N // 128, K // 128, device=dev, generator=gen) * 0.08 + 0.02
        xs = torch.rand(rows_a, K // 128, device=dev, generator=gen) * 0.08 + 0.02
        fmoe.invoke_fused_moe_kernel(x, wq, C, xs, ws, None, tw, ids, s_, e_, n_, second_form, topk_arg, cfg,
                                     **dict(kw, use_fp8_w8a8=True), block_shape=[128, 128])
        torch.cuda.synchronize()
        want = torch.empty(slots.numel(), N, device=dev)
        for i, t in enumerate(slots.tolist()):
            e = int(flat[t])
            wf = wq[e].float() * ws[e].repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
            xf = x[arow[i]].float() * xs[arow[i]].repeat_interleave(128)
            want[i] = wf @ xf
        del wb, wq
    elif mode == "int8":
        wq = torch.randint(-127, 128, (E, N, K), dtype=torch.int8, device=dev, generator=gen)
        x = torch.randint(-128, 128, (rows_a, K), dtype=torch.int8, device=dev, generator=gen)
        ws = torch.rand(E, N, 1, device=dev, generator=gen) * 0.019 + 0.001
        xs = torch.rand(rows_a, 1, device=dev, generator=gen) * 0.009 + 0.001
        fmoe.invoke_fused_moe_kernel(x, wq, C, xs, ws, None, tw, ids, s_, e_, n_, second_form, topk_arg, cfg,
                                     **dict(kw, use_int8_w8a8=True))
        torch.cuda.synchronize()
        want = torch.empty(slots.numel(), N, device=dev)
        for i, t in enumerate(slots.tolist()):
            e = int(flat[t])
            want[i] = ((wq[e].double() @ x[arow[i]].double()) * xs[arow[i]].double() * ws[e, :, 0].double()).float()
        del wq
    elif mode == "h16":
        wq = torch.empty(E, N, K, device=dev, dtype=dtype).normal_(0, 0.03, generator=gen)
        x = torch.randn(rows_a, K, device=dev, generator=gen).to(dtype)
        fmoe.invoke_fused_moe_kernel(x, wq, C, None, None, None, tw, ids, s_, e_, n_, second_form, topk_arg, cfg, **kw)
        torch.cuda.synchronize()
        want = torch.empty(slots.numel(), N, device=dev)
        for i, t in enumerate(slots.tolist()):
            want[i] = wq[int(flat[t])].float() @ x[arow[i]].float()
        del wq
    else:
        wq = torch.randint(-127, 128, (E, N, K), dtype=torch.int8, device=dev, generator=gen)
        x = torch.randn(rows_a, K, device=dev, generator=gen).to(dtype)
        ws = (torch.rand(E, N, device=dev, generator=gen) * 0.002 + 0.0002).to(dtype)
        fmoe.invoke_fused_moe_kernel(x, wq, C, None, ws, None, tw, ids, s_, e_, n_, second_form, topk_arg, cfg,
                                     **dict(kw, use_int8_w8a16=True), block_shape=[0, -1])
        torch.cuda.synchronize()
        want = torch.empty(slots.numel(), N, device=dev)
        for i, t in enumerate(slots.tolist()):
            e = int(flat[t])
            want[i] = (wq[e].float() @ x[arow[i]].float()) * ws[e].float()
        del wq
    if second_form:
        want = want * tw.reshape(-1)[slots][:, None]
    check(f"grouped seed={seed} {mode}", C.view(-1, N)[slots], want,
          rtol=1.5e-2 if mode == "fp8" else 1e-2, atol=(1.5e-2 * float(want.abs().mean()) + 1e-2) if mode == "fp8" else 1e-2)
    del C, x
    torch.cuda.empty_cache()


@pytest.mark.parametrize("first", range(0, 64, 8))
def test_dense_operators_on_layer_shapes(first):
    for seed in range(first, first + 8):
        dense_case(seed)


@pytest.mark.parametrize("first", range(0, 96, 12))
def test_grouped_gemm_on_layer_shapes(first):
    for seed in range(first, first + 12):
        grouped_case(seed)
