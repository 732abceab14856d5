"""GPU parity of routing, token->expert alignment and the activation glue
kernels against the CPU oracle.  Integer outputs (expert ids, sorted ids, block
table, fp8/int8 codes) are bit-exact; floating-point outputs are within
rtol 1e-2 / atol 1e-2 (in practice far tighter)."""
import numpy as np
import pytest
import torch

from oracle import fp8 as of8
from oracle import w8a8 as o8
from oracle import moe as om

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


@pytest.fixture(scope="module")
def ops():
    from vllm_gcu_amd.kernels import _custom_ops
    return _custom_ops


@pytest.fixture(scope="module")
def fmoe():
    from vllm_gcu_amd.kernels import fused_moe
    return fused_moe


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def min_margin(p, k):
    """smallest gap between consecutive sorted scores around the selection
    boundary; the seeded inputs must not hold near-ties"""
    s = -np.sort(-p, axis=-1)
    return float(np.min(s[:, :k] - s[:, 1:k + 1]))


# ------------------------------------------------------------- routing ----
@pytest.mark.parametrize("M,E,T", [(512, 8, 2), (256, 256, 8), (33, 60, 6), (1, 128, 1), (7, 1000, 4)])
def test_topk_softmax_ids_bit_exact(ops, M, E, T):
    print(f"case topk_softmax {M}x{E} top{T}", flush=True)
    g = np.random.default_rng(0).standard_normal((M, E)).astype(np.float32)
    assert min_margin(om.softmax_f32(g), T) > 1e-7
    w = torch.empty(M, T, dtype=torch.float32, device="cuda")
    ids = torch.empty(M, T, dtype=torch.int32, device="cuda")
    tei = torch.empty(M, T, dtype=torch.int32, device="cuda")
    ops.topk_softmax(w, ids, tei, dev(g))
    wo, io, to = om.topk_softmax(g, T)
    assert np.array_equal(ids.cpu().numpy(), io)
    assert np.array_equal(tei.cpu().numpy(), to)
    np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=1e-5, atol=1e-7)
    w2, i2 = ops.fused_topk(None, dev(g), T, True)
    wr, ir, _ = om.topk_softmax(g, T, renormalize=True)
    assert np.array_equal(i2.cpu().numpy(), ir)
    np.testing.assert_allclose(w2.cpu().numpy(), wr, rtol=1e-5, atol=1e-7)


def test_topk_softmax_ties_go_to_lower_index(ops):
    g = np.zeros((3, 16), dtype=np.float32)
    g[1, [3, 9]] = 2.0
    g[2, :] = -1.0
    w = torch.empty(3, 4, dtype=torch.float32, device="cuda")
    ids = torch.empty(3, 4, dtype=torch.int32, device="cuda")
    tei = torch.empty(3, 4, dtype=torch.int32, device="cuda")
    ops.topk_softmax(w, ids, tei, dev(g))
    assert ids.cpu().tolist() == [[0, 1, 2, 3], [3, 9, 0, 1], [0, 1, 2, 3]]
    assert np.array_equal(ids.cpu().numpy(), om.topk_softmax(g, 4)[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_topk_softmax_half_inputs(ops, dtype):
    g = torch.from_numpy(np.random.default_rng(2).standard_normal((40, 64)).astype(np.float32)).to(dtype)
    w = torch.empty(40, 2, dtype=torch.float32, device="cuda")
    ids = torch.empty(40, 2, dtype=torch.int32, device="cuda")
    ops.topk_softmax(w, ids, None, g.cuda())
    wo, io, _ = om.topk_softmax(g.float().numpy(), 2)
    # half-precision logits tie often; compare the selected *scores*
    p = om.softmax_f32(g.float().numpy())
    np.testing.assert_allclose(np.take_along_axis(p, ids.cpu().numpy().astype(np.int64), -1), wo, rtol=1e-5)
    np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("func,use_bias,renorm", [("softmax", False, True), ("sigmoid", True, True),
                                                   ("sigmoid", False, False), ("softmax", True, False)])
@pytest.mark.parametrize("M,E,T,ng,tg", [(256, 256, 8, 8, 4), (17, 64, 6, 8, 3), (5, 32, 4, 4, 2)])
def test_grouped_topk_bit_exact_ids(fmoe, func, use_bias, renorm, M, E, T, ng, tg):
    print(f"case grouped_topk {M}x{E} {func} bias={use_bias}", flush=True)
    rng = np.random.default_rng(1)
    g = rng.standard_normal((M, E)).astype(np.float32)
    bias = rng.normal(scale=0.1, size=E).astype(np.float32) if use_bias else None
    wo, io = om.grouped_topk(g, T, renorm, ng, tg, func, bias)
    w, ids = fmoe.grouped_topk(dev(g), dev(g), T, renorm, ng, tg, func, None if bias is None else dev(bias))
    assert w.dtype == torch.float32 and ids.dtype == torch.int32
    assert np.array_equal(ids.cpu().numpy(), io)
    np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=2e-5, atol=1e-7)
    per = E // ng
    for m in range(M):
        row = ids[m].cpu().numpy()
        assert len(set(row.tolist())) == T and len({int(e) // per for e in row}) <= tg


# --------------------------------------------------------------- align ----
def check_align(sorted_ids, expert_ids, npp, topk_ids, E, B, valid_rows=None, expert_map=None):
    so, eo, no = om.moe_align_block_size(topk_ids, E, B, valid_rows, expert_map)
    n = int(no[0])
    assert int(npp.cpu()[0]) == n
    assert np.array_equal(sorted_ids.cpu().numpy(), so)          # including pads and the unused tail
    assert np.array_equal(expert_ids.cpu().numpy()[:n // B], eo[:n // B])


@pytest.mark.parametrize("M,T,E,B", [(512, 2, 8, 64), (256, 8, 256, 64), (256, 8, 256, 16), (1, 1, 4, 16),
                                     (8192, 8, 256, 128), (3, 2, 8, 64), (1000, 6, 60, 32)])
def test_moe_align_bit_exact(fmoe, M, T, E, B):
    print(f"case align {M}x{T} E={E} B={B}", flush=True)
    ids = np.random.default_rng(M + E).integers(0, E, size=(M, T)).astype(np.int32)
    s, e, n = fmoe.moe_align_block_size(dev(ids), B, E)
    assert s.shape == (M * T + E * (B - 1),) and e.shape == ((M * T + E * (B - 1)) // B,)
    check_align(s, e, n, ids, E, B)


def test_moe_align_upstream_docstring_case(fmoe):
    ids = np.array([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=np.int32)
    s, e, n = fmoe.moe_align_block_size(dev(ids), 4, 5)
    assert int(n[0]) == 16
    assert s.cpu().tolist()[:16] == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert e.cpu().tolist()[:4] == [1, 2, 3, 4]


def test_moe_align_pad_variant_map_and_int64(fmoe, ops):
    rng = np.random.default_rng(9)
    ids = rng.integers(0, 16, size=(300, 4)).astype(np.int32)
    size = torch.tensor([123], dtype=torch.int32, device="cuda")
    s, e, n = fmoe.moe_align_block_size(dev(ids), 64, 16, None, size)
    check_align(s, e, n, ids, 16, 64, valid_rows=123)
    emap = rng.permutation(16).astype(np.int32)
    s, e, n = fmoe.moe_align_block_size(dev(ids), 64, 16, dev(emap), size)
    check_align(s, e, n, ids, 16, 64, valid_rows=123, expert_map=emap)
    s, e, n = fmoe.moe_align_block_size(dev(ids), 64, 16, dev(emap))
    check_align(s, e, n, ids, 16, 64, expert_map=emap)
    # fused variant with the map inside the operator, int64 ids
    cap = ids.size + 16 * 63
    s = torch.empty(cap, dtype=torch.int32, device="cuda")
    e = torch.empty(cap // 64, dtype=torch.int32, device="cuda")
    n = torch.empty(1, dtype=torch.int32, device="cuda")
    torch.ops._C.exts_moe_align_block_size(s, e, n, dev(ids.astype(np.int64)), size, dev(emap), 16, 64)
    check_align(s, e, n, ids, 16, 64, valid_rows=123, expert_map=emap)
    # invalid expert ids (masked tokens) are skipped
    ids2 = ids.copy()
    ids2[::7, 0] = -1
    s, e, n = fmoe.moe_align_block_size(dev(ids2), 64, 16)
    check_align(s, e, n, ids2, 16, 64)


# ---------------------------------------------------- activation glue ----
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_silu_and_mul_and_pad(ops, dtype):
    x = (torch.randn(37, 2, 512, generator=torch.Generator().manual_seed(0)) * 2).to(dtype)
    want = om.silu_and_mul(x.float().numpy())
    out = torch.empty(37, 2, 256, dtype=dtype, device="cuda")
    torch.ops._C.silu_and_mul(out, x.cuda())
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # exact after rounding to the activation dtype, up to 1 ulp from expf
    ref = torch.from_numpy(want).to(dtype).float().numpy()
    assert np.mean(out.float().cpu().numpy() == ref) > 0.99
    out2 = torch.full((37, 2, 256), 7.0, dtype=dtype, device="cuda")
    torch.ops._C.silu_and_mul_pad(out2.view(-1, 256), x.cuda().view(-1, 512), torch.tensor([20], dtype=torch.int32, device="cuda"))
    o2 = out2.view(-1, 256).float().cpu().numpy()
    np.testing.assert_allclose(o2[:20], want.reshape(-1, 256)[:20], rtol=RTOL, atol=ATOL)
    assert np.all(o2[20:] == 7.0)
    # 3-D input: `size` counts tokens (leading dimension), not flattened rows
    out3 = torch.full((37, 2, 256), 7.0, dtype=dtype, device="cuda")
    torch.ops._C.silu_and_mul_pad(out3, x.cuda(), torch.tensor([20], dtype=torch.int32, device="cuda"))
    o3 = out3.float().cpu().numpy()
    np.testing.assert_allclose(o3[:20], want[:20], rtol=RTOL, atol=ATOL)
    assert np.all(o3[20:] == 7.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,K,gs", [(256, 7168, 128), (5, 256, 64), (33, 1024, 256)])
def test_per_token_group_quant_fp8_bit_exact(ops, dtype, rows, K, gs):
    print(f"case group-quant {rows}x{K} g={gs} {dtype}", flush=True)
    x = torch.randn(rows, K, generator=torch.Generator().manual_seed(rows)).to(dtype)
    x[0, :gs] = 0                                     # all-zero group -> eps floor
    x[1 % rows, 3] = 300.0
    q, s = ops.per_token_group_quant_fp8(x.cuda(), gs)
    qo, so = of8.per_token_group_quant_fp8(x.float().numpy(), gs)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (rows, K // gs)
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), qo)
    # _with_size: rows past the count stay untouched
    qb = torch.zeros(rows, K, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    sb = torch.full((rows, K // gs), -1.0, dtype=torch.float32, device="cuda")
    nv = max(1, rows // 2)
    torch.ops._C.dynamic_per_token_group_fp8_quant_with_size(qb, sb, x.cuda(), torch.tensor([nv], dtype=torch.int32, device="cuda"), gs)
    assert np.array_equal(qb.view(torch.uint8).cpu().numpy()[:nv], qo[:nv])
    assert np.all(qb.view(torch.uint8).cpu().numpy()[nv:] == 0) and np.all(sb.cpu().numpy()[nv:] == -1.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_per_token_group_quant_fp8_rounding_boundaries_bit_exact(ops, dtype):
    """Quotients at and next to the midpoints between fp8 codes, group scales over 30 binades:
    the kernel divides through a shared reciprocal with residual corrections and must produce the
    codes of the IEEE division the oracle uses."""
    rng = np.random.default_rng(11)
    rows, K, gs = 384, 2048, 128
    table = of8.e4m3fn_decode_table().astype(np.float64)
    pos = np.sort(table[np.isfinite(table) & (table >= 0)])
    mids = (pos[:-1] + pos[1:]) / 2                         # rounding boundaries of e4m3fn
    lo, hi = (-14, 15) if dtype == torch.float16 else (-20, 20)
    scale = np.exp2(rng.uniform(lo, hi - 9, size=(rows, K // gs, 1))) * rng.uniform(1, 2, size=(rows, K // gs, 1))
    target = rng.choice(mids, size=(rows, K // gs, gs)) * rng.choice([1 - 2.0 ** -12, 1.0, 1 + 2.0 ** -12],
                                                                     size=(rows, K // gs, gs))
    x = target * scale * rng.choice([-1.0, 1.0], size=target.shape)
    x[:, :, 0] = 448.0 * scale[:, :, 0]                     # the element that sets the group's scale
    xt = torch.from_numpy(x.reshape(rows, K).astype(np.float32)).to(dtype)
    q, s = ops.per_token_group_quant_fp8(xt.cuda(), gs)
    qo, so = of8.per_token_group_quant_fp8(xt.float().numpy(), gs)
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), qo)


def test_silu_mul_group_quant_equals_unfused_sequence(ops):
    # csrc equivalence table: silu_mul_per_token_group_quant == silu_and_mul then
    # dynamic_per_token_group_fp8_quant (vllm_gcu/compilation/fx_fusion.py:102-108)
    x = torch.randn(256, 8, 4096, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).cuda()
    mid = torch.empty(256, 8, 2048, dtype=torch.bfloat16, device="cuda")
    torch.ops._C.silu_and_mul(mid, x)
    q_ref, s_ref = ops.per_token_group_quant_fp8(mid, 128)
    q = torch.empty(256, 8, 2048, dtype=torch.float8_e4m3fn, device="cuda")
    s = torch.empty(256, 8, 16, dtype=torch.float32, device="cuda")
    torch.ops._C.silu_mul_per_token_group_quant_with_size(q, s, x, torch.tensor([256], dtype=torch.int32, device="cuda"), 128)
    assert torch.equal(q.view(torch.uint8), q_ref.view(torch.uint8)) and torch.equal(s, s_ref)
    # and against the CPU oracle (rounded gate output, then group quant)
    a = om.silu_and_mul(x[:4].float().cpu().numpy())
    a = torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    qo, so = of8.per_token_group_quant_fp8(a, 128)
    got = q[:4].view(torch.uint8).cpu().numpy()
    assert np.mean(got == qo) > 0.995                    # expf ulp differences only
    np.testing.assert_allclose(s[:4].cpu().numpy(), so, rtol=1e-2)
    # partial size: only the first 100 tokens
    q2 = torch.zeros(256, 8, 2048, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    s2 = torch.zeros(256, 8, 16, dtype=torch.float32, device="cuda")
    torch.ops._C.silu_mul_per_token_group_quant_with_size(q2, s2, x, torch.tensor([100], dtype=torch.int32, device="cuda"), 128)
    assert torch.equal(q2[:100].view(torch.uint8), q_ref[:100].view(torch.uint8))
    assert torch.all(q2[100:].view(torch.uint8) == 0)


def test_per_token_and_static_fp8_quant(ops):
    x = torch.randn(19, 384, generator=torch.Generator().manual_seed(5)).to(torch.float16)
    q, s = ops.scaled_fp8_quant(x.cuda(), use_per_token_if_dynamic=True)
    qo, so = of8.per_token_quant_fp8(x.float().numpy())
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), qo) and np.array_equal(s.cpu().numpy(), so)
    sc = torch.tensor([0.02], dtype=torch.float32)
    q, _ = ops.scaled_fp8_quant(x.cuda(), sc.cuda())
    y = np.clip(x.float().numpy() / np.float32(0.02), -448, 448).astype(np.float32)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), of8.to_e4m3fn(y))


def test_mul_and_silu_mul_static_quant_equal_unfused_sequences(ops):
    # mul_static_fp8_quant == (left * right rounded to the input dtype) then static_scaled_fp8_quant;
    # silu_mul_static_int8_quant == silu_and_mul then static_scaled_int8_quant
    # (the fusion tables of vllm_gcu/compilation/fusion.py:129-152)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(37, 2, 512, generator=g).to(torch.bfloat16).cuda()
    sc = torch.tensor([0.05], dtype=torch.float32, device="cuda")
    n = torch.tensor([30], dtype=torch.int32, device="cuda")
    got = torch.zeros(37, 2, 256, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    torch.ops._C.mul_static_fp8_quant(got, x, sc, n)
    mid = (x[..., :256].float() * x[..., 256:].float()).to(torch.bfloat16)
    ref = torch.empty(37, 2, 256, dtype=torch.float8_e4m3fn, device="cuda")
    torch.ops._C.static_scaled_fp8_quant(ref, mid, sc)
    assert torch.equal(got[:30].view(torch.uint8), ref[:30].view(torch.uint8))
    assert torch.all(got[30:].view(torch.uint8) == 0)
    want = of8.to_e4m3fn(np.clip(mid[:30].float().cpu().numpy() / np.float32(0.05), -448, 448).astype(np.float32))
    assert np.array_equal(got[:30].view(torch.uint8).cpu().numpy(), want)

    for scale in (torch.tensor(0.02, dtype=torch.float32), torch.rand(256, generator=g) * 0.05 + 0.01):
        xs = torch.randn(19, 512, generator=g).to(torch.float16).cuda()
        q = torch.empty(19, 256, dtype=torch.int8, device="cuda")
        ops.silu_mul_quant(q, xs, scale.cuda())
        mid = torch.empty(19, 256, dtype=torch.float16, device="cuda")
        torch.ops._C.silu_and_mul(mid, xs)
        ref, _, _ = ops.scaled_int8_quant(mid, scale.cuda())
        assert torch.equal(q, ref)
        # and the CPU oracle on the same rounded activation
        assert np.array_equal(q.cpu().numpy(), o8.static_scaled_int8_quant(mid.cpu().numpy(), scale.numpy()))


@pytest.mark.parametrize("dtype,odtype", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
def test_moe_sum_pad(ops, dtype, odtype):
    x = torch.randn(50, 8, 1024, generator=torch.Generator().manual_seed(6)).to(dtype)
    out = torch.full((50, 1024), 3.0, dtype=odtype, device="cuda")
    torch.ops._moe_C.moe_sum_pad(out, x.cuda(), torch.tensor([41], dtype=torch.int32, device="cuda"), 1, False)
    want = om.moe_sum(x.float().numpy())
    got = out.float().cpu().numpy()
    if odtype == torch.float32:
        assert np.array_equal(got[:41], want[:41])           # same left-to-right fp32 sum
    else:
        assert np.array_equal(got[:41], torch.from_numpy(want[:41]).to(odtype).float().numpy())
    assert np.all(got[41:] == 3.0)


def test_valid_token_count_is_read_on_the_device_under_graph_replay(ops):
    """The ``*_pad`` / ``*_with_size`` operators take a device count so that a captured graph can be
    replayed with another number of valid tokens: the count (tokens) times the slots per token must
    be taken inside the kernel, not on the host at capture time."""
    rng = np.random.default_rng(3)
    M, T, D = 24, 4, 256
    x = dev(rng.standard_normal((M, T, 2 * D)).astype(np.float16))
    count = torch.full((1,), M, dtype=torch.int32, device="cuda")
    out = torch.zeros((M, T, D), dtype=torch.float16, device="cuda")
    q = torch.zeros((M, T, D), dtype=torch.float8_e4m3fn, device="cuda")
    qs = torch.zeros((M, T, D // 128), dtype=torch.float32, device="cuda")

    def step():
        torch.ops._C.silu_and_mul_pad(out, x, count)
        torch.ops._C.silu_mul_per_token_group_quant_with_size(q, qs, x, count, 128)

    step()                                      # eager warm-up, as a serving loop does before capturing
    torch.cuda.synchronize()
    full = out.clone()
    full_q = q.view(torch.uint8).clone()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    for n in (M, 5, 17, 0, M):
        count.fill_(n)
        out.fill_(-1.0)
        q.view(torch.uint8).fill_(0x7f)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out[:n], full[:n]), n
        assert (out[n:] == -1.0).all(), n       # rows past the count are left alone
        assert torch.equal(q.view(torch.uint8)[:n], full_q[:n]), n
        assert (q.view(torch.uint8)[n:] == 0x7f).all(), n
