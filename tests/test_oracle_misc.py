"""Pins oracle/w8a8.py, oracle/fp8.py and oracle/moe.py (no GPU)."""
import numpy as np
import pytest

from oracle import fp8, moe, norm, w8a8


# ---------------------------------------------------------------- int8 ----
def test_dynamic_int8_quant_known_rows():
    x = np.array([[127.0, -63.5, 0.5, 1.5, 2.5, -2.5],      # absmax 127 -> scale 1
                  [0.0, 0.0, 0.0, 0.0, 0.0, 0.0],             # zero row
                  [254.0, -254.0, 1.0, 3.0, -1.0, 5.0]], dtype=np.float32)
    q, s = w8a8.dynamic_scaled_int8_quant(x)
    assert s.shape == (3, 1) and s.dtype == np.float32
    assert s[:, 0].tolist() == [1.0, 0.0, 2.0]
    # round half to even: -63.5 -> -64, 0.5 -> 0, 1.5 -> 2, 2.5 -> 2, -2.5 -> -2
    assert q[0].tolist() == [127, -64, 0, 2, 2, -2]
    assert q[1].tolist() == [0] * 6
    # x/2: 0.5 -> 0, 1.5 -> 2, -0.5 -> 0, 2.5 -> 2
    assert q[2].tolist() == [127, -127, 0, 2, 0, 2]


def test_static_int8_quant_saturation_and_reciprocal_dtype():
    x = np.array([[1000.0, -1000.0, 3.0, 0.3]], dtype=np.float16)
    q = w8a8.static_scaled_int8_quant(x, np.float32(0.3))
    inv = np.float32(np.float16(1.0 / np.float32(0.3)))       # reciprocal lives in fp16
    want = [127, -128, int(np.rint(np.float32(3.0) * inv)), int(np.rint(np.float32(np.float16(0.3)) * inv))]
    assert q[0].tolist() == want
    qc = w8a8.static_scaled_int8_quant(np.ones((2, 3), np.float32), np.array([0.5, 0.25, 2.0], np.float32))
    assert qc.tolist() == [[2, 4, 0], [2, 4, 0]]              # 0.5 rounds to even 0


def test_int8_gemm_exact_vs_int64_bruteforce():
    rng = np.random.default_rng(0)
    a = rng.integers(-128, 128, size=(7, 2304), dtype=np.int8)
    b = rng.integers(-127, 128, size=(2304, 9), dtype=np.int8)
    a[0, :] = -128
    b[:, 0] = -127                                           # largest magnitude column
    got = w8a8.int8_gemm_i32(a, b)
    want = a.astype(np.int64) @ b.astype(np.int64)
    assert got.dtype == np.int32 and np.array_equal(got.astype(np.int64), want)


def test_scaled_mm_epilogue_shapes():
    acc = np.array([[100, -200], [300, 400]], dtype=np.int32)
    out = w8a8.scaled_mm_epilogue(acc, np.array([[0.5], [0.25]], np.float32), np.array([2.0, 4.0], np.float32))
    assert out.tolist() == [[100.0, -400.0], [150.0, 400.0]]
    out = w8a8.scaled_mm_epilogue(acc, np.float32(0.5), np.array([[2.0], [4.0]], np.float32),
                                  bias=np.array([1.0, -1.0]))
    assert out.tolist() == [[101.0, -401.0], [301.0, 799.0]]


def test_weight_only_int8_matches_float64():
    rng = np.random.default_rng(1)
    x = rng.integers(-3, 4, size=(3, 128)).astype(np.float16)
    w = rng.integers(-128, 128, size=(5, 128), dtype=np.int8)
    s = (2.0 ** -rng.integers(3, 6, size=5)).astype(np.float16)
    got = w8a8.weight_only_int8(x, w, s, -1)
    want = x.astype(np.float64) @ (w.astype(np.float64) * s.astype(np.float64)[:, None]).T
    assert np.array_equal(got.astype(np.float64), want)
    sg = (2.0 ** -rng.integers(3, 6, size=(2, 5))).astype(np.float16)
    got = w8a8.weight_only_int8(x, w, sg, 64)
    wd = w.astype(np.float64).reshape(5, 2, 64) * sg.T.astype(np.float64)[:, :, None]
    assert np.array_equal(got.astype(np.float64), x.astype(np.float64) @ wd.reshape(5, 128).T)


# ----------------------------------------------------------------- fp8 ----
def test_e4m3fn_table_landmarks():
    t = fp8.e4m3fn_decode_table()
    assert t[0x00] == 0.0 and t[0x7E] == 448.0 and t[0xFE] == -448.0
    assert np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    assert t[0x01] == 2.0 ** -9 and t[0x08] == 2.0 ** -6 and t[0x38] == 1.0
    assert t[0x3C] == 1.5 and t[0x40] == 2.0


def test_to_e4m3fn_matches_table_bruteforce():
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.uniform(-448, 448, 300), rng.normal(0, 1, 300),
                        rng.normal(0, 0.01, 100),
                        # exact ties between neighbours: (1+1/16) -> even (1.0), (1+3/16) -> 1.25
                        np.array([1.0625, 1.1875, 17.0, 19.0, 416.0 + 16.0, 448.0, -448.0, 0.0,
                                  2.0 ** -10, 3 * 2.0 ** -10])]).astype(np.float32)
    got = fp8.to_e4m3fn(x)
    want = fp8.e4m3fn_encode_bruteforce(x)
    assert np.array_equal(got, want)
    assert fp8.from_e4m3fn(fp8.to_e4m3fn(np.array([1.0625, 1.1875], np.float32))).tolist() == [1.0, 1.25]


def test_per_token_group_quant_fp8_closed_form():
    x = np.zeros((2, 256), dtype=np.float32)
    x[0, :128] = np.linspace(-448, 448, 128)        # absmax 448 -> scale 1
    x[0, 128:] = 0.0                                # all-zero group -> eps floor
    x[1, :128] = 2 * np.linspace(-448, 448, 128)    # scale 2
    x[1, 128:] = 7.0
    q, s = fp8.per_token_group_quant_fp8(x, 128)
    assert s.shape == (2, 2)
    assert s[0, 0] == 1.0 and s[1, 0] == 2.0
    assert s[0, 1] == np.float32(np.float32(1e-10) / np.float32(448.0))
    assert s[1, 1] == np.float32(np.float32(7.0) / np.float32(448.0))
    assert np.array_equal(q[0, :128], q[1, :128])
    assert np.all(q[0, 128:] == 0)
    # 7 / (7/448) rounds to 448 exactly or to its fp32 neighbour; both clamp/encode to 0x7E
    assert np.all(q[1, 128:] == 0x7E)
    assert q[0, 0] == 0xFE and q[0, 127] == 0x7E


def test_block_fp8_gemm_vs_float64():
    rng = np.random.default_rng(3)
    M, K, N = 4, 256, 160
    a = rng.integers(0, 0x41, size=(M, K)).astype(np.uint8) | (rng.integers(0, 2, size=(M, K)).astype(np.uint8) << 7)
    b = rng.integers(0, 0x41, size=(N, K)).astype(np.uint8) | (rng.integers(0, 2, size=(N, K)).astype(np.uint8) << 7)
    a[a & 0x7F == 0x7F] = 0
    b[b & 0x7F == 0x7F] = 0
    As = rng.uniform(0.5, 2, size=(M, 2)).astype(np.float32)
    Bs = rng.uniform(0.5, 2, size=(2, 2)).astype(np.float32)
    got = fp8.block_fp8_gemm(a, As, b, Bs)
    t = fp8.e4m3fn_decode_table()
    want = np.zeros((M, N))
    for kb in range(2):
        part = t[a[:, kb * 128:(kb + 1) * 128]] @ t[b[:, kb * 128:(kb + 1) * 128]].T
        want += part * As[:, kb:kb + 1].astype(np.float64) * np.repeat(Bs[:, kb], 128)[:N][None, :]
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-4)


# ------------------------------------------------------------- routing ----
def test_topk_softmax_bruteforce_and_ties():
    g = np.array([[0.0, 1.0, 1.0, -1.0], [2.0, 0.0, 0.0, 2.0]], dtype=np.float32)
    w, ids, tei = moe.topk_softmax(g, 2)
    assert ids.tolist() == [[1, 2], [0, 3]]          # ties -> lower index first
    e = np.exp(g[0].astype(np.float64)); p = e / e.sum()
    np.testing.assert_allclose(w[0], [p[1], p[2]], rtol=1e-6)
    assert tei.tolist() == [[0, 2], [1, 3]]          # k * M + row
    w2, _, _ = moe.topk_softmax(g, 2, renormalize=True)
    np.testing.assert_allclose(w2.sum(-1), 1.0, rtol=1e-6)


def _grouped_topk_scalar(g, topk, renorm, ngroup, tgroup, func, bias):
    M, E = g.shape
    per = E // ngroup
    W = np.zeros((M, topk)); I = np.zeros((M, topk), dtype=int)
    for m in range(M):
        row = g[m].astype(np.float64)
        if func == "softmax":
            e = np.exp(row - row.max()); sc = e / e.sum()
        else:
            sc = 1 / (1 + np.exp(-row))
        sel = sc + (bias.astype(np.float64) if bias is not None else 0)
        gs = []
        for G in range(ngroup):
            v = sorted(sel[G * per:(G + 1) * per], reverse=True)
            gs.append(v[0] + v[1] if bias is not None else v[0])
        keep = sorted(range(ngroup), key=lambda G: (-gs[G], G))[:tgroup]
        cand = [i for i in range(E) if i // per in keep]
        best = sorted(cand, key=lambda i: (-sel[i], i))[:topk]
        ww = np.array([sc[i] for i in best])
        if renorm:
            ww = ww / ww.sum()
        W[m] = ww; I[m] = best
    return W, I


@pytest.mark.parametrize("func,use_bias", [("softmax", False), ("sigmoid", True), ("sigmoid", False), ("softmax", True)])
def test_grouped_topk_vs_scalar_bruteforce(func, use_bias):
    rng = np.random.default_rng(4)
    g = rng.normal(size=(16, 32)).astype(np.float32)
    bias = rng.normal(scale=0.1, size=32).astype(np.float32) if use_bias else None
    w, ids = moe.grouped_topk(g, 4, True, 4, 2, func, bias)
    W, I = _grouped_topk_scalar(g, 4, True, 4, 2, func, bias)
    assert np.array_equal(ids, I)
    np.testing.assert_allclose(w, W, rtol=2e-5)
    # structure: ids distinct, inside exactly 2 groups
    for m in range(16):
        assert len(set(ids[m])) == 4 and len({i // 8 for i in ids[m]}) <= 2


# --------------------------------------------------------------- align ----
def test_moe_align_upstream_docstring_case():
    topk_ids = np.array([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=np.int32)
    s, e, n = moe.moe_align_block_size(topk_ids, 5, 4)
    assert n[0] == 16 and s.shape == (12 + 5 * 3,) and e.shape == (27 // 4,)
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert e[:4].tolist() == [1, 2, 3, 4]
    assert np.all(s[16:] == 12)


def test_moe_align_invariants_pad_and_map():
    rng = np.random.default_rng(5)
    ids = rng.integers(0, 8, size=(50, 2)).astype(np.int32)
    s, e, n = moe.moe_align_block_size(ids, 8, 16)
    npp = int(n[0]); flat = ids.reshape(-1)
    assert npp % 16 == 0
    valid = s[:npp][s[:npp] < flat.size]
    assert sorted(valid.tolist()) == list(range(flat.size))
    for b in range(npp // 16):
        blk = s[b * 16:(b + 1) * 16]; v = blk[blk < flat.size]
        assert len(v) > 0 and np.all(flat[v] == e[b]) and np.all(np.diff(v) > 0)
    # _pad variant: only the first 20 rows
    s2, e2, n2 = moe.moe_align_block_size(ids, 8, 16, valid_rows=20)
    v2 = s2[:int(n2[0])]; v2 = v2[v2 < flat.size]
    assert sorted(v2.tolist()) == list(range(40))
    # expert_map relabels blocks
    emap = np.array([7, 6, 5, 4, 3, 2, 1, 0])
    _, e3, _ = moe.moe_align_block_size(ids, 8, 16, expert_map=emap)
    assert np.array_equal(e3[:npp // 16], 7 - e[:npp // 16])
    # an empty expert takes no block
    ids4 = np.array([[0, 2]], dtype=np.int32)
    s4, e4, n4 = moe.moe_align_block_size(ids4, 3, 4)
    assert n4[0] == 8 and e4[:2].tolist() == [0, 2] and s4[:8].tolist() == [0, 2, 2, 2, 1, 2, 2, 2]


def test_silu_sum_and_fused_experts_identity():
    x = np.array([[0.0, 1.0, -2.0, 3.0, 5.0, 7.0]], dtype=np.float32)
    out = moe.silu_and_mul(x)
    want = [0.0, 1.0 / (1 + np.exp(-1.0)) * 5.0, -2.0 / (1 + np.exp(2.0)) * 7.0]
    np.testing.assert_allclose(out[0], want, rtol=1e-6)
    assert moe.moe_sum(np.arange(12, dtype=np.float32).reshape(2, 3, 2)).tolist() == [[6.0, 9.0], [24.0, 27.0]]
    # fused sequence == naive per-expert MoE
    # (vllm_gcu/models/deepseek_moe_quant/deepseek_moe_quant.py:168-187 pattern)
    rng = np.random.default_rng(6)
    M, H, I, E, T = 6, 16, 8, 4, 2
    xs = rng.normal(size=(M, H)).astype(np.float32)
    w1 = rng.normal(size=(E, H, 2 * I)).astype(np.float32) * 0.3
    w2 = rng.normal(size=(E, I, H)).astype(np.float32) * 0.3
    tw, ti, _ = moe.topk_softmax(rng.normal(size=(M, E)).astype(np.float32), T, True)
    got = moe.fused_experts(xs, lambda e: w1[e], lambda e: w2[e], tw, ti, lambda a: a.astype(np.float32))
    want = np.zeros((M, H))
    for m in range(M):
        for t in range(T):
            e = ti[m, t]
            h = xs[m].astype(np.float64) @ w1[e].astype(np.float64)
            a = h[:I] / (1 + np.exp(-h[:I])) * h[I:]
            want[m] += tw[m, t] * (a @ w2[e].astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [np.uint8, np.uint16])
def test_kslab_pack_is_inverted_by_scalar_walk_and_keeps_kib_runs(dtype):
    rng = np.random.default_rng(5)
    N, K = 128, 256
    w = rng.integers(0, np.iinfo(dtype).max, size=(N, K), dtype=dtype)
    p = w8a8.kslab_pack(w)
    assert p.shape == w.shape and p.dtype == w.dtype
    assert np.array_equal(w8a8.kslab_unpack(p), w)
    # batched input packs each matrix on its own
    both = w8a8.kslab_pack(np.stack([w, w[::-1]]))
    assert np.array_equal(both[0], p) and np.array_equal(w8a8.kslab_unpack(both[1]), w[::-1])
    # first KiB = vector 0 of tile 0 of block (0, 0): lane l holds 16 bytes of row l % 16 at byte 32*wb*(l//16)
    wb = w.dtype.itemsize
    kib = p.view(np.uint8).reshape(-1)[:1024].reshape(64, 16)
    rows = w.view(np.uint8).reshape(N, K * wb)
    for lane in (0, 1, 15, 16, 37, 63):
        off = 32 * wb * (lane // 16)
        assert np.array_equal(kib[lane], rows[lane % 16, off:off + 16])


def _f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float32)


def test_rms_norm_closed_forms_and_invariants():
    rng = np.random.default_rng(41)
    K = 256
    w = _f16(rng.uniform(0.5, 1.5, K))
    # constant row: z / rms(z) = sign -> out = sign * w (eps = 0)
    for c in (3.0, -0.25):
        out = norm.rms_norm(np.full((1, K), c, np.float32), w, 0.0, _f16)
        assert np.array_equal(out[0], np.sign(c) * w)
    # power-of-two scale invariance is exact without eps
    x = _f16(rng.standard_normal((5, K)))
    assert np.array_equal(norm.rms_norm(x, w, 0.0, _f16), norm.rms_norm(4.0 * x, w, 0.0, _f16))
    # float64 evaluation within the rounding of two fp16 roundings
    ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5) * w
    np.testing.assert_allclose(norm.rms_norm(x, w, 1e-5, _f16), ref, rtol=2e-3, atol=1e-4)
    # a huge eps shrinks the output towards zero: rsqrt(var + eps) ~ eps^-1/2
    big = norm.rms_norm(x, w, 1e6, _f16)
    np.testing.assert_allclose(big, _f16(_f16(x * np.float32(1e-3)) * w), rtol=2e-3, atol=1e-6)


def test_fused_add_rms_norm_is_add_then_norm():
    rng = np.random.default_rng(43)
    K = 128
    x, r = _f16(rng.standard_normal((4, K))), _f16(rng.standard_normal((4, K)) * 3)
    w = _f16(rng.uniform(0.5, 1.5, K))
    out, z = norm.fused_add_rms_norm(x, r, w, 1e-6, _f16)
    assert np.array_equal(z, _f16(x + r))
    assert np.array_equal(out, norm.rms_norm(z, w, 1e-6, _f16))


def test_moe_expert_int8_quant_known_rows_and_scalar_loop():
    """q[t] = sat_s8(rne(x[t // topk] * rec[expert(t)])), product in float32
    (oracle/w8a8.py; the reference stores reciprocals, w8a8.py:226-236)."""
    # hand-written rows: K = 6, two experts
    x = np.array([[1.0, 2.5, -2.5, 3.5, 1000.0, -1000.0],      # ties at .5 go to even; saturation
                  [0.0, 0.0, 0.0, 0.0, 0.0, 0.0]], np.float16)  # zero row
    rec = np.array([[1.0, 1.0, 1.0, 1.0, 1.0, 1.0],
                    [0.5, 0.2, 0.2, 1.0, 0.127, 0.128]], np.float32)
    ids = np.array([[0, 1], [1, 0]], np.int32)                  # topk 2
    q = w8a8.moe_expert_int8_quant(x, rec, ids)
    assert q.dtype == np.int8 and q.shape == (4, 6)
    assert q[0].tolist() == [1, 2, -2, 4, 127, -128]            # expert 0: 2.5 -> 2, -2.5 -> -2, 3.5 -> 4
    # expert 1: the float32 products decide (0.2 is not exact), evaluated one by one
    want1 = [int(np.clip(np.rint(np.float32(a) * np.float32(b)), -128, 127)) for a, b in zip(x[0], rec[1])]
    assert q[1].tolist() == want1 and want1[0] == 0 and want1[4] == 127 and want1[5] == -128
    assert not q[2].any() and not q[3].any()
    # scalar loop over (token, slot), topk 1 and 2, float64 product where exact -> same rounding
    rng = np.random.default_rng(11)
    for topk in (1, 2):
        M, K, E = 5, 16, 3
        xr = (rng.integers(-40, 41, size=(M, K)) / 4.0).astype(np.float16)     # quarter steps: exact products
        rr = (2.0 ** rng.integers(-2, 3, size=(E, K))).astype(np.float32)      # powers of two
        tid = rng.integers(0, E, size=(M, topk)).astype(np.int32)
        got = w8a8.moe_expert_int8_quant(xr, rr, tid)
        for m in range(M):
            for s in range(topk):
                e = int(tid[m, s])
                for k in range(K):
                    y = float(xr[m, k]) * float(rr[e, k])
                    r = round(y)                        # Python rounds half to even
                    assert int(got[m * topk + s, k]) == max(-128, min(127, r))
    # 1-D ids are one slot per row
    got = w8a8.moe_expert_int8_quant(x, rec, np.array([1, 0], np.int32))
    assert got[0].tolist() == want1 and not got[1].any()


def test_per_token_quant_fp8_is_group_quant_with_one_group():
    """dynamic_per_token_scaled_fp8_quant: one scale per row = absmax / 448
    (csrc/src/dynamic_per_token_scaled_fp8_quant.cpp; FP8_E4M3_MAX native_vllm.h:34)."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal((4, 96)).astype(np.float32)
    x[2] = 0.0
    x[3, 5] = 448.0 * 3
    q, s = fp8.per_token_quant_fp8(x)
    assert q.shape == x.shape and s.shape == (4, 1)
    absmax = np.abs(x).max(axis=-1)
    assert np.array_equal(s[:, 0], (np.maximum(absmax, np.float32(1e-10)) / np.float32(448.0)).astype(np.float32))
    # the largest element of each non-zero row lands exactly on +-448 (code 0x7e / 0xfe)
    for m in (0, 1, 3):
        k = int(np.abs(x[m]).argmax())
        assert int(q[m, k]) & 0x7F == 0x7E
    assert not q[2].any()
    # equals the group quantiser called with the whole row as its group, and rows are independent
    q2, s2 = fp8.per_token_group_quant_fp8(x, 96)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    q1, s1 = fp8.per_token_quant_fp8(x[1:2])
    assert np.array_equal(q1[0], q[1]) and s1[0, 0] == s[1, 0]
    # dequantised codes reproduce x within half an e4m3 step (2^-4 relative) of the row maximum
    back = fp8.from_e4m3fn(q) * s
    assert np.all(np.abs(back - x) <= absmax[:, None] / 16 + 1e-12)


def test_scaled_fp8_mm_vs_float64_and_block_identity():
    """Scales outside the K sum (cutlass_scaled_mm.cpp:12-36 on fp8 operands): float64 brute force, every
    scale shape, and the identity with the block-scaled GEMM when the block scales do not vary along K
    and the channel scales do not vary inside a 128-column block."""
    rng = np.random.default_rng(31)
    M, K, N = 5, 256, 256
    a = fp8.to_e4m3fn(np.clip(rng.standard_normal((M, K)) * 3, -448, 448).astype(np.float32))
    b = fp8.to_e4m3fn(np.clip(rng.standard_normal((N, K)) * 0.5, -448, 448).astype(np.float32))
    xs = rng.uniform(0.01, 0.1, size=M).astype(np.float32)
    ws = rng.uniform(0.001, 0.02, size=N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tab = fp8.e4m3fn_decode_table()
    want = (tab[a] @ tab[b].T) * xs[:, None].astype(np.float64) * ws[None, :].astype(np.float64) + bias
    got = fp8.scaled_fp8_mm(a, xs, b, ws, bias)
    assert got.dtype == np.float32 and got.shape == (M, N)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    # scale shapes: [M, 1] / [N, 1] equal the flat ones; scalars broadcast
    assert np.array_equal(fp8.scaled_fp8_mm(a, xs.reshape(M, 1), b, ws.reshape(N, 1), bias), got)
    one = fp8.scaled_fp8_mm(a, np.float32(0.5), b, np.array([0.25], np.float32))
    np.testing.assert_allclose(one, (tab[a] @ tab[b].T) * 0.125, rtol=1e-5, atol=1e-5)
    # a known small case: codes 0x38 = 1.0, 0x40 = 2.0, 0xb8 = -1.0
    a1 = np.array([[0x38, 0x40, 0xb8, 0x00]], np.uint8)
    b1 = np.array([[0x40, 0x40, 0x40, 0x40], [0x38, 0x00, 0x38, 0x7e]], np.uint8)
    assert fp8.scaled_fp8_mm(a1, 2.0, b1, np.array([1.0, 0.5], np.float32)).tolist() == [[8.0, 0.0]]
    # block identity (exact here: scales are powers of two, so scaling commutes with the fp32 additions)
    xs2 = (2.0 ** rng.integers(-4, 1, size=M)).astype(np.float32)
    wsb = (2.0 ** rng.integers(-6, -2, size=N // 128)).astype(np.float32)
    blk = fp8.block_fp8_gemm(a, np.repeat(xs2[:, None], K // 128, 1), b, np.repeat(wsb[:, None], K // 128, 1))
    pc = fp8.scaled_fp8_mm(a, xs2, b, np.repeat(wsb, 128))
    np.testing.assert_allclose(pc, blk, rtol=2e-6, atol=1e-6)
