"""Pins the int4 format restatements in oracle/w4.py with hand-derived
known-answer words, inverses and scalar brute force (no GPU)."""
import numpy as np
import pytest

from oracle import w4


def i32(x):
    return np.array(x, dtype=np.uint32).view(np.int32)


def test_gptq_weight_known_words():
    # nibble i of a word is row 8r+i: 0x76543210 -> 0..7, 0xFEDCBA98 -> 8..15
    qw = i32([[0x76543210, 0xFEDCBA98], [0xFFFFFFFF, 0x00000000], [0x0000000F, 0xF0000000]])
    w = w4.gptq_unpack_weight(qw)
    assert w.shape == (24, 2)
    assert w[:8, 0].tolist() == [0, 1, 2, 3, 4, 5, 6, 7]
    assert w[:8, 1].tolist() == [8, 9, 10, 11, 12, 13, 14, 15]
    assert w[8:16, 0].tolist() == [15] * 8 and w[8:16, 1].tolist() == [0] * 8
    assert w[16:24, 0].tolist() == [15, 0, 0, 0, 0, 0, 0, 0]
    assert w[16:24, 1].tolist() == [0, 0, 0, 0, 0, 0, 0, 15]


def test_gptq_zeros_known_words_and_plus_one_wrap():
    # nibble j of column c is n = 8c+j; z = (stored + 1) & 15
    qz = i32([[0x76543210, 0xFEDCBA98]])
    z = w4.gptq_unpack_zeros(qz)
    assert z.shape == (1, 16)
    assert z[0].tolist() == [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 0]


def test_awq_known_word_interleave():
    # nibble i -> temp column i; logical column j reads temp [0,4,1,5,2,6,3,7][j]
    q = i32([[0x76543210]])
    assert w4.awq_unpack(q)[0].tolist() == [0, 4, 1, 5, 2, 6, 3, 7]
    q = i32([[0x0000000F, 0x000000F0]])
    assert w4.awq_unpack(q)[0].tolist() == [15, 0, 0, 0, 0, 0, 0, 0,
                                              0, 0, 15, 0, 0, 0, 0, 0]


@pytest.mark.parametrize("seed", [0, 1])
def test_pack_unpack_inverses_all_values(seed):
    rng = np.random.default_rng(seed)
    K, N, G = 256, 32, 2
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    q[:16, 0] = np.arange(16)          # every nibble value present
    z = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    z[0, :16] = np.arange(16)
    assert np.array_equal(w4.gptq_unpack_weight(w4.gptq_pack_weight(q)), q)
    assert np.array_equal(w4.gptq_unpack_zeros(w4.gptq_pack_zeros(z)), z)
    assert np.array_equal(w4.awq_unpack(w4.awq_pack(q)), q)
    assert np.array_equal(w4.ref_halfgroup_unpack(w4.ref_halfgroup_pack(q)), q)


def test_gptq_unpack_bruteforce_scalar():
    rng = np.random.default_rng(3)
    qw = rng.integers(-2**31, 2**31 - 1, size=(4, 5), dtype=np.int64).astype(np.int32)
    w = w4.gptq_unpack_weight(qw)
    for r in range(4):
        for n in range(5):
            word = int(qw[r, n]) & 0xFFFFFFFF
            for i in range(8):
                assert w[8 * r + i, n] == (word >> (4 * i)) & 15
    qz = rng.integers(-2**31, 2**31 - 1, size=(3, 2), dtype=np.int64).astype(np.int32)
    z = w4.gptq_unpack_zeros(qz)
    for g in range(3):
        for c in range(2):
            word = int(qz[g, c]) & 0xFFFFFFFF
            for j in range(8):
                assert z[g, 8 * c + j] == (((word >> (4 * j)) & 15) + 1) % 16


def test_awq_unpack_bruteforce_scalar():
    rng = np.random.default_rng(4)
    q = rng.integers(-2**31, 2**31 - 1, size=(3, 4), dtype=np.int64).astype(np.int32)
    w = w4.awq_unpack(q)
    order = [0, 4, 1, 5, 2, 6, 3, 7]
    for r in range(3):
        for c in range(4):
            word = int(q[r, c]) & 0xFFFFFFFF
            for j in range(8):
                assert w[r, 8 * c + j] == (word >> (4 * order[j])) & 15


def test_halfgroup_known_bytes_and_bruteforce():
    K, N = 256, 3
    w = np.zeros((K, N), dtype=np.uint8)
    for k in range(K):
        for n in range(N):
            w[k, n] = (k * 7 + n * 3 + (k // 64)) % 16
    rw = w4.ref_halfgroup_pack(w)
    assert rw.shape == (K // 2, N) and rw.dtype == np.uint8
    for G in range(K // 128):
        for i in range(64):
            for n in range(N):
                lo = w[G * 128 + i, n]
                hi = w[G * 128 + 64 + i, n]
                assert rw[G * 64 + i, n] == lo | (hi << 4)
    # literal: first group, rows 0 and 64 of column 0 -> byte 0
    assert int(rw[0, 0]) == int(w[0, 0]) + 16 * int(w[64, 0])


def test_rearrange_gptq_restatement():
    rng = np.random.default_rng(5)
    K, N, g = 256, 16, 128
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    rweight, zeros_f = w4.rearrange_gptq(w4.gptq_pack_weight(q), w4.gptq_pack_zeros(z), s)
    assert np.array_equal(w4.ref_halfgroup_unpack(rweight), q)
    assert zeros_f.dtype == np.float16
    # z*s rounded once to fp16
    want = (z.astype(np.float64) * s.astype(np.float64)).astype(np.float16)
    assert np.array_equal(zeros_f, want)


def test_rearrange_awq_restatement():
    rng = np.random.default_rng(6)
    K, N, g = 128, 16, 128
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = rng.uniform(0.001, 0.01, size=(K // g, N)).astype(np.float16)
    rw, zi = w4.rearrange_awq(w4.awq_pack(q), w4.awq_pack(z), s, zeros_in_int8=True)
    assert rw.dtype == np.int8 and zi.dtype == np.int8
    assert np.array_equal(w4.ref_halfgroup_unpack(rw.view(np.uint8)), q)
    assert np.array_equal(zi, z.astype(np.int8))
    rw2, z2 = w4.rearrange_awq(w4.awq_pack(q), None, s, use_w4a8=True, rearrange_group=64)
    assert z2 is None
    got = w4.ref_halfgroup_unpack(rw2, 64).astype(np.int8)
    assert np.array_equal(got, ((q.astype(np.int8) - 8) & 15))


def test_rearrange_awq_w4a8_branch_scalar_walk():
    """use_w4a8 (rearrange.py:104-106): nibbles hold w - 8 in two's complement, zeros dropped;
    with rearrange_group 64 the low nibble of byte row 32 G + i is k = 64 G + i, the high
    nibble k = 64 G + 32 + i -- checked element by element."""
    rng = np.random.default_rng(21)
    K, N = 128, 16
    wl = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.02, size=(K // 64, N)).astype(np.float32)
    rw, z = w4.rearrange_awq(w4.awq_pack(wl), None, scales, rearrange_group=64, zeros_in_int8=True, use_w4a8=True)
    assert z is None and rw.dtype == np.int8 and rw.shape == (K // 2, N)
    b = rw.view(np.uint8)
    for k in range(K):
        G, i = divmod(k, 64)
        for n in range(N):
            byte = int(b[32 * G + (i & 31), n])
            nib = (byte >> 4) if i >= 32 else (byte & 15)
            signed = nib - 16 if nib >= 8 else nib
            assert signed == int(wl[k, n]) - 8


def test_native_layout_inverse_and_spot_checks():
    rng = np.random.default_rng(7)
    K, N = 256, 256
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    packed = w4.native_pack(q)
    assert packed.shape == (K // 8, N) and packed.dtype == np.int32
    assert np.array_equal(w4.native_unpack(packed, K, N), q)
    flat = packed.view(np.uint32).reshape(-1)
    # word address of (slab S, group g, tile t, lane, step s)
    def word(S, g, t, lane, s):
        return int(flat[((((S * (K // 128) + g) * 8 + t) * 64 + lane) * 4) + s])
    # k = 128g + 32s + 8kq + j ; n = 128S + 8c + t ; nibble [0,4,1,5,2,6,3,7][j]
    wd = word(1, 1, 5, 16 * 2 + 9, 3)
    k0, n = 128 + 96 + 16, 128 + 72 + 5
    nibs = [(wd >> (4 * p)) & 15 for p in range(8)]
    assert nibs[0] == q[k0 + 0, n] and nibs[4] == q[k0 + 1, n]
    assert nibs[1] == q[k0 + 2, n] and nibs[5] == q[k0 + 3, n]
    assert nibs[2] == q[k0 + 4, n] and nibs[6] == q[k0 + 5, n]
    assert nibs[3] == q[k0 + 6, n] and nibs[7] == q[k0 + 7, n]


def test_dequantize_closed_form_and_gemm_exact_cases():
    rng = np.random.default_rng(8)
    K, N, g, M = 256, 24, 128, 5
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    # power-of-two scales and small-integer activations: every product and
    # every partial sum is exactly representable -> float64 brute force must
    # agree bit for bit
    s = (2.0 ** -rng.integers(4, 8, size=(K // g, N))).astype(np.float16)
    x = rng.integers(-4, 5, size=(M, K)).astype(np.float16)
    out = w4.w4a16_gemm(x, q, z, s, g)
    want = np.zeros((M, N), dtype=np.float64)
    for k in range(K):
        wk = (q[k].astype(np.float64) - z[k // g].astype(np.float64)) * s[k // g].astype(np.float64)
        want += x[:, k:k + 1].astype(np.float64) * wk[None, :]
    assert np.array_equal(out.astype(np.float64), want)
    # z = None means the symmetric default 8
    out8 = w4.w4a16_gemm(x, q, None, s, g)
    out8b = w4.w4a16_gemm(x, q, np.full_like(z, 8), s, g)
    assert np.array_equal(out8, out8b)
    # pre-scaled-zero form describes the same matrix when z*s is exact
    zs = (z.astype(np.float32) * s.astype(np.float32)).astype(np.float16)
    assert np.array_equal(w4.dequantize_prescaled_zeros(q, zs, s, g), w4.dequantize(q, z, s, g))
    # bias
    b = rng.integers(-3, 4, size=N).astype(np.float16)
    assert np.array_equal(w4.w4a16_gemm(x, q, z, s, g, bias=b), out + b.astype(np.float32))


# ------------------------------------------------------------------------
# Golden vectors written from the reference's own rearrange.py
# (tests/golden/make_rearrange_vectors.py; rearrange.py:6-133)
# ------------------------------------------------------------------------
def _golden():
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rearrange_vectors.npz")
    return np.load(path, allow_pickle=False)


def test_rearrange_gptq_equals_reference_vectors():
    g = _golden()
    rw, zf = w4.rearrange_gptq(g["gptq_g128_qweight"], g["gptq_g128_qzeros"], g["gptq_g128_scales"])
    assert rw.dtype == np.uint8 and np.array_equal(rw, g["gptq_g128_rweight"])
    assert zf.dtype == np.float16 and np.array_equal(zf.view(np.uint16), g["gptq_g128_zeros"].view(np.uint16))
    # the first packed zero word is all ones: every nibble 15 wraps to 0 -> z*s == 0
    assert np.all(g["gptq_g128_zeros"][0, :8] == 0)
    rw2, z2 = w4.rearrange_gptq(g["gptq_g128_qweight"], None, g["gptq_g128_scales"])
    assert z2 is None and np.array_equal(rw2, g["gptq_g128_rweight"])


def test_rearrange_awq_equals_reference_vectors():
    g = _golden()
    qw, qz, sc = g["awq_qweight"], g["awq_qzeros"], g["awq_scales"]
    rw, zf = w4.rearrange_awq(qw, qz, sc)
    assert rw.dtype == np.uint8 and np.array_equal(rw, g["awq_fzeros_rweight"])
    assert zf.dtype == np.float16 and np.array_equal(zf.view(np.uint16), g["awq_fzeros_zeros"].view(np.uint16))
    rw, zi = w4.rearrange_awq(qw, qz, sc, zeros_in_int8=True)
    assert rw.dtype == np.int8 and np.array_equal(rw.view(np.uint8), g["awq_fzeros_rweight"])
    assert zi.dtype == np.int8 and np.array_equal(zi, g["awq_i8zeros_zeros"])
    rw, zn = w4.rearrange_awq(qw, qz, sc, rearrange_group=64, zeros_in_int8=True, use_w4a8=True)
    assert zn is None and rw.dtype == np.int8 and np.array_equal(rw, g["awq_w4a8_g64_rweight"])


def test_native_pack_zeros_known_word():
    """Nibble j of word c holds z[g, 8c + j], true value: columns 0..7 -> 0x76543210."""
    z = np.arange(16, dtype=np.uint8).reshape(1, 16)
    words = w4.native_pack_zeros(z).view(np.uint32)
    assert words.shape == (1, 2)
    assert int(words[0, 0]) == 0x76543210 and int(words[0, 1]) == 0xFEDCBA98
    # and it differs from the GPTQ exporter's word (which stores z - 1)
    assert int(w4.gptq_pack_zeros(z).view(np.uint32)[0, 0]) == 0x6543210F
    # scalar walk on random data
    rng = np.random.default_rng(3)
    z = rng.integers(0, 16, size=(3, 24), dtype=np.uint8)
    words = w4.native_pack_zeros(z).view(np.uint32)
    for gi in range(3):
        for n in range(24):
            assert (int(words[gi, n // 8]) >> (4 * (n % 8))) & 15 == int(z[gi, n])
