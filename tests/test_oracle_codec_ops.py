"""Pins the CPU oracle's codec and per-op functions WITHOUT the reference running (it is Java; the
image has no JVM, and the reference ships no golden vectors): known answers from the reference's own
self-check input, closed forms, brute force in float64, and invariants chosen so that a dropped
term, a wrong sign/index or a transposed operand fails."""
import math

import numpy as np
import pytest

from tests import np_ref


# ---------------------------------------------------------------- codec (J/Quant.java)

def test_quant_main_known_answer(orc):
    # Input of the reference's own self-check Quant.main (J/Quant.java:69-77): d[i] = i, i < 100.
    enc = orc.quant_encode(np.arange(100, dtype=np.float32))
    assert enc.size == 264
    assert bytes(enc[:8]).hex() == "0000000042c60000"  # big-endian 0.0f, 99.0f
    assert list(enc[8:18]) == [0, 3, 5, 8, 10, 13, 15, 18, 21, 23]
    assert enc[8 + 50] == 129 and enc[8 + 98] == 252 and enc[8 + 99] == 255
    assert not enc[8 + 100:].any()  # filler
    # independent integer derivation: round-half-up of i/99*255
    want = [int(math.floor(i / 99.0 * 255.0 + 0.5)) for i in range(100)]
    assert list(enc[8:108]) == want


def test_quant_sizes(orc):
    for n, b in [(1, 264), (256, 264), (257, 528), (288 * 288, 324 * 264), (4096 * 4096, 65536 * 264)]:
        assert orc.quant_nbytes(n) == b


def test_quant_constant_group_and_nan_rule(orc):
    # range == 0 -> 0/0 = NaN -> Math.round gives 0 -> all-zero payload, decodes to min
    enc = orc.quant_encode(np.full(300, 0.25, dtype=np.float32))
    assert not enc[8:264].any() and not enc[264 + 8:].any()
    np.testing.assert_array_equal(orc.quant_decode(enc, 0, 300), np.full(300, 0.25, np.float32))


def test_quant_round_half_up_is_exact(orc):
    # A value whose scaled code is just below .5 must not be rounded up by a float add of 0.5.
    # group = [0, 255, v]: (v-0)/255*255 ~ v; v = 0.49999997 (largest float below 0.5) -> code 0
    v = np.nextafter(np.float32(0.5), np.float32(0))
    enc = orc.quant_encode(np.array([0, 255, v, 0.5, 1.5, 2.5], dtype=np.float32))
    assert list(enc[8:14]) == [0, 255, 0, 1, 2, 3]  # ties go up (2.5 -> 3), not to even


def test_quant_error_bound_idempotence_and_acceptance_rule(orc):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(5000) * 0.02).astype(np.float32)
    enc = orc.quant_encode(x)
    dec = orc.quant_decode(enc, 0, x.size)
    mn, mx, codes = np_ref.parse_quant(enc)
    rng_per = np.repeat(mx - mn, 256)[:x.size].astype(np.float64)
    assert np.all(np.abs(dec.astype(np.float64) - x) <= rng_per / 510.0 * (1 + 1e-4) + 1e-9)
    # min and max of every group are reproduced exactly by code 0 and code 255
    for g in range(mn.size):
        seg = x[g * 256:(g + 1) * 256]
        assert mn[g] == seg.min() and mx[g] == seg.max()
    # encode(decode(encode(x))) keeps every code; the header max may move by an ulp (min + range rounds)
    mn2, mx2, codes2 = np_ref.parse_quant(orc.quant_encode(dec))
    np.testing.assert_array_equal(codes2, codes)
    np.testing.assert_array_equal(mn2, mn)
    np.testing.assert_allclose(mx2, mx, rtol=2e-7)
    # the reference's own acceptance rule (J/Quant.java:119-120,147) on random slices
    diff = np.abs(dec - x)
    assert not np.any((diff / np.abs(x) > 0.01) & (diff > 1e-2))
    # slices decode to the same values as the whole
    for s, n in [(0, 1), (255, 2), (256, 256), (300, 1000), (4999, 1)]:
        np.testing.assert_array_equal(orc.quant_decode(enc, s, n), dec[s:s + n])
    # independent parser agrees with the two dequant forms to float64 accuracy
    np.testing.assert_allclose(dec, np_ref.dequant64(enc, x.size), rtol=0, atol=3e-8)


# ---------------------------------------------------------------- matvec (K/MatMul.java)

@pytest.mark.parametrize("n,d,widx", [(256, 7, 0), (512, 5, 256 * 3), (288, 6, 288 * 288), (48, 9, 32),
                                        (1, 5, 17), (768, 4, 0), (300, 3, 13)])
def test_matmul_i8_vs_float64(orc, n, d, widx):
    rng = np.random.default_rng(n * 31 + d)
    total = widx + n * d + 37
    w = (rng.standard_normal(total) * 0.02).astype(np.float32)
    enc = orc.quant_encode(w)
    x = rng.standard_normal(n).astype(np.float32)
    got = orc.matmul_i8(x, enc, widx, n, d)
    W = np_ref.dequant64(enc, total)[widx:widx + n * d].reshape(d, n)
    want = W @ x.astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-5 * np.abs(W).sum(axis=1).max() * np.abs(x).max())
    # the literal per-element walk handles every case and must agree bit for bit where both apply
    np.testing.assert_array_equal(got, orc.matmul_i8(x, enc, widx, n, d, "_unaligned"))


def test_matmul_i8_aligned_fast_path_bit_equal_to_literal_walk(orc):
    rng = np.random.default_rng(5)
    n, d, widx = 1024, 37, 256 * 11
    w = (rng.standard_normal(widx + n * d) * 0.02).astype(np.float32)
    enc = orc.quant_encode(w)
    x = rng.standard_normal(n).astype(np.float32)
    a = orc.matmul_i8(x, enc, widx, n, d, "_aligned")
    b = orc.matmul_i8(x, enc, widx, n, d, "_unaligned")
    np.testing.assert_array_equal(a, b)
    # sequential fp32 order, no FMA: reproduce one row with numpy float32 scalar ops
    mn, mx, codes = np_ref.parse_quant(enc)
    row = 5
    val = np.float32(0)
    for j in range(n):
        f = widx + row * n + j
        g = f // 256
        rm = np.float32(np.float32(mx[g] - mn[g]) / np.float32(255))
        wv = np.float32(np.float32(np.float32(codes[g, f % 256]) * rm) + mn[g])
        val = np.float32(val + np.float32(wv * x[j]))
    assert a[row] == val


def test_matmul_f32(orc):
    rng = np.random.default_rng(9)
    n, d = 96, 33
    w = rng.standard_normal(n * d + 5).astype(np.float32)
    x = rng.standard_normal(n).astype(np.float32)
    got = orc.matmul_f32(x, w, 5, n, d)
    want = w[5:].reshape(d, n).astype(np.float64) @ x
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)
    v = np.float32(0)
    for j in range(n):
        v = np.float32(v + np.float32(w[5 + 2 * n + j] * x[j]))
    assert got[2] == v


# ---------------------------------------------------------------- rmsnorm (K/RootMeanSquare, K/WeightNormalizeAndScale)

def test_rms_closed_form_and_wns(orc):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(288).astype(np.float32)
    ss = orc.rms(x)
    assert abs(ss[0] - 1.0 / math.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5)) < 2e-6
    assert orc.rms(np.zeros(16, np.float32))[0] == np.float32(1.0) / np.float32(math.sqrt(np.float32(1e-5)))
    # all-ones weight (constant group decodes exactly to 1) -> plain RMSNorm
    enc1 = orc.quant_encode(np.ones(1000, np.float32))
    out = orc.wns_i8(x, enc1, 300, ss)
    np.testing.assert_array_equal(out, np.float32(1) * (ss[0] * x))
    # general weights at an offset that straddles groups; uses the (c/255)*range+min form
    w = (rng.standard_normal(1000) * 0.02 + 1).astype(np.float32)
    enc = orc.quant_encode(w)
    out = orc.wns_i8(x, enc, 300, ss)
    want = np_ref.dequant64(enc, 1000)[300:588] * (float(ss[0]) * x.astype(np.float64))
    np.testing.assert_allclose(out, want, rtol=3e-7, atol=0)
    dec = orc.quant_decode(enc, 300, 288)
    np.testing.assert_array_equal(out, dec * (ss[0] * x))  # same dequant expression as Quant.decode


# ---------------------------------------------------------------- RoPE (K/ApplyRope.java)

def test_rope(orc):
    dim, hs, seq = 96, 48, 16
    c, s = orc.rope_table(dim, hs, seq)
    assert c.size == dim // 2 * seq
    # freq constants: hs=128, i=2 -> 10000^(-2/128)
    c128, s128 = orc.rope_table(128, 128, 2)
    assert abs(math.cos(0.86596435) - c128[64 + 1]) < 1e-7 and abs(math.sin(0.86596435) - s128[64 + 1]) < 1e-7
    assert np.all(c[:dim // 2] == 1) and np.all(s[:dim // 2] == 0)  # pos 0: identity
    rng = np.random.default_rng(3)
    q0 = rng.standard_normal(dim).astype(np.float32)
    k0 = rng.standard_normal(dim).astype(np.float32)
    q, k = q0.copy(), k0.copy()
    orc.rope(q, k, c, s, 0, dim, dim)
    np.testing.assert_array_equal(q, q0)
    np.testing.assert_array_equal(k, k0)
    # pair norms preserved and equality with complex rotation
    pos = 7
    q, k = q0.copy(), k0.copy()
    orc.rope(q, k, c, s, pos, dim, dim)
    i = np.arange(0, dim, 2)
    ang = pos * 10000.0 ** (-((i % hs) / hs))
    want = (q0[0::2] + 1j * q0[1::2]) * np.exp(1j * ang)
    np.testing.assert_allclose(q[0::2], want.real, atol=2e-6)
    np.testing.assert_allclose(q[1::2], want.imag, atol=2e-6)
    np.testing.assert_allclose(q[0::2] ** 2 + q[1::2] ** 2, q0[0::2] ** 2 + q0[1::2] ** 2, rtol=1e-5)
    # relative-position property: <R_p q, R_p' k> depends only on p - p'
    def dot_at(p, pp):
        a, b = q0.copy(), k0.copy()
        dummy = k0.copy()
        orc.rope(a, dummy, c, s, p, dim, dim)
        dummy = q0.copy()
        orc.rope(dummy, b, c, s, pp, dim, dim)
        return float(a[:hs].astype(np.float64) @ b[:hs])
    assert abs(dot_at(9, 4) - dot_at(12, 7)) < 1e-4
    assert abs(dot_at(9, 4) - dot_at(9, 5)) > 1e-3
    # kv_dim < dim rotates only the first kv_dim entries of k
    q, k = q0.copy(), k0.copy()
    orc.rope(q, k, c, s, pos, dim, 48)
    np.testing.assert_array_equal(k[48:], k0[48:])
    assert not np.array_equal(k[:48], k0[:48])


# ---------------------------------------------------------------- attention (K/AttentionLoop, K/ExpSumNormalize, K/AccumWeightedValue)

def _attention(orc, q, K, V, tmp1, h, seq_len, kv_dim, hs, pos, kv_mul=1):
    L = orc.lib()
    att = np.zeros(8 * seq_len, np.float32)
    xb = np.full(q.size, 7.0, np.float32)
    base = (h // kv_mul) * hs
    L.orc_attention_loop(orc._fp(q), orc._fp(K), orc._fp(att), orc._fp(tmp1), h, h * seq_len, base, kv_dim,
                         h * hs, pos, hs)
    scores = att[h * seq_len:h * seq_len + pos + 1].copy()
    L.orc_exp_sum_normalize(orc._fp(att), orc._fp(tmp1), h, h * seq_len, pos + 1)
    L.orc_accum_weighted_value(orc._fp(xb), orc._fp(att), orc._fp(V), pos, h * hs, base, hs, kv_dim, h * seq_len)
    return scores, att[h * seq_len:h * seq_len + pos + 1].copy(), xb


@pytest.mark.parametrize("hs", [48, 64, 128, 6])
def test_attention_vs_textbook(orc, hs):
    rng = np.random.default_rng(hs)
    H, seq_len, pos = 3, 32, 20
    dim = H * hs
    q = rng.standard_normal(dim).astype(np.float32)
    K = rng.standard_normal(seq_len * dim).astype(np.float32)
    V = rng.standard_normal(seq_len * dim).astype(np.float32)
    tmp1 = np.zeros(64, np.float32)
    tmp1[0] = 30.0  # head 0's slot also holds 1/rms(x) in the forward pass
    for h in range(H):
        scores, p, xb = _attention(orc, q, K, V, tmp1, h, seq_len, dim, hs, pos)
        Kh = K.reshape(seq_len, dim)[:pos + 1, h * hs:(h + 1) * hs].astype(np.float64)
        Vh = V.reshape(seq_len, dim)[:pos + 1, h * hs:(h + 1) * hs].astype(np.float64)
        s = Kh @ q[h * hs:(h + 1) * hs].astype(np.float64) / math.sqrt(hs)
        np.testing.assert_allclose(scores, s, atol=3e-5 * max(1, hs ** 0.5))
        pw = np.exp(s - s.max())
        pw /= pw.sum()
        np.testing.assert_allclose(p, pw, rtol=2e-4, atol=1e-7)  # shift quirk only costs ulps of the shift
        assert abs(p.sum() - 1) < 1e-5
        np.testing.assert_allclose(xb[h * hs:(h + 1) * hs], pw @ Vh, atol=1e-4)
        # other heads' slots untouched
        mask = np.ones(dim, bool)
        mask[h * hs:(h + 1) * hs] = False
        assert np.all(xb[mask] == 7.0)
        # side effect: running max over element-wise products, never below the previous slot value
        prod_max = (Kh * q[h * hs:(h + 1) * hs]).max()
        assert tmp1[h] == np.float32(max(30.0 if h == 0 else 0.0, prod_max))


def test_attention_pos0_is_exact_copy_of_v(orc):
    rng = np.random.default_rng(11)
    hs, H, seq_len = 64, 2, 8
    dim = hs * H
    q = rng.standard_normal(dim).astype(np.float32)
    K = rng.standard_normal(seq_len * dim).astype(np.float32)
    V = rng.standard_normal(seq_len * dim).astype(np.float32)
    tmp1 = np.zeros(8, np.float32)
    for h in range(H):
        _, p, xb = _attention(orc, q, K, V, tmp1, h, seq_len, dim, hs, 0)
        assert p[0] == 1.0
        np.testing.assert_array_equal(xb[h * hs:(h + 1) * hs], V[h * hs:(h + 1) * hs])


def test_softmax_skips_normalisation_when_sum_is_zero(orc):
    x = np.array([0.0, 1.0, 2.0, 0, 0], np.float32)
    mx = np.array([500.0], np.float32)  # exp underflows to 0 for every entry
    orc.lib().orc_exp_sum_normalize(orc._fp(x), orc._fp(mx), 0, 0, 3)
    assert np.all(x[:3] == 0)


def test_multiquery_key_base(orc):
    # kv_mul = 2: heads 0,1 share kv head 0; heads 2,3 share kv head 1
    rng = np.random.default_rng(13)
    hs, H, kvh, seq_len, pos = 16, 4, 2, 8, 5
    dim, kv_dim = hs * H, hs * kvh
    q = rng.standard_normal(dim).astype(np.float32)
    K = rng.standard_normal(seq_len * kv_dim).astype(np.float32)
    V = rng.standard_normal(seq_len * kv_dim).astype(np.float32)
    tmp1 = np.zeros(8, np.float32)
    for h in range(H):
        scores, p, xb = _attention(orc, q, K, V, tmp1, h, seq_len, kv_dim, hs, pos, kv_mul=2)
        kh = (h // 2) * hs
        Kh = K.reshape(seq_len, kv_dim)[:pos + 1, kh:kh + hs].astype(np.float64)
        np.testing.assert_allclose(scores, Kh @ q[h * hs:(h + 1) * hs].astype(np.float64) / 4.0, atol=1e-5)


# ---------------------------------------------------------------- SiLU LUT (K/Silu.java), residual, argmax

def test_silu_lut_known_values_and_bound(orc):
    t = orc.silu_table()
    assert t[4096] == np.float32(0.5)
    assert abs(t[4095] - 0.49969482) < 1e-7
    # the integer multiplier 819 (not 819.2) puts val = 0 at position 4095.0 exactly
    assert abs(orc.silu_lookup(t, 0.0) - 0.49969482) < 1e-7
    assert abs(orc.silu_lookup(t, 1.0) - 0.73077047) < 1e-6
    assert abs(orc.silu_lookup(t, -1.0) - 0.26874948) < 1e-6
    assert abs(orc.silu_lookup(t, -5.0) - 0.00669285) < 1e-8  # position 0 -> exact branch
    assert orc.silu_lookup(t, 7.0) == np.float32(1.0 / (1.0 + math.exp(-7.0)))
    vs = np.linspace(-4.99, 4.99, 4001)
    got = np.array([orc.silu_lookup(t, float(np.float32(v))) for v in vs])
    exact = np_ref.sigmoid64(vs.astype(np.float32))
    rel = np.abs(got - exact) / exact
    assert rel.max() < 7.3e-4 and rel.max() > 3e-4  # the systematic error is really there
    np.testing.assert_allclose(got, np_ref.silu_lut64(vs.astype(np.float32)), rtol=3e-7)
    hb = np.array([0.3, -2.0, 6.0], np.float32)
    hb2 = np.array([1.5, 0.5, -1.0], np.float32)
    h = hb.copy()
    orc.silu(h, hb2, t)
    for i in range(3):
        assert h[i] == np.float32(hb[i] * np.float32(np.float32(orc.silu_lookup(t, float(hb[i]))) * hb2[i]))


def test_accum_and_argmax(orc):
    a = np.array([1, 2, 3], np.float32)
    b = np.array([0.5, -2, 1e-8], np.float32)
    orc.lib().orc_accum(orc._fp(a), orc._fp(b), 3)
    np.testing.assert_array_equal(a, np.array([1.5, 0, 3], np.float32))
    assert orc.argmax(np.array([1, 5, 5, 2], np.float32)) == 1  # first of equal maxima
    assert orc.argmax(np.array([3, 1], np.float32)) == 0
    assert orc.argmax(np.array([-1, -1, -0.5], np.float32)) == 2


# ---------------------------------------------------------------- synthetic generator

def test_synth_statistics_and_determinism(orc):
    a = orc.synth_fill(7, 3, 0, 200000)
    assert abs(a.mean()) < 2e-4 and abs(a.std() - 0.02) < 2e-4
    b = orc.synth_fill(7, 3, 1000, 50)
    np.testing.assert_array_equal(a[1000:1050], b)  # counter based: any slice, any thread count
    assert not np.array_equal(orc.synth_fill(7, 4, 0, 50), a[:50])
    assert not np.array_equal(orc.synth_fill(8, 3, 0, 50), a[:50])
    # independent restatement of the stated formula in python integers
    M = (1 << 64) - 1
    def sm(z):
        z = (z + 0x9E3779B97F4A7C15) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)
    base = (7 * 0x9E3779B97F4A7C15 + 3 * 0xD1B54A32D192ED03) & M
    scale = np.float32(0.02) / np.float32(37837.2265625)
    for i in (0, 1, 12345):
        r = sm((base + i) & M)
        s = (r & 0xFFFF) + ((r >> 16) & 0xFFFF) + ((r >> 32) & 0xFFFF) + (r >> 48) - 131070
        assert a[i] == np.float32(np.float32(s) * scale)
    p = orc.synth_prompt(5, 64, 32000)
    assert p.min() >= 3 and p.max() < 32000 and len(set(p.tolist())) > 50
