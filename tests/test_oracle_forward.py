"""Pins the oracle's whole forward pass, token loop and file formats against an independent float64
textbook Llama-2 decoder (tests/np_ref.py) and byte-level format readers written here."""
import os
import struct

import numpy as np
import pytest

from tests import np_ref

NAMES = ["rms_att", "wq", "wk", "wv", "wo", "rms_ffn", "w1", "w2", "w3", "rms_final"]


def make_model(orc, dim, hidden, L, H, kvH, vocab, seq, shared, seed):
    m = orc.Model(dim=dim, hidden_dim=hidden, n_layers=L, n_heads=H, n_kv_heads=kvH, vocab_size=vocab,
                  seq_len=seq, shared_weights=shared)
    m.fill_synth(seed, 0.02)
    # rms weights ~ N(0, 0.02) would make activations tiny; exercise realistic magnitudes too
    rng = np.random.default_rng(seed)
    for t in (orc.T_RMS_ATT, orc.T_RMS_FFN, orc.T_RMS_FINAL):
        n = m.tensor_floats(t)
        m.set_quant(t, orc.quant_encode((1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)))
    # matrices with a larger spread so attention is not uniform
    for t in (orc.T_WQ, orc.T_WK):
        n = m.tensor_floats(t)
        m.set_quant(t, orc.quant_encode((0.15 * rng.standard_normal(n)).astype(np.float32)))
    return m


def textbook_of(orc, m, sigmoid):
    c = m.cfg
    cfg = dict(dim=c.dim, hidden_dim=c.hidden_dim, n_layers=c.n_layers, n_heads=c.n_heads,
               n_kv_heads=c.n_kv_heads, vocab_size=c.vocab_size, seq_len=c.seq_len)
    tensors = {NAMES[t]: np_ref.dequant64(m.quant(t), m.tensor_floats(t)) for t in range(10)}
    return np_ref.TextbookLlama(cfg, tensors, m.emb(), m.wcls(), sigmoid=sigmoid)


SHAPES = [
    # dim hidden L H kvH vocab seq shared   (aligned / unaligned-to-256 / multiquery / head 48)
    (64, 256, 2, 4, 4, 50, 12, 1),
    (96, 160, 2, 2, 2, 40, 10, 0),      # head_size 48, rows straddle groups, layer offsets unaligned
    (32, 48, 3, 4, 2, 30, 8, 1),        # n_kv_heads < n_heads
    (256, 512, 1, 2, 2, 64, 6, 0),      # fully 256-aligned (takes the aligned matvec path)
]


@pytest.mark.parametrize("shape", SHAPES)
def test_forward_vs_textbook_every_pos(orc, shape):
    m = make_model(orc, *shape, seed=3)
    tb = textbook_of(orc, m, np_ref.silu_lut64)
    tb_exact = textbook_of(orc, m, np_ref.sigmoid64)
    rng = np.random.default_rng(0)
    toks = rng.integers(0, shape[5], size=shape[6])
    worst_exact = 0.0
    for pos, tok in enumerate(toks):
        got = m.forward(int(tok), pos).astype(np.float64)
        want = tb.forward(int(tok), pos)
        scale = np.abs(want).max()
        assert np.abs(got - want).max() / scale < 2e-5, (pos, np.abs(got - want).max() / scale)
        we = tb_exact.forward(int(tok), pos)
        worst_exact = max(worst_exact, np.abs(got - we).max() / np.abs(we).max())
        # KV cache row written at (l, pos)
        L, S, kvd = shape[2], shape[6], m.kv_dim
        kc = m.buffer(orc.B_KCACHE).reshape(L, S, kvd)
        np.testing.assert_allclose(kc[:, pos], tb.K[:, pos], atol=2e-5 * max(1.0, np.abs(tb.K[:, pos]).max()))
        assert not kc[:, pos + 1:].any()
    # the LUT's systematic sigmoid error is visible but small against an exact-sigmoid decoder
    assert worst_exact < 2e-3


def test_forward_pos0_attention_is_copy_of_v(orc):
    m = make_model(orc, 64, 256, 2, 4, 4, 50, 12, 1, seed=4)
    m.forward_layers(7, 0, 1)  # stops after layer 0; xb then holds the W2 output, so tap before: rerun ops
    # xb after attention is overwritten later in the layer, so check through the cache instead:
    # with one timestep softmax is exactly 1.0 and attention output == v (value_cache row 0), which makes
    # layer 0's residual x = emb + Wo v.  Recompute that with the oracle's own matvec and compare bits.
    v = m.buffer(orc.B_VCACHE)[:64].copy()
    wo_v = orc.matmul_i8(v, m.quant(orc.T_WO), 0, 64, 64)
    np.testing.assert_array_equal(m.buffer(orc.B_XB2), wo_v)


def test_tmp1_quirk_state(orc):
    # tmp1[0] is the last 1/rms; tmp1[h>=1] only ever grows (never reset across layers or tokens)
    m = make_model(orc, 64, 256, 2, 4, 4, 50, 12, 1, seed=5)
    prev = np.zeros(4)
    for pos in range(5):
        m.forward(3 + pos, pos)
        t = m.buffer(orc.B_TMP1)[:4].copy()
        assert np.all(t[1:] >= prev[1:])
        prev = t
    x = m.buffer(orc.B_X)  # holds the final-normed x (in place, J/Run.java:165)
    assert t[0] > 0


def test_generate_loop_semantics(orc):
    m = make_model(orc, 64, 256, 2, 4, 4, 50, 12, 1, seed=6)
    prompt = np.array([5, 9, 11], np.int32)
    out, logits, sec = m.generate_greedy(prompt, 8, want_logits=True)
    assert list(out[:3]) == [5, 9, 11]  # prompt ids are forced as outputs of pos 0..2
    # replay by hand: BOS first, then feed `next`
    m.reset()
    tok = 1
    for pos in range(len(out)):
        lg = m.forward(tok, pos)
        np.testing.assert_array_equal(lg, logits[pos])
        nxt = int(prompt[pos]) if pos < 3 else int(np.argmax(lg))  # np.argmax is also first-max
        assert nxt == out[pos]
        tok = nxt
    # stop rule: a forced 1 ends the loop right after it is emitted
    m.reset()
    out2, _, _ = m.generate_greedy(np.array([5, 1, 7], np.int32), 8)
    assert list(out2) == [5, 1]
    # steps <= 0 or > seq_len clamps to seq_len
    m.reset()
    out3, _, _ = m.generate_greedy(prompt, 0)
    assert len(out3) <= 12 and (len(out3) == 12 or out3[-1] == 1)


def write_bin(path, cfg, emb, tensors_f32, wcls=None):
    """llama2.c v0 checkpoint: 7 LE int32, fp32 tensors in file order, freq_cis, optional classifier."""
    dim, hidden, L, H, kvH, vocab, seq = cfg
    with open(path, "wb") as f:
        f.write(struct.pack("<7i", dim, hidden, L, H, kvH, vocab if wcls is None else -vocab, seq))
        f.write(np.asarray(emb, "<f4").tobytes())
        for t in tensors_f32:
            f.write(np.asarray(t, "<f4").tobytes())
        hs = dim // H
        f.write(np.zeros(seq * hs // 2 * 2, "<f4").tobytes())
        if wcls is not None:
            f.write(np.asarray(wcls, "<f4").tobytes())


@pytest.mark.parametrize("shared", [1, 0])
def test_checkpoint_and_quant_cache_files(orc, tmp_path, shared):
    cfg = (32, 48, 2, 4, 2, 30, 8)
    dim, hidden, L, H, kvH, vocab, seq = cfg
    rng = np.random.default_rng(8)
    kvd = dim * kvH // H
    sizes = [L * dim, L * dim * dim, L * dim * kvd, L * dim * kvd, L * dim * dim, L * dim, L * dim * hidden,
             L * hidden * dim, L * dim * hidden, dim]
    tens = [(rng.standard_normal(n) * 0.05).astype(np.float32) for n in sizes]
    emb = (rng.standard_normal(vocab * dim) * 0.05).astype(np.float32)
    wcls = None if shared else (rng.standard_normal(vocab * dim) * 0.05).astype(np.float32)
    path = str(tmp_path / "tiny.bin")
    write_bin(path, cfg, emb, tens, wcls)
    m = orc.Model.load(path, write_caches=True)
    assert m.cfg.shared_weights == shared and m.cfg.vocab_size == vocab
    np.testing.assert_array_equal(m.emb(), emb)
    np.testing.assert_array_equal(m.wcls(), emb if shared else wcls)
    stems = ["l_rms_att_weight", "l_wq", "l_wk", "l_wv", "l_wo", "l_rms_ffn_weight", "l_w1", "l_w2", "l_w3",
             "rms_final_weight"]
    for t, stem in enumerate(stems):
        qp = tmp_path / ("tiny_%s_256_8.quant" % stem)  # J/TransformerWeights.java:194, J/Quant.java:195-197
        raw = qp.read_bytes()
        (n,) = struct.unpack("<i", raw[:4])  # LE int32 byte count, J/BinFileWriter.java:26-32
        assert n == len(raw) - 4 == -(-sizes[t] // 256) * 264
        np.testing.assert_array_equal(np.frombuffer(raw[4:], np.uint8), m.quant(t))
        np.testing.assert_array_equal(m.quant(t), orc.quant_encode(tens[t]))
    lg1 = m.forward(3, 0).copy()
    # second load takes the cache branch (floats skipped); poison the fp32 tensors to prove it
    write_bin(path, cfg, emb, [np.zeros_like(t) for t in tens], wcls)
    m2 = orc.Model.load(path, write_caches=False)
    np.testing.assert_array_equal(m2.forward(3, 0), lg1)
    # wrong-size cache is rejected (J/TransformerWeights.java:228-232)
    bad = tmp_path / "tiny_l_wq_256_8.quant"
    bad.write_bytes(struct.pack("<i", 264) + bytes(264))
    with pytest.raises(RuntimeError):
        orc.Model.load(path, write_caches=False)
