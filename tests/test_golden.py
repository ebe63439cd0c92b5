"""Committed fixtures (tests/golden/, written by make_fixtures.py): a tiny checkpoint with its .quant caches and the
expected logits / greedy tokens.  CPU: the oracle reproduces them from the files, and an independent numpy reader of
the two file formats agrees with the caches.  GPU: the library loads the same files and matches."""
import os
import shutil
import struct

import numpy as np
import pytest

from tests import np_ref

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
STEMS = ["l_rms_att_weight", "l_wq", "l_wk", "l_wv", "l_wo", "l_rms_ffn_weight", "l_w1", "l_w2", "l_w3", "rms_final_weight"]


def read_bin_independently(path):
    raw = open(path, "rb").read()
    dim, hidden, L, H, kvH, vocab, seq = struct.unpack("<7i", raw[:28])
    shared = vocab > 0
    vocab = abs(vocab)
    kvd = dim * kvH // H
    sizes = [vocab * dim, L * dim, L * dim * dim, L * dim * kvd, L * dim * kvd, L * dim * dim, L * dim, L * dim * hidden,
             L * hidden * dim, L * dim * hidden, dim]
    off, out = 28, []
    for n in sizes:
        out.append(np.frombuffer(raw, "<f4", n, off))
        off += 4 * n
    off += 4 * seq * (dim // H)
    wcls = out[0] if shared else np.frombuffer(raw, "<f4", vocab * dim, off)
    return (dim, hidden, L, H, kvH, vocab, seq, shared), out[0], out[1:], wcls


def test_fixture_files_and_oracle(orc, tmp_path):
    cfg, emb, tens, wcls = read_bin_independently(os.path.join(G, "tiny.bin"))
    assert cfg[:7] == (32, 48, 2, 4, 2, 40, 12) and not cfg[7]
    for t, stem in enumerate(STEMS):
        raw = open(os.path.join(G, "tiny_%s_256_8.quant" % stem), "rb").read()
        assert struct.unpack("<i", raw[:4])[0] == len(raw) - 4 == -(-tens[t].size // 256) * 264
        enc = np.frombuffer(raw[4:], np.uint8)
        # the cache decodes (independent parser, float64) to the fp32 tensor within half a quantization step
        mn, mx, _ = np_ref.parse_quant(enc)
        step = np.repeat((mx - mn).astype(np.float64) / 255.0, 256)[:tens[t].size]
        assert np.all(np.abs(np_ref.dequant64(enc, tens[t].size) - tens[t]) <= step / 2 * (1 + 1e-4) + 1e-9)
    exp = np.load(os.path.join(G, "expected.npz"))
    for f in os.listdir(G):  # load from a copy so nothing is written into the fixtures
        if f.startswith("tiny"):
            shutil.copy(os.path.join(G, f), tmp_path / f)
    m = orc.Model.load(str(tmp_path / "tiny.bin"), write_caches=False)
    toks, logits, _ = m.generate_greedy(exp["prompt"], 12, want_logits=True)
    np.testing.assert_array_equal(toks, exp["tokens"])
    np.testing.assert_array_equal(logits, exp["logits"])
    # and the textbook float64 decoder on the dequantized caches agrees with the committed logits
    names = ["rms_att", "wq", "wk", "wv", "wo", "rms_ffn", "w1", "w2", "w3", "rms_final"]
    tb = np_ref.TextbookLlama(dict(dim=32, hidden_dim=48, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=40, seq_len=12),
                              {names[t]: np_ref.dequant64(m.quant(t), tens[t].size) for t in range(10)}, emb, wcls)
    tok = 1
    for pos in range(len(toks)):
        want = tb.forward(tok, pos)
        assert np.abs(exp["logits"][pos] - want).max() / np.abs(want).max() < 2e-5
        tok = int(exp["tokens"][pos])


@pytest.mark.gpu
def test_library_on_fixture_checkpoint(tmp_path):
    import llama2j_amd as l2j
    for f in os.listdir(G):
        if f.startswith("tiny"):
            shutil.copy(os.path.join(G, f), tmp_path / f)
    exp = np.load(os.path.join(G, "expected.npz"))
    g = l2j.Transformer.from_checkpoint(str(tmp_path / "tiny.bin"), write_caches=False)   # cache branch
    toks, _ = g.decode_greedy(exp["prompt"], 12)
    np.testing.assert_array_equal(toks, exp["tokens"])
    g.reset()
    tok = 1
    for pos in range(len(toks)):
        lg = g.forward(tok, pos)
        assert np.abs(lg - exp["logits"][pos]).max() / np.abs(exp["logits"][pos]).max() < 1e-3
        tok = int(toks[pos])
    # without the caches the GPU encoder must reproduce the committed .quant bytes exactly
    for f in os.listdir(tmp_path):
        if f.endswith(".quant"):
            os.remove(tmp_path / f)
    g2 = l2j.Transformer.from_checkpoint(str(tmp_path / "tiny.bin"), write_caches=True)
    for stem in STEMS:
        name = "tiny_%s_256_8.quant" % stem
        assert open(tmp_path / name, "rb").read() == open(os.path.join(G, name), "rb").read()
    np.testing.assert_array_equal(g2.decode_greedy(exp["prompt"], 12)[0], exp["tokens"])
