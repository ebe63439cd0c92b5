"""CPU-side tests of libllama2j_hip.so: the C ABI loads and exports every declared symbol, the host
codec and file formats agree bit for bit with the oracle, and error paths return codes (never abort).
No compute call needs a GPU here."""
import ctypes as C
import os
import re
import struct

import numpy as np
import pytest

import llama2j_amd as l2j
from llama2j_amd import binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "llama2j_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(l2j_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 28
    L = C.CDLL(l2j.lib_path())
    for name in declared:
        assert hasattr(L, name), name
    assert declared == set(B._signatures().keys())  # the python binding covers the whole ABI


def test_host_codec_matches_oracle_bit_for_bit(orc):
    q = l2j.Quant(256, 8)
    rng = np.random.default_rng(0)
    for n in (1, 100, 256, 257, 5000, 288 * 288, 300000):
        x = (rng.standard_normal(n) * 0.02).astype(np.float32)
        enc = q.encode(x)
        np.testing.assert_array_equal(enc, orc.quant_encode(x))
        assert q.numberOfBytesByFloatSize(n) == orc.quant_nbytes(n) == enc.size
        for s, m in [(0, n), (n // 3, n - n // 3), (n - 1, 1)]:
            np.testing.assert_array_equal(q.decode(enc, s, m), orc.quant_decode(enc, s, m))
    # the reference's own self-check input (J/Quant.java:69-77) and the special cases
    enc = q.encode(np.arange(100, dtype=np.float32))
    assert bytes(enc[:8]).hex() == "0000000042c60000" and list(enc[8:12]) == [0, 3, 5, 8] and enc[8 + 99] == 255
    assert not q.encode(np.full(10, 3.0, np.float32))[8:].any()
    v = np.nextafter(np.float32(0.5), np.float32(0))
    assert list(q.encode(np.array([0, 255, v, 0.5, 2.5], np.float32))[8:13]) == [0, 255, 0, 1, 3]
    assert q.extension() == "_256_8.quant" and q.encodedBytesPerGroup() == 264
    with pytest.raises(ValueError):
        l2j.Quant(128, 8)


def test_quant_cache_files(orc, tmp_path):
    q = l2j.Quant()
    x = (np.random.default_rng(1).standard_normal(1000) * 0.02).astype(np.float32)
    enc = q.encode(x)
    p = str(tmp_path / "m_l_wq_256_8.quant")
    q.write_file(p, enc)
    raw = open(p, "rb").read()
    assert struct.unpack("<i", raw[:4])[0] == enc.size and raw[4:] == enc.tobytes()
    np.testing.assert_array_equal(q.read_file(p, enc.size), enc)
    # the oracle's reader and writer produce / accept the same file
    buf = np.empty(enc.size, np.uint8)
    assert orc.lib().orc_read_quant_file(p.encode(), orc._u8(buf), buf.size) == enc.size
    np.testing.assert_array_equal(buf, enc)
    p2 = str(tmp_path / "o.quant")
    assert orc.lib().orc_write_quant_file(p2.encode(), orc._u8(enc), enc.size) == 0
    assert open(p2, "rb").read() == raw
    with pytest.raises(l2j.L2JError) as e:
        q.read_file(p, enc.size - 264)  # larger than expected -> size error
    assert e.value.code == -2
    with pytest.raises(l2j.L2JError) as e:
        q.read_file(str(tmp_path / "absent.quant"), 10)
    assert e.value.code == -6
    # file name rule (J/TransformerWeights.java:194)
    assert q.cache_path("models/stories15M.bin", l2j.TENSOR.WQ) == "models/stories15M_l_wq_256_8.quant"
    assert q.cache_path("x.y.bin", l2j.TENSOR.RMS_FINAL) == "./x.y_rms_final_weight_256_8.quant"
    with pytest.raises(l2j.L2JError):
        q.cache_path("a.bin", l2j.TENSOR.TOK_EMB)


def test_checkpoint_header(tmp_path):
    p = str(tmp_path / "h.bin")
    open(p, "wb").write(struct.pack("<7i", 288, 768, 6, 6, 6, -32000, 256))
    cfg = l2j.Config()
    assert l2j.lib().l2j_read_checkpoint_header(p.encode(), C.byref(cfg)) == 0
    assert (cfg.dim, cfg.hidden_dim, cfg.n_layers, cfg.n_heads, cfg.n_kv_heads, cfg.vocab_size, cfg.seq_len) == \
        (288, 768, 6, 6, 6, 32000, 256)
    assert cfg.shared_weights == 0 and cfg.group_size == 256 and cfg.bits == 8
    open(p, "wb").write(b"short")
    assert l2j.lib().l2j_read_checkpoint_header(p.encode(), C.byref(cfg)) == -6


def test_bytes_per_token_matches_published_denominators():
    # weights per token in the reference's storage format (int8 + min/max, fp32 classifier and embedding row)
    c7 = l2j.Config(4096, 11008, 32, 32, 32, 32000, 4096, 0)
    w = l2j.lib().l2j_bytes_per_token(C.byref(c7), -1)  # pos = -1: no KV read
    assert w == 6678655104 + 524288000 + 4096 * 4 + 2 * 32 * 4096 * 4
    c15 = l2j.Config(288, 768, 6, 6, 6, 32000, 256, 1)
    assert l2j.lib().l2j_bytes_per_token(C.byref(c15), -1) == 6162816 + 36864000 + 288 * 4 + 2 * 6 * 288 * 4
    kv = l2j.lib().l2j_bytes_per_token(C.byref(c7), 3839) - w
    assert kv == 2 * 32 * 3840 * 4096 * 4


def test_error_paths_without_gpu():
    L = l2j.lib()
    if L.l2j_device_count() > 0:
        pytest.skip("a GPU is present; the no-device path is covered on CPU boxes")
    with pytest.raises(l2j.L2JError) as e:
        l2j.Transformer(l2j.Config(64, 256, 2, 4, 4, 50, 12))
    assert e.value.code == -4 and "no HIP device" in str(e.value)
    h = C.c_void_p()
    assert L.l2j_create(None, C.byref(h)) == -1
    for bad in (l2j.Config(60, 256, 2, 4, 4, 50, 12),          # dim % 16
                l2j.Config(64, 256, 2, 4, 3, 50, 12),          # n_heads % n_kv_heads
                l2j.Config(64, 256, 0, 4, 4, 50, 12),          # zero layers
                l2j.Config(64, 256, 2, 4, 4, 50, 12, 1, 128)): # group size
        assert L.l2j_create(C.byref(bad), C.byref(h)) == -1
        assert L.l2j_last_error()
    assert L.l2j_forward(None, 1, 0, None) == -1
    assert L.l2j_finalize(None) == -1
    L.l2j_destroy(None)  # no-op


def test_rows_of_a_batch_are_cut_where_the_reference_loop_stops():
    import llama2j_amd as l2j
    rows = np.array([[5, 9, 1, 7, 1], [4, 4, 4, 4, 4], [1, 2, 3, 4, 5]], dtype=np.int32)
    cut = l2j.Transformer.until_bos(rows)
    assert [list(r) for r in cut] == [[5, 9, 1], [4, 4, 4, 4, 4], [1]]
