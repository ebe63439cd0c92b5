"""GPU parity tests: everything goes through the C ABI of libllama2j_hip.so and is checked against the
CPU oracle (a restatement of llama2j's CPU mode; the reference itself is Java and was never executed)
on the same seeded inputs.

Bars: bit-exact for bytes, codes and token ids; logits within 1e-3 of the oracle's, measured as
max|delta| / max|logit| per step (the tolerance the task states); first 64 greedy tokens identical."""
import ctypes as C
import os
import sys
import time

import numpy as np
import pytest

import llama2j_amd as l2j
from llama2j_amd import BUFFER, TENSOR

pytestmark = pytest.mark.gpu

LOGIT_TOL = 1e-3

# oracle tensor index -> library tensor id (file order; the library adds the fp32 tensors at both ends)
QT = [TENSOR.RMS_ATT, TENSOR.WQ, TENSOR.WK, TENSOR.WV, TENSOR.WO, TENSOR.RMS_FFN, TENSOR.W1, TENSOR.W2,
      TENSOR.W3, TENSOR.RMS_FINAL]


@pytest.fixture(params=["token", "phase"])
def launch_mode(request, monkeypatch):
    """The forward pass as one whole-token launch (the default for large models) or as one launch per phase
    (the default for small ones); the library reads the switch when a transformer is finalized."""
    monkeypatch.setenv("L2J_FUSE", "1" if request.param == "token" else "0")
    return request.param


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def make_pair(orc, shape, seed, sigma=0.02, realistic=False, upload="bytes"):
    """An oracle model and a GPU transformer holding bit-identical weights."""
    dim, hidden, L, H, kvH, vocab, seq, shared = shape
    m = orc.Model(dim=dim, hidden_dim=hidden, n_layers=L, n_heads=H, n_kv_heads=kvH, vocab_size=vocab, seq_len=seq,
                  shared_weights=shared)
    m.fill_synth(seed, sigma)
    if realistic:  # norm weights near 1 and wider q/k so attention is far from uniform
        rng = np.random.default_rng(seed)
        for t in (orc.T_RMS_ATT, orc.T_RMS_FFN, orc.T_RMS_FINAL):
            m.set_quant(t, orc.quant_encode((1.0 + 0.1 * rng.standard_normal(m.tensor_floats(t))).astype(np.float32)))
        # (narrower for long rows: the reference shifts its softmax by a running maximum of element products, and scores
        # more than 87 below it underflow to an all-zero attention row there, which the GPU's true softmax does not copy)
        wide = 0.12 * min(1.0, 256.0 / dim)
        for t in (orc.T_WQ, orc.T_WK):
            m.set_quant(t, orc.quant_encode((wide * rng.standard_normal(m.tensor_floats(t))).astype(np.float32)))
    g = l2j.Transformer(l2j.Config(dim, hidden, L, H, kvH, vocab, seq, shared))
    if upload == "synthetic":
        g.fill_synthetic(seed, sigma)
    else:
        g.upload_f32(TENSOR.TOK_EMB, m.emb())
        if not shared:
            g.upload_f32(TENSOR.WCLS, m.wcls())
        for t in range(10):
            g.upload_quant(QT[t], m.quant(t))
    g.finalize()
    return m, g


def rel_err(got, want):
    return float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max())


TINY = [
    (64, 256, 2, 4, 4, 50, 12, 1),
    (96, 160, 2, 2, 2, 40, 10, 0),      # head 48; rows and layers straddle quantization groups
    (32, 48, 3, 4, 2, 30, 8, 1),        # multiquery (kv_mul 2), kv_dim 16
    (256, 512, 2, 2, 2, 64, 6, 0),      # 256-aligned, head 128
    (512, 1024, 1, 2, 2, 100, 8, 0),    # head 256 (64 lanes per cache row)
    (64, 4352, 1, 4, 4, 40, 6, 0),      # W2 rows of 272 chunks: one row per wave, two steps of four chunks per lane
    (64, 8448, 1, 4, 4, 40, 6, 0),      # W2 rows of 528 chunks: one row per wave, one step of six chunks per lane
    (1280, 1536, 1, 10, 10, 64, 6, 0),  # rows of 80 and 96 chunks: two chunks per lane
    (4352, 256, 1, 34, 34, 40, 6, 0),   # rows of 272 chunks: five chunks per lane, three of them requested ahead
]


# ------------------------------------------------------------------ load path: bytes and codes, bit exact

def test_upload_read_back_and_gpu_encoder_are_bit_exact(orc):
    shape = (96, 160, 2, 2, 2, 40, 10, 0)
    m, g = make_pair(orc, shape, seed=11)
    for t in range(10):
        ref = m.quant(t)
        np.testing.assert_array_equal(g.read_quant(QT[t], 0, ref.size // 264), ref)
    # GPU Quant.encode from fp32 (tail group partial for the rms tensors: 2*96 = 192 floats)
    g2 = l2j.Transformer(l2j.Config(*shape))
    rng = np.random.default_rng(3)
    for t in range(10):
        x = (rng.standard_normal(m.tensor_floats(t)) * 0.02).astype(np.float32)
        x[::97] = 0.0
        if t == 1:
            x[:256] = 0.5  # constant group -> NaN rule -> zero codes
        g2.upload_f32_quantize(QT[t], x)
        np.testing.assert_array_equal(g2.read_quant(QT[t], 0, orc.quant_nbytes(x.size) // 264), orc.quant_encode(x))
    # in two slices at a group boundary
    x = (rng.standard_normal(m.tensor_floats(1)) * 0.02).astype(np.float32)
    g2.upload_f32_quantize(QT[1], x[:512], first=0)
    g2.upload_f32_quantize(QT[1], x[512:], first=512)
    np.testing.assert_array_equal(g2.read_quant(QT[1], 0, orc.quant_nbytes(x.size) // 264), orc.quant_encode(x))
    # the reference's self-check vector through the GPU encoder
    g3 = l2j.Transformer(l2j.Config(16, 16, 1, 1, 1, 4, 4, 1))
    v = np.zeros(256, np.float32)
    v[:100] = np.arange(100)
    g3.upload_f32_quantize(TENSOR.WQ, v)
    enc = g3.read_quant(TENSOR.WQ, 0, 1)
    assert bytes(enc[:8]).hex() == "0000000042c60000"
    assert list(enc[8:18]) == [0, 3, 5, 8, 10, 13, 15, 18, 21, 23] and enc[8 + 50] == 129 and enc[8 + 99] == 255


def test_seeded_fill_matches_oracle_generator_bit_for_bit(orc):
    shape = (96, 160, 2, 2, 2, 400, 10, 0)
    m, g = make_pair(orc, shape, seed=5, upload="synthetic")
    for t in range(10):
        ref = m.quant(t)
        np.testing.assert_array_equal(g.read_quant(QT[t], 0, ref.size // 264), ref)
    lg = g.forward(7, 0)
    want = m.forward(7, 0)
    assert rel_err(lg, want) < LOGIT_TOL  # embedding and classifier fills agree too


# ------------------------------------------------------------------ op level (the pattern of Mode.TEST)

@pytest.mark.parametrize("shape", TINY)
def test_per_layer_taps_match_oracle(orc, shape):
    m, g = make_pair(orc, shape, seed=21, realistic=True)
    m.enable_taps()
    rng = np.random.default_rng(1)
    toks = rng.integers(0, shape[5], size=shape[6])
    L = shape[2]
    pairs = [(BUFFER.Q, orc.TAP_Q), (BUFFER.K, orc.TAP_K), (BUFFER.V, orc.TAP_V), (BUFFER.XB, orc.TAP_ATT_OUT),
             (BUFFER.XB2, orc.TAP_X_ATT), (BUFFER.HB, orc.TAP_HB), (BUFFER.X, orc.TAP_X_FFN)]
    for pos, tok in enumerate(toks):
        want = m.forward(int(tok), pos).copy()
        got = g.forward_taps(int(tok), pos)
        for l in range(L):
            for gb, ob in pairs:
                a, b = g.read(gb, layer=l), m.tap(ob, l)
                # reference's own per-kernel thresholds are absolute 1e-5..1e-3 (K/Kernel.java:175-196)
                tol = 2e-5 * max(1.0, float(np.abs(b).max()))
                assert np.abs(a - b).max() <= tol, (pos, l, gb, float(np.abs(a - b).max()), tol)
        assert rel_err(got, want) < 1e-4
        # cache rows: row pos written, later rows untouched (zero)
        kc = g.read(BUFFER.KCACHE, layer=L - 1).reshape(shape[6], -1)
        np.testing.assert_allclose(kc[pos], m.tap(orc.TAP_K, L - 1), atol=2e-5 * max(1.0, float(np.abs(kc[pos]).max())))
        assert not kc[pos + 1:].any()
    # pos 0: softmax of one score is exactly 1, so attention output == v bit for bit
    m.reset(); g.reset()
    m.forward(3, 0); g.forward_taps(3, 0)
    dim, hs, kv_mul = shape[0], shape[0] // shape[3], shape[3] // shape[4]
    i = np.arange(dim)
    np.testing.assert_array_equal(g.read(BUFFER.XB, layer=0), g.read(BUFFER.V, layer=0)[i // hs // kv_mul * hs + i % hs])


def test_token_kernel_equals_kernel_by_kernel_launch_and_is_deterministic(orc, launch_mode):
    m, g = make_pair(orc, TINY[1], seed=31, realistic=True)
    outs = []
    for rep in range(3):
        g.reset()
        seq = [g.forward(5 + p, p).copy() for p in range(6)]
        outs.append(np.stack(seq))
    np.testing.assert_array_equal(outs[0], outs[1])
    np.testing.assert_array_equal(outs[0], outs[2])
    g.reset()
    # the kernel-by-kernel path (used for taps) folds attention splits in another order: equal to rounding
    eager = np.stack([g.forward_taps(5 + p, p).copy() for p in range(6)])
    eager2 = np.stack([g.forward_taps(5 + p, p).copy() for p in range(6)])
    np.testing.assert_array_equal(eager, eager2)
    assert rel_err(outs[0], eager) < 1e-5
    # fused argmax == first-max of the logits the same forward produced
    g.reset()
    for p in range(6):
        nxt = g.forward_argmax(5 + p, p)
        assert nxt == int(np.argmax(outs[0][p]))


@pytest.mark.parametrize("shape", TINY)
def test_forward_matches_oracle_in_both_launch_modes(orc, shape, launch_mode):
    # every tiny shape (head 16..256, multiquery, unaligned rows) through l2j_forward at every position
    m, g = make_pair(orc, shape, seed=23, realistic=True)
    rng = np.random.default_rng(2)
    for pos, tok in enumerate(rng.integers(0, shape[5], size=shape[6])):
        assert rel_err(g.forward(int(tok), pos), m.forward(int(tok), pos)) < 1e-4, pos


# Row lengths on both sides of the steps at which the kernels change the chunks a lane holds (64, 128, 256, 320 chunks
# for row pairs; 512 and 768 for single rows), odd head counts, multiquery, shared and separate classifier.
BOUNDARY = [
    (1024, 12304, 1, 8, 4, 40, 6, 1),     # rows of 64 chunks; W2 rows of 769
    (1040, 8208, 1, 65, 65, 40, 6, 1),    # 65 chunks; 513
    (2048, 4112, 1, 8, 8, 40, 6, 0),      # 128; 257
    (2064, 5136, 2, 43, 43, 40, 6, 1),    # 129; 321
    (3200, 1040, 1, 40, 20, 40, 6, 1),    # 200; 65
    (4112, 5120, 1, 257, 257, 40, 6, 0),  # 257; 320
    (5120, 12288, 1, 32, 16, 40, 6, 1),   # 320; 768
    (5136, 8192, 1, 107, 107, 40, 6, 1),  # 321; 512
]


@pytest.mark.parametrize("shape", BOUNDARY)
def test_row_length_boundaries_in_both_launch_modes(orc, shape, launch_mode):
    m, g = make_pair(orc, shape, seed=29, realistic=True)
    rng = np.random.default_rng(4)
    for pos, tok in enumerate(rng.integers(0, shape[5], size=4)):
        assert rel_err(g.forward(int(tok), pos), m.forward(int(tok), pos)) < 1e-4, pos


def test_split_attention_in_both_launch_modes(orc, launch_mode):
    # contexts long enough that attention is split over several workgroups (whole-token launch: beyond 64
    # positions; kernel-by-kernel: beyond 32) and folded by the last arriver; multiquery, head 16
    shape = (64, 96, 2, 4, 2, 40, 200, 1)
    m, g = make_pair(orc, shape, seed=33, realistic=True)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, shape[5], size=shape[6])
    fused = []
    for pos, tok in enumerate(toks):
        want = m.forward(int(tok), pos)
        got = g.forward(int(tok), pos)
        assert rel_err(got, want) < 1e-4, pos
        fused.append(got.copy())
    g.reset()
    for pos, tok in enumerate(toks):
        got = g.forward_taps(int(tok), pos)
        assert rel_err(got, fused[pos]) < 1e-5, pos


def test_kernel_timing_entry_point(orc, launch_mode):
    # every kernel class launches and reports a time, deep enough in the context that attention is split;
    # the measurement leaves the context usable (same tokens before and after)
    shape = (64, 96, 2, 4, 2, 40, 200, 1)
    m, g = make_pair(orc, shape, seed=34, realistic=True)
    prompt = orc.synth_prompt(34, 4, shape[5])
    before, _ = g.decode_greedy(prompt, 160)
    for k in range(6):
        us, nbytes = g.time_kernel(k, 150, rounds=2)
        assert us > 0.0 and nbytes > 0, k
    if launch_mode == "token":
        us, nbytes = g.time_kernel(l2j.KERNEL.TOKEN, 150, rounds=2)
        assert us > 0.0 and nbytes == g.bytes_per_token(150)
    else:  # no whole-token kernel in this mode
        with pytest.raises(l2j.L2JError) as e:
            g.time_kernel(l2j.KERNEL.TOKEN, 150, rounds=1)
        assert e.value.code == -3
    g.reset()
    after, _ = g.decode_greedy(prompt, 160)
    np.testing.assert_array_equal(before, after)
    want, _, _ = m.generate_greedy(prompt, 160)
    np.testing.assert_array_equal(after, want)


@pytest.mark.parametrize("env", [{"L2J_BY_VALUE": "0"}, {"L2J_LAYERS_PER_LAUNCH": "1"}, {"L2J_BY_VALUE": "1"},
                                 {"L2J_SELF_CONTAINED": "0"}, {"L2J_SELF_CONTAINED": "1"}, {"L2J_SELF_CONTAINED": "2"},
                                 {"L2J_GRAPH_TOKENS": "1"}, {"L2J_GRAPH_TOKENS": "7"}, {"L2J_GRAPH": "0"}])
def test_whole_token_kernel_hand_over_variants(orc, monkeypatch, env):
    # the whole-token kernel with grid barriers instead of the hand-over by value, with one launch per layer (which
    # implies barriers), by value (the default: the kernel alternates two sets of vectors and steps the token loop
    # itself), by value with k_fill_unset before and / or k_finish after every token, with other numbers of tokens per
    # graph replay and without graphs: same tokens as the oracle, deep enough that attention runs in several splits
    monkeypatch.setenv("L2J_FUSE", "1")
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    for shape in ((64, 96, 3, 4, 2, 40, 200, 1), (256, 512, 2, 2, 2, 64, 96, 0)):
        m, g = make_pair(orc, shape, seed=61, realistic=True)
        prompt = orc.synth_prompt(61, 4, shape[5])
        want, _, _ = m.generate_greedy(prompt, min(160, shape[6]))
        got, _ = g.decode_greedy(prompt, min(160, shape[6]))
        np.testing.assert_array_equal(got, want)
        g.close()


@pytest.mark.parametrize("shape", [(4352, 256, 1, 34, 34, 40, 6, 0), (768, 2048, 2, 12, 12, 64, 8, 1), (288, 768, 2, 6, 6, 64, 8, 1)])
def test_general_token_kernel_on_shapes_that_have_an_instance_of_their_own(orc, monkeypatch, shape):
    # rows of 272, 48 and 18 chunks: by default k_token is instantiated with five, one and one chunks per lane for them
    monkeypatch.setenv("L2J_FUSE", "1")
    monkeypatch.setenv("L2J_TOKEN_SPECIAL", "0")
    m, g = make_pair(orc, shape, seed=67, realistic=True)
    rng = np.random.default_rng(6)
    for pos, tok in enumerate(rng.integers(0, shape[5], size=shape[6])):
        assert rel_err(g.forward(int(tok), pos), m.forward(int(tok), pos)) < 1e-4, pos


def test_whole_token_kernel_between_other_launches(orc, monkeypatch):
    """The self-contained whole-token kernel keeps its own book on which activation vectors read 'unwritten'.  Launches
    that write those vectors behind its back (per-layer taps, phases timed on their own) must not confuse it: tokens
    and logits of forwards mixed with such launches equal the oracle's, and the live taps name the set the last token used."""
    monkeypatch.setenv("L2J_FUSE", "1")
    shape = (256, 512, 3, 2, 2, 64, 40, 0)
    m, g = make_pair(orc, shape, seed=71, realistic=True)
    m.enable_taps()
    tok = 1
    for pos in range(24):
        want = m.forward(tok, pos).copy()
        if pos % 5 == 3:
            got = g.forward_taps(tok, pos)            # per-phase launches: they leave values in set 0
        elif pos % 5 == 4:
            g.time_kernel(l2j.KERNEL.W13, pos, 1)     # a phase on its own, then the whole-token kernel again
            got = g.forward(tok, pos)
        else:
            got = g.forward(tok, pos)                 # consecutive whole-token launches alternate the sets
            x, ref = g.read(BUFFER.X), m.tap(orc.TAP_X_FFN, shape[2] - 1)   # the residual stream the classifier read
            assert np.abs(x - ref).max() <= 2e-5 * max(1.0, float(np.abs(ref).max())), pos
        assert rel_err(got, want) < LOGIT_TOL, pos
        tok = int(np.argmax(want))
    m.close(); g.close()


def test_decode_stops_inside_a_replayed_batch(orc, monkeypatch):
    """The decode loop replays several tokens per graph launch and enqueues the next batch before it has looked at
    this one's tokens; a sequence that emits token 1 in the middle of a batch still ends there (J/Run.java:670-672)."""
    monkeypatch.setenv("L2J_FUSE", "1")
    monkeypatch.setenv("L2J_GRAPH_TOKENS", "8")
    shape = (64, 96, 2, 4, 4, 3, 200, 1)   # a vocabulary of three: token 1 comes up within a few steps
    for seed in range(40, 48):
        m, g = make_pair(orc, shape, seed=seed, realistic=True)
        want, _, _ = m.generate_greedy(np.array([2, 0, 2, 2, 0], np.int32), 200)
        got, sec = g.decode_greedy(np.array([2, 0, 2, 2, 0], np.int32), 200)
        np.testing.assert_array_equal(got, want)
        assert sec >= 0.0
        # and the context is usable afterwards: a fresh decode gives the same tokens
        g.reset()
        got2, _ = g.decode_greedy(np.array([2, 0, 2, 2, 0], np.int32), 200)
        np.testing.assert_array_equal(got2, want)
        m.close(); g.close()


def test_barrier_time_out_is_reported_not_hung(orc, monkeypatch):
    # a spin limit of zero makes the bounded waits of the whole-token kernel give up at once: every kernel still
    # runs to its end, the call reports the failure, and a context with the normal limit is unaffected
    shape = (64, 96, 2, 4, 2, 40, 32, 1)
    monkeypatch.setenv("L2J_FUSE", "1")
    monkeypatch.setenv("L2J_BARRIER_SPINS", "0")
    monkeypatch.setenv("L2J_FALLBACK", "0")
    m, bad = make_pair(orc, shape, seed=50)
    failures = 0
    for pos in range(8):
        try:
            bad.forward(3, pos)
        except l2j.L2JError as e:
            assert e.code == -4 and "bounded wait" in str(e)
            failures += 1
    assert failures > 0
    monkeypatch.setenv("L2J_BARRIER_SPINS", "20000")
    m2, good = make_pair(orc, shape, seed=50)
    for pos in range(8):
        assert rel_err(good.forward(3, pos), m2.forward(3, pos)) < 1e-4
    # the context whose waits expired works again once the stale state is gone
    bad.close()


def test_waits_that_run_out_fall_back_to_one_launch_per_phase(orc, monkeypatch):
    """The whole-token kernel needs every workgroup resident; when its bounded waits run out (forced here by a spin limit of
    zero; in the field by another process holding compute units) the context switches to one launch per phase for good
    and repeats the call: the caller sees correct results, not an error."""
    shape = (64, 96, 2, 4, 2, 40, 32, 1)
    monkeypatch.setenv("L2J_FUSE", "1")
    monkeypatch.setenv("L2J_BARRIER_SPINS", "0")
    for entry in ("forward", "forward_argmax", "decode_greedy", "decode_sample"):
        m, g = make_pair(orc, shape, seed=51, realistic=True)
        assert g.get_option("fuse") == 1 and g.get_option("fallback") == 1
        prompt = orc.synth_prompt(51, 3, shape[5])
        if entry == "forward":
            assert rel_err(g.forward(3, 0), m.forward(3, 0)) < 1e-4
        elif entry == "forward_argmax":
            assert g.forward_argmax(3, 0) == int(np.argmax(m.forward(3, 0)))
        elif entry == "decode_greedy":
            np.testing.assert_array_equal(g.decode_greedy(prompt, 24)[0], m.generate_greedy(prompt, 24)[0])
        else:
            np.testing.assert_array_equal(g.decode_sample(prompt, 24, 0.0, 0.9, 7)[0], m.generate_greedy(prompt, 24)[0])
        assert g.get_option("fuse") == 0          # the switch is for good
        m.reset()
        for pos in range(4):                      # and the context goes on working, phase by phase
            assert rel_err(g.forward(5, pos), m.forward(5, pos)) < 1e-4
        m.close(); g.close()


def test_two_contexts_decode_from_two_threads(orc, launch_mode):
    # forwards of different contexts take turns on the device: concurrent decodes give the sequential answers
    import threading
    shape = (64, 96, 2, 4, 2, 40, 96, 1)
    pairs = [make_pair(orc, shape, seed=40 + i, realistic=True) for i in range(2)]
    prompts = [orc.synth_prompt(40 + i, 3, shape[5]) for i in range(2)]
    want = [g.decode_greedy(p, 90)[0].copy() for (m, g), p in zip(pairs, prompts)]
    for m, g in pairs:
        g.reset()
    got = [None, None]

    def work(i):
        for rep in range(3):
            pairs[i][1].reset()
            got[i] = pairs[i][1].decode_greedy(prompts[i], 90)[0].copy()

    ts = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    for i in range(2):
        np.testing.assert_array_equal(got[i], want[i])
        np.testing.assert_array_equal(got[i], pairs[i][0].generate_greedy(prompts[i], 90)[0])


def test_argmax_first_max_tie_rule(orc, launch_mode):
    # identical classifier rows give exactly equal logits: the lowest index must win (J/Sampler.java:51)
    shape = (64, 256, 1, 4, 4, 1000, 4, 0)
    m, g0 = make_pair(orc, shape, seed=41)
    g0.close()
    w = m.wcls().reshape(1000, 64)
    x = m.forward(3, 0)
    top = int(np.argmax(x))
    for dup in (top + 1, 998, 999):
        if dup != top:
            w[dup] = w[top]
    w[0] = w[top]  # index 0 ties too and must win
    g = l2j.Transformer(l2j.Config(*shape))
    g.upload_f32(TENSOR.TOK_EMB, m.emb()); g.upload_f32(TENSOR.WCLS, m.wcls())
    for t in range(10):
        g.upload_quant(QT[t], m.quant(t))
    g.finalize()
    lg = g.forward(3, 0)
    assert lg[0] == lg[top] == lg[999]
    assert g.forward_argmax(3, 0) == 0 == orc.argmax(m.forward(3, 0))


# ------------------------------------------------------------------ token loop

def test_decode_greedy_loop_semantics(orc, launch_mode):
    m, g = make_pair(orc, TINY[0], seed=51, realistic=True)
    prompt = np.array([5, 9, 11], np.int32)
    want, _, _ = m.generate_greedy(prompt, 10)
    got, sec = g.decode_greedy(prompt, 10)
    np.testing.assert_array_equal(got, want)
    assert list(got[:3]) == [5, 9, 11] and sec > 0
    # a forced BOS (1) ends the loop right after it is emitted (J/Run.java:670-672)
    m.reset(); g.reset()
    got, _ = g.decode_greedy(np.array([5, 1, 7], np.int32), 10)
    assert list(got) == [5, 1] == list(m.generate_greedy(np.array([5, 1, 7], np.int32), 10)[0])
    # steps <= 0 and steps > seq_len clamp to seq_len (J/Run.java:599-603)
    for steps in (0, 1000):
        m.reset(); g.reset()
        want, _, _ = m.generate_greedy(prompt, steps)
        got, _ = g.decode_greedy(prompt, steps)
        np.testing.assert_array_equal(got, want)
        assert len(got) <= 12
    # empty prompt; single step
    m.reset(); g.reset()
    np.testing.assert_array_equal(g.decode_greedy(np.zeros(0, np.int32), 5)[0], m.generate_greedy(np.zeros(0, np.int32), 5)[0])
    g.reset()
    assert len(g.decode_greedy(prompt, 1)[0]) == 1


def test_error_codes_on_gpu(orc):
    L = l2j.lib()
    g = l2j.Transformer(l2j.Config(64, 256, 2, 4, 4, 50, 12, 1))
    with pytest.raises(l2j.L2JError) as e:
        g.forward(1, 0)
    assert e.value.code == -3  # forward before finalize
    with pytest.raises(l2j.L2JError) as e:
        g.finalize()
    assert e.value.code == -3  # tensors missing
    with pytest.raises(l2j.L2JError) as e:
        g.upload_quant(TENSOR.WQ, np.zeros(264, np.uint8))
    assert e.value.code == -2  # wrong byte count (J/TransformerWeights.java:228-232)
    with pytest.raises(l2j.L2JError) as e:
        g.upload_quant(TENSOR.TOK_EMB, np.zeros(264, np.uint8))
    assert e.value.code == -1
    with pytest.raises(l2j.L2JError) as e:
        g.upload_f32(TENSOR.TOK_EMB, np.zeros(7, np.float32))
    assert e.value.code == -2
    with pytest.raises(l2j.L2JError) as e:
        g.upload_quant_layer(TENSOR.RMS_ATT, 0, np.zeros(264, np.uint8))
    assert e.value.code == -1  # a layer of 64 floats is not a whole group
    g.fill_synthetic(1)
    g.finalize()
    for tok, pos in [(-1, 0), (50, 0), (1, -1), (1, 12)]:
        with pytest.raises(l2j.L2JError) as e:
            g.forward(tok, pos)
        assert e.value.code == -1
    with pytest.raises(l2j.L2JError) as e:
        g.upload_quant(TENSOR.WQ, np.zeros(264 * 32, np.uint8))
    assert e.value.code == -3  # upload after finalize
    with pytest.raises(l2j.L2JError) as e:
        g.decode_greedy(np.array([77], np.int32), 4)
    assert e.value.code == -1  # prompt id outside the vocabulary
    with pytest.raises(l2j.L2JError):
        g.read(BUFFER.KCACHE, layer=5)
    g.forward(1, 0)  # still usable after errors


def test_upload_by_layer_and_from_threads(orc):
    # the reference uploads from ten threads at once (J/TransformerWeights.java:52,204)
    import threading
    shape = (256, 512, 2, 2, 2, 64, 6, 0)
    m, g0 = make_pair(orc, shape, seed=61, realistic=True)
    want = g0.forward(3, 0)
    g0.close()
    g = l2j.Transformer(l2j.Config(*shape))
    g.upload_f32(TENSOR.TOK_EMB, m.emb()); g.upload_f32(TENSOR.WCLS, m.wcls())
    errs = []

    def up(t):
        try:
            ref = m.quant(t)
            if QT[t] in (TENSOR.RMS_ATT, TENSOR.RMS_FFN, TENSOR.RMS_FINAL):
                g.upload_quant(QT[t], ref)
            else:
                per = ref.size // 2
                for l in range(2):
                    g.upload_quant_layer(QT[t], l, ref[l * per:(l + 1) * per])
        except Exception as ex:  # pragma: no cover
            errs.append(ex)
    th = [threading.Thread(target=up, args=(t,)) for t in range(10)]
    [t.start() for t in th]
    [t.join() for t in th]
    assert not errs
    g.finalize()
    np.testing.assert_array_equal(g.forward(3, 0), want)


def test_error_text_is_kept_per_context_across_threads(orc):
    """A failing call on thread A, the message fetched on thread B (a Java virtual thread may be mounted on another
    carrier thread for its second downcall): l2j_ctx_last_error has it, the thread-local l2j_last_error of B does not."""
    import threading
    g = l2j.Transformer(l2j.Config(64, 128, 1, 4, 4, 64, 8, 1))
    other = l2j.Transformer(l2j.Config(64, 128, 1, 4, 4, 64, 8, 1))
    L = l2j.lib()
    rcs, seen = [], {}

    def a():
        bad = np.zeros(264, np.uint8)
        rcs.append(L.l2j_upload_quant(g._h, TENSOR.WQ, bad.ctypes.data_as(C.POINTER(C.c_uint8)), bad.size))

    def b():
        seen["ctx"] = g.last_error()
        seen["other"] = other.last_error()
        seen["thread"] = L.l2j_last_error().decode()
    for f in (a, b):
        t = threading.Thread(target=f)
        t.start()
        t.join()
    assert rcs == [-2]
    assert "numberOfBytesByFloatSize" in seen["ctx"]
    assert seen["other"] == "" and "numberOfBytesByFloatSize" not in seen["thread"]
    # an option that fixes a launch shape is refused once the shapes are fixed; an unknown one always
    g.fill_synthetic(1, 0.02)
    g.set_option("threads", 512)
    g.finalize()
    with pytest.raises(l2j.L2JError) as e:
        g.set_option("threads", 1024)
    assert e.value.code == -3 and "threads" in str(e.value)
    with pytest.raises(l2j.L2JError) as e:
        g.set_option("no_such_option", 1)
    assert e.value.code == -1
    g.set_option("sampler_scan", 0)  # allowed at any time
    g.close(); other.close()


def test_options_override_the_process_defaults(orc, monkeypatch):
    """The same model finalized with the launch mode given per context (no environment involved) computes the same
    logits on the whole-token path, with grid barriers, and with one launch per phase."""
    shape = (256, 512, 2, 2, 2, 64, 6, 0)
    for k in ("L2J_FUSE", "L2J_BY_VALUE", "L2J_GRAPH"):
        monkeypatch.delenv(k, raising=False)
    m = orc.Model(dim=shape[0], hidden_dim=shape[1], n_layers=shape[2], n_heads=shape[3], n_kv_heads=shape[4],
                  vocab_size=shape[5], seq_len=shape[6], shared_weights=shape[7])
    m.fill_synth(9, 0.02)
    want = [m.forward(3 + p, p).copy() for p in range(4)]
    for opts in ({"fuse": 1}, {"fuse": 1, "by_value": 0}, {"fuse": 0}, {"fuse": 1, "graph": 0}, {"fuse": 0, "graph": 0}):
        g = l2j.Transformer(l2j.Config(*shape), options=opts)
        g.fill_synthetic(9, 0.02)
        g.finalize()
        for p in range(4):
            assert rel_err(g.forward(3 + p, p), want[p]) < LOGIT_TOL, (opts, p)
        # the decode loop times itself with the device's wall clock: the rate is known here, and a run has a duration
        assert g.get_option("wall_clock_khz") > 0
        toks, sec = g.decode_greedy(np.array([3, 4], dtype=np.int32), 6)
        assert len(toks) > 1 and 0.0 < sec < 1.0
        with pytest.raises(l2j.L2JError):
            g.set_option("wall_clock_khz", 5)        # read-only
        g.close()
    m.close()


def test_checkpoint_loader_and_quant_caches(orc, tmp_path):
    from tests.test_oracle_forward import write_bin
    cfg = (64, 96, 2, 4, 2, 30, 8)
    dim, hidden, L, H, kvH, vocab, seq = cfg
    rng = np.random.default_rng(8)
    kvd = dim * kvH // H
    sizes = [L * dim, L * dim * dim, L * dim * kvd, L * dim * kvd, L * dim * dim, L * dim, L * dim * hidden,
             L * hidden * dim, L * dim * hidden, dim]
    tens = [(rng.standard_normal(n) * 0.05).astype(np.float32) for n in sizes]
    tens[0] += 1; tens[5] += 1; tens[9] += 1
    emb = (rng.standard_normal(vocab * dim) * 0.05).astype(np.float32)
    wcls = (rng.standard_normal(vocab * dim) * 0.05).astype(np.float32)
    path = str(tmp_path / "tiny.bin")
    write_bin(path, cfg, emb, tens, wcls)
    g = l2j.Transformer.from_checkpoint(path, write_caches=True)   # quantizes on the GPU, writes caches
    c = g.config
    assert (c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len, c.shared_weights) == cfg + (0,)
    stems = ["l_rms_att_weight", "l_wq", "l_wk", "l_wv", "l_wo", "l_rms_ffn_weight", "l_w1", "l_w2", "l_w3",
             "rms_final_weight"]
    for t, stem in enumerate(stems):
        raw = (tmp_path / ("tiny_%s_256_8.quant" % stem)).read_bytes()
        assert int.from_bytes(raw[:4], "little") == len(raw) - 4
        np.testing.assert_array_equal(np.frombuffer(raw[4:], np.uint8), orc.quant_encode(tens[t]))
    lg = g.forward(3, 0)
    mo = orc.Model.load(path, write_caches=False)                    # the oracle reads OUR cache files
    assert rel_err(lg, mo.forward(3, 0)) < 1e-4
    # second load takes the cache branch: poison the fp32 tensors to prove the floats are skipped
    write_bin(path, cfg, emb, [np.zeros_like(t) for t in tens], wcls)
    g2 = l2j.Transformer.from_checkpoint(path, write_caches=False)
    np.testing.assert_array_equal(g2.forward(3, 0), lg)
    (tmp_path / "tiny_l_wq_256_8.quant").write_bytes((264).to_bytes(4, "little") + bytes(264))
    with pytest.raises(l2j.L2JError) as e:
        l2j.Transformer.from_checkpoint(path)
    assert e.value.code == -2
    with pytest.raises(l2j.L2JError) as e:
        l2j.Transformer.from_checkpoint(str(tmp_path / "absent.bin"))
    assert e.value.code == -6


# ------------------------------------------------------------------ whole model, the five benchmark configurations

def run_config(orc, name, shape, seed, n_prompt, n_steps, n_logit_steps, late=None):
    """Greedy decode on both sides: identical tokens; per-step logits for the first n_logit_steps."""
    say("[%s] building seed=%d shape=%s" % (name, seed, shape))
    t0 = time.time()
    m, g = make_pair(orc, shape, seed, upload="synthetic")
    say("[%s] weights ready in %.1fs" % (name, time.time() - t0))
    prompt = orc.synth_prompt(seed, n_prompt, shape[5])
    t0 = time.time()
    want_tok, want_logits, cpu_sec = m.generate_greedy(prompt, n_steps, want_logits=True)
    say("[%s] oracle %d steps in %.1fs (%d threads)" % (name, len(want_tok), time.time() - t0, orc.lib().orc_num_threads()))
    got_tok, gpu_sec = g.decode_greedy(prompt, n_steps)
    say("[%s] gpu    %d steps, %.1f tok/s" % (name, len(got_tok), (len(got_tok) - 1) / max(gpu_sec, 1e-9)))
    n_cmp = min(len(want_tok), n_prompt + 64)
    np.testing.assert_array_equal(got_tok[:n_cmp], want_tok[:n_cmp])   # first 64 greedy tokens identical
    np.testing.assert_array_equal(got_tok, want_tok)
    # per-step logits: replay the same token stream through l2j_forward
    g.reset()
    tok, worst, min_gap = 1, 0.0, 1e9
    for pos in range(min(n_logit_steps, len(want_tok))):
        lg = g.forward(tok, pos)
        worst = max(worst, rel_err(lg, want_logits[pos]))
        if pos >= n_prompt:
            top2 = np.partition(want_logits[pos], -2)[-2:]
            min_gap = min(min_gap, float(top2[1] - top2[0]) / float(np.abs(want_logits[pos]).max()))
        tok = int(want_tok[pos])
    say("[%s] worst max|dlogit|/max|logit| = %.3g over %d steps; min relative top-2 gap = %.3g" %
        (name, worst, min(n_logit_steps, len(want_tok)), min_gap))
    assert worst < LOGIT_TOL
    if late:
        # The configuration's full length: the GPU decodes all of it, the rows its decode left in the KV cache are copied
        # into the oracle, and the oracle's single forwards at the last positions must give the GPU's logits and the token
        # the GPU's own loop emitted there (the oracle would need minutes to get there by itself).
        n_total, positions = late
        L, kvd = shape[2], shape[0] // shape[3] * shape[4]
        g.reset()
        toks, sec = g.decode_greedy(prompt, n_total)
        assert len(toks) == n_total, "the decode stopped early (token 1): pick another seed"
        np.testing.assert_array_equal(toks[:len(want_tok)], want_tok)
        kc, vc = m.buffer(orc.B_KCACHE).reshape(L, shape[6], kvd), m.buffer(orc.B_VCACHE).reshape(L, shape[6], kvd)
        for l in range(L):
            kc[l, :n_total] = g.read(BUFFER.KCACHE, layer=l, off=0, n=n_total * kvd).reshape(n_total, kvd)
            vc[l, :n_total] = g.read(BUFFER.VCACHE, layer=l, off=0, n=n_total * kvd).reshape(n_total, kvd)
        for pos in positions:
            tok = int(toks[pos - 1])
            want = m.forward(tok, pos).copy()
            got = g.forward(tok, pos)
            e = rel_err(got, want)
            say("[%s] %d steps at %.1f tok/s; pos %d: max|dlogit|/max|logit| = %.3g" % (name, n_total, (n_total - 1) / sec, pos, e))
            assert e < LOGIT_TOL, pos
            assert int(np.argmax(want)) == int(np.argmax(got)) == int(toks[pos]), pos
    m.close(); g.close()


def test_config1_stories15m_shape(orc, launch_mode):
    # dim 288: quantization groups straddle rows and layers, head 48; 8 prompt ids + 248 greedy
    run_config(orc, "15M", (288, 768, 6, 6, 6, 32000, 256, 1), seed=101, n_prompt=8, n_steps=256, n_logit_steps=256)


def test_config2_stories110m_shape(orc, launch_mode):
    # the configuration's full length: 16 prompt ids + 512 greedy tokens, logits at all 528 steps
    run_config(orc, "110M", (768, 2048, 12, 12, 12, 32000, 1024, 1), seed=102, n_prompt=16, n_steps=16 + 512,
               n_logit_steps=16 + 512)


def test_config3_llama2_7b_shape(orc):
    # 32 prompt ids + 64 greedy tokens against the oracle (the oracle takes ~0.3 s per token per 16 cores)
    # then the configuration's 32 + 256 on the GPU, and the oracle on the GPU's cache at the last positions
    run_config(orc, "7B", (4096, 11008, 32, 32, 32, 32000, 4096, 0), seed=103, n_prompt=32, n_steps=32 + 64,
               n_logit_steps=32 + 64, late=(32 + 256, (160, 285, 286, 287)))


def test_config4_long_context_attention(orc):
    # 7B attention geometry (32 heads x 128, seq 4096) with 2 layers: the KV cache is seeded with the
    # same random rows on both sides, then steps at positions deep in the context are compared.
    shape = (4096, 11008, 2, 32, 32, 32000, 4096, 1)
    m, g = make_pair(orc, shape, seed=104, upload="synthetic")
    rng = np.random.default_rng(4)
    kvd, S = 4096, 4096
    kc, vc = m.buffer(orc.B_KCACHE).reshape(2, S, kvd), m.buffer(orc.B_VCACHE).reshape(2, S, kvd)
    for l in range(2):
        k = (rng.standard_normal((S, kvd)) * 0.5).astype(np.float32)
        v = rng.standard_normal((S, kvd)).astype(np.float32)
        kc[l], vc[l] = k, v
        g.write_kv(l, 0, k, v)
    m.enable_taps()
    for pos in (3584, 3840, 4095, 127, 128, 1000):
        want = m.forward(17, pos).copy()
        got = g.forward_taps(17, pos)
        for l in range(2):
            a, b = g.read(BUFFER.XB, layer=l), m.tap(orc.TAP_ATT_OUT, l)
            assert np.abs(a - b).max() <= 2e-5 * max(1.0, float(np.abs(b).max())), (pos, l)
        assert rel_err(got, want) < LOGIT_TOL, pos
        assert rel_err(g.forward(17, pos), want) < LOGIT_TOL, pos  # the whole-token launch at the same position
    # round trip of the cache taps
    np.testing.assert_array_equal(g.read(BUFFER.VCACHE, layer=1, off=5 * kvd, n=kvd), vc[1, 5])


def test_config4_long_context_full_size(orc):
    """The 32-layer 7B shape deep in its context, on the whole-token path the long-context benchmark times.  The
    oracle cannot prefill 3584 positions in a test's time, so the GPU decodes the whole sequence (3584 forced prompt
    ids, then greedy to position 4095), its KV cache is copied into the oracle layer by layer, and the oracle then runs
    single forwards at chosen positions on that cache: logits within the bar and the same argmax as the token the
    GPU's own decode loop emitted there."""
    shape = (4096, 11008, 32, 32, 32, 32000, 4096, 0)
    L, S, kvd = shape[2], shape[6], 4096
    say("[C4 full] building")
    t0 = time.time()
    m, g = make_pair(orc, shape, seed=104, upload="synthetic")
    prompt = orc.synth_prompt(104, 3584, shape[5])
    toks, sec = g.decode_greedy(prompt, S)
    say("[C4 full] weights + %d GPU steps in %.1fs (%.1f tok/s after the first)" % (len(toks), time.time() - t0, (len(toks) - 1) / sec))
    assert len(toks) == S, "the decode stopped early (token 1): pick another seed"
    np.testing.assert_array_equal(toks[:3584], prompt)
    t0 = time.time()
    kc, vc = m.buffer(orc.B_KCACHE).reshape(L, S, kvd), m.buffer(orc.B_VCACHE).reshape(L, S, kvd)
    for l in range(L):
        kc[l] = g.read(BUFFER.KCACHE, layer=l).reshape(S, kvd)
        vc[l] = g.read(BUFFER.VCACHE, layer=l).reshape(S, kvd)
    say("[C4 full] cache copied into the oracle in %.1fs" % (time.time() - t0))
    worst = 0.0
    for pos in (3584, 3585, 3840, 4094, 4095):
        tok = int(toks[pos - 1])
        want = m.forward(tok, pos).copy()       # reads rows < pos of the GPU's cache, writes its own row pos
        got = g.forward(tok, pos)               # the whole-token launch replayed at that position
        e = rel_err(got, want)
        worst = max(worst, e)
        top2 = np.partition(want, -2)[-2:]
        say("[C4 full] pos %d: max|dlogit|/max|logit| = %.3g, relative top-2 gap %.3g" %
            (pos, e, float(top2[1] - top2[0]) / float(np.abs(want).max())))
        assert e < LOGIT_TOL, pos
        assert int(np.argmax(want)) == int(np.argmax(got)) == int(toks[pos]), pos
        # the row the oracle wrote at pos equals the one the GPU's decode left there
        for l in (0, L - 1):
            a = g.read(BUFFER.KCACHE, layer=l, off=pos * kvd, n=kvd)
            assert np.abs(a - kc[l, pos]).max() <= 2e-5 * max(1.0, float(np.abs(kc[l, pos]).max())), (pos, l)
    say("[C4 full] worst relative logit error %.3g" % worst)
    m.close(); g.close()


def test_llama2_70b_width_grouped_query(orc):
    # the 70B geometry (dim 8192, hidden 28672, 64 heads sharing 8 kv heads) at 4 layers: rows of two and seven steps,
    # 32 prompt ids + the first 64 greedy tokens, logits at all 96 steps
    run_config(orc, "70B width", (8192, 28672, 4, 64, 8, 32000, 4096, 0), seed=106, n_prompt=32, n_steps=32 + 64,
               n_logit_steps=32 + 64)


def test_llama2_70b_shape_full_depth(orc):
    # all 80 layers (72 GB of weights on the one GPU, the same again on the host for the oracle, which runs at
    # ~0.7 tok/s on 16 cores): 4 prompt ids + 12 greedy tokens, logits at all 16 steps
    run_config(orc, "70B", (8192, 28672, 80, 64, 8, 32000, 4096, 0), seed=107, n_prompt=4, n_steps=4 + 12,
               n_logit_steps=4 + 12)


def test_config5_llama2_13b_shape(orc):
    # the reference's int offsets overflow at this size (J/TransformerWeights.java:89); 64-bit here.
    # 32 prompt ids + the first 64 greedy tokens, logits at all 96 steps (the oracle runs at ~3.7 tok/s on 16 cores)
    run_config(orc, "13B", (5120, 13824, 40, 40, 40, 32000, 4096, 0), seed=105, n_prompt=32, n_steps=32 + 64,
               n_logit_steps=32 + 64, late=(32 + 256, (286, 287)))
