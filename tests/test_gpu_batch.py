"""Sixteen or thirty-two sequences at once (l2j_decode_greedy_batch, l2j_batch_matmul): the matrix-core path must give
every sequence what it gets alone.  Checked through the C ABI against the single-sequence path (itself pinned against the CPU oracle
in test_gpu_parity.py), against the oracle directly, and against float64 products of the dequantized weights."""
import numpy as np
import pytest

import llama2j_amd as l2j
from llama2j_amd import TENSOR
from llama2j_amd.binding import L2JError

pytestmark = pytest.mark.gpu

LOGIT_TOL = 1e-3   # per step: max |logit - oracle's| / max |oracle's logit|, the bar of the single-sequence path


def rel_err(got, want):
    return float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max())


def oracle_of(orc, shape, seed):
    m = orc.Model(dim=shape[0], hidden_dim=shape[1], n_layers=shape[2], n_heads=shape[3], n_kv_heads=shape[4],
                  vocab_size=shape[5], seq_len=shape[6], shared_weights=shape[7])
    m.fill_synth(seed, 0.02)
    return m


def check_against_oracle(m, prompt, steps, tokens, logits, what):
    """The oracle's own greedy loop from the same prompt: the same tokens (until it stops at token 1; the batch runs on), and at
    every one of those steps the batched path's logits within the bar of the oracle's."""
    m.reset()
    want_tok, want_logits, _ = m.generate_greedy(prompt, steps, want_logits=True)
    np.testing.assert_array_equal(tokens[:len(want_tok)], want_tok, err_msg=what)
    worst = max(rel_err(logits[pos], want_logits[pos]) for pos in range(len(want_tok)))
    assert worst < LOGIT_TOL, (what, worst)
    return worst

def same_until_a_tie(got, want, logits, what):
    """The batched path and the single-sequence path add the same products in different orders (their logits agree to a
    few 1e-6 of the largest), so a sequence may part ways where its two best logits lie that close together, and only
    there: the same tokens up to the first difference, and at that step the two tokens' logits (the batched path's) within
    1e-5 of the largest."""
    diff = np.flatnonzero(got != want)
    if diff.size == 0:
        return
    pos = int(diff[0])
    lg = logits[pos]
    gap = abs(float(lg[got[pos]]) - float(lg[want[pos]]))
    assert gap <= 1e-5 * float(np.abs(lg).max()), (what, pos, int(got[pos]), int(want[pos]), gap)


SHAPES = [
    (512, 1024, 4, 8, 8, 1008, 64, 1),      # head 64, shared classifier
    (512, 1024, 2, 8, 2, 1008, 64, 0),      # grouped-query attention: 8 heads on 2 kv heads
    (1024, 2816, 2, 8, 4, 2000, 96, 0),     # head 128, rows of 4 and 11 groups (an odd number of groups: a last slice of one)
    (512, 768, 2, 2, 2, 512, 40, 1),        # head 256
    (512, 1024, 2, 8, 2, 1008, 640, 0),     # 640 positions: the row slots of the attention kernel go round forty times
]


def dequantized(g, tensor, layer, rows, K):
    """One layer's matrix as float64, from the .quant bytes the library serialises (min, max big-endian, 256 codes)."""
    per = rows * K // 256
    raw = g.read_quant(tensor, layer * per, per).reshape(per, 264)
    hdr = raw[:, :8].copy().view(">f4").astype(np.float32)
    mn, mx = hdr[:, 0], hdr[:, 1]
    rm = ((mx - mn) / np.float32(255.0)).astype(np.float32)          # K/MatMul.java:137
    w = raw[:, 8:].astype(np.float32) * rm[:, None] + mn[:, None]    # K/MatMul.java:141
    return w.reshape(rows, K).astype(np.float64)


def test_matrix_core_product_matches_float64():
    shape = (1024, 2816, 2, 8, 4, 2000, 96, 0)
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(7, 0.02)
    g.finalize()
    rng = np.random.default_rng(0)
    kvd = 1024 * 4 // 8
    for tensor, rows, K in ((TENSOR.WQ, 1024, 1024), (TENSOR.WK, kvd, 1024), (TENSOR.W1, 2816, 1024), (TENSOR.W2, 1024, 2816)):
        x = (rng.standard_normal((16, K)) * np.exp(rng.uniform(-3, 3, (16, 1)))).astype(np.float32)
        want = x.astype(np.float64) @ dequantized(g, tensor, 1, rows, K).T
        got, _ = g.batch_matmul(tensor, 1, x, rows)
        err = np.abs(got - want).max(axis=1) / np.abs(want).max(axis=1)      # per sequence
        assert err.max() < 5e-6, (int(tensor), float(err.max()))
    g.close()


@pytest.mark.parametrize("n_seq", [16, 32])
@pytest.mark.parametrize("shape", [SHAPES[1], SHAPES[2], SHAPES[3]])
def test_the_layers_of_a_step_in_one_launch_give_the_same(orc, shape, n_seq):
    """Option batch_fuse = 1 runs all layers of a step in one resident kernel with grid barriers (deferred rmsnorm scalars,
    its own attention phase): the tokens of the launch-per-phase step, and the oracle's logits within the same bar."""
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(9, 0.02)
    g.finalize()
    rng = np.random.default_rng(shape[1] + n_seq)
    steps = shape[6]
    prompts = [rng.integers(2, shape[5], size=int(rng.integers(0, 9))).astype(np.int32) for _ in range(n_seq - 2)]
    want, _ = g.decode_greedy_batch(prompts, steps, n_seq=n_seq)
    g.set_option("batch_fuse", 1)
    got, logits = g.decode_greedy_batch(prompts, steps, n_seq=n_seq, want_logits=True)
    again, _ = g.decode_greedy_batch(prompts, steps, n_seq=n_seq)
    g.close()
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(again, got)
    m = oracle_of(orc, shape, 9)
    for b in (0, n_seq // 2, n_seq - 1):
        p = prompts[b] if b < len(prompts) else np.zeros(0, dtype=np.int32)
        check_against_oracle(m, p, steps, got[b], logits[:, b], "sequence %d against the oracle" % b)
    m.close()


@pytest.mark.parametrize("n_seq", [16, 32])
@pytest.mark.parametrize("shape", SHAPES)
def test_every_sequence_gets_what_it_gets_alone(orc, shape, n_seq):
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(9, 0.02)
    g.finalize()
    rng = np.random.default_rng(shape[0] + shape[4] + n_seq)
    steps = shape[6]
    prompts = [rng.integers(2, shape[5], size=int(rng.integers(0, 9))).astype(np.int32) for _ in range(n_seq - 3)]   # three without a prompt
    got, sec = g.decode_greedy_batch(prompts, steps, n_seq=n_seq)
    assert got.shape == (n_seq, steps) and sec > 0
    got2, logits = g.decode_greedy_batch(prompts, steps, n_seq=n_seq, want_logits=True)   # (the same buffers and graph again)
    np.testing.assert_array_equal(got2, got)
    for b in range(n_seq):
        p = prompts[b] if b < len(prompts) else np.zeros(0, dtype=np.int32)
        g.reset()
        want, _ = g.decode_greedy(p, steps)          # stops after token 1; the batch runs on
        same_until_a_tie(got[b, :len(want)], want, logits[:, b], "sequence %d" % b)
        np.testing.assert_array_equal(got[b, :len(p)], p)
    # every sequence against the oracle as well: its tokens, and the logits of every step
    m = oracle_of(orc, shape, 9)
    worst = 0.0
    for b in range(n_seq):
        p = prompts[b] if b < len(prompts) else np.zeros(0, dtype=np.int32)
        worst = max(worst, check_against_oracle(m, p, steps, got[b], logits[:, b], "sequence %d against the oracle" % b))
    print("batched logits vs oracle: worst max|d|/max|logit| = %.3g over %d sequences x %d steps" % (worst, n_seq, steps), flush=True)
    # the context's own cache and loop state are untouched: a single decode after the batch is what it was before
    g.reset()
    again, _ = g.decode_greedy(prompts[0], steps)
    np.testing.assert_array_equal(again, got[0, :len(again)])
    m.close(); g.close()


@pytest.mark.parametrize("shape,n_seq,steps", [
    ((4096, 11008, 3, 32, 32, 32000, 48, 0), 32, 40),      # the widths of Llama-2-7B: rows of 16 and 43 groups
    ((4096, 11008, 3, 32, 32, 32000, 48, 0), 16, 40),
    ((8192, 28672, 2, 64, 8, 32000, 32, 0), 32, 24),       # the widths of Llama-2-70B: 64 heads on 8 kv heads, rows of 32 and 112 groups
])
def test_published_widths_match_the_single_decode_and_the_oracle(orc, shape, n_seq, steps):
    """At the matrix sizes of the published models (a few layers of them) every sequence of a batch gets the tokens of its
    own single-sequence decode, and four of them (the first, two in the middle, the one without a prompt) the oracle's
    tokens and, step by step, its logits."""
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(21, 0.02)
    g.finalize()
    rng = np.random.default_rng(n_seq + shape[0])
    prompts = [rng.integers(2, shape[5], size=int(rng.integers(0, 7))).astype(np.int32) for _ in range(n_seq - 1)]
    got, logits = g.decode_greedy_batch(prompts, steps, n_seq=n_seq, want_logits=True)
    for b in range(n_seq):
        p = prompts[b] if b < len(prompts) else np.zeros(0, dtype=np.int32)
        g.reset()
        want, _ = g.decode_greedy(p, steps)
        np.testing.assert_array_equal(got[b, :len(want)], want, err_msg="sequence %d" % b)
    g.close()
    m = oracle_of(orc, shape, 21)
    worst = 0.0
    for b in (0, n_seq // 3, n_seq // 2 + 1, n_seq - 1):
        p = prompts[b] if b < len(prompts) else np.zeros(0, dtype=np.int32)
        worst = max(worst, check_against_oracle(m, p, steps, got[b], logits[:, b], "sequence %d against the oracle" % b))
    print("batched logits vs oracle at widths %s: worst max|d|/max|logit| = %.3g" % (shape[:2], worst), flush=True)
    m.close()


def test_buffers_and_graph_are_kept_between_calls_and_replaced_when_they_do_not_fit():
    """The context owns the batched path's buffers: a second call with fewer steps and other prompts runs in them (other
    strides than its own arguments'), a call with more steps or another sequence count replaces them."""
    shape = (512, 1024, 2, 8, 2, 1008, 96, 0)
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(5, 0.02)
    g.finalize()
    rng = np.random.default_rng(11)
    for n_seq, steps, longest in ((32, 48, 9), (32, 20, 4), (32, 64, 12), (16, 30, 6), (16, 30, 1)):
        prompts = [rng.integers(2, shape[5], size=int(rng.integers(0, longest + 1))).astype(np.int32) for _ in range(n_seq)]
        got, _ = g.decode_greedy_batch(prompts, steps, n_seq=n_seq)
        for b in (0, 1, n_seq - 1):
            g.reset()
            want, _ = g.decode_greedy(prompts[b], steps)
            np.testing.assert_array_equal(got[b, :len(want)], want, err_msg="%d sequences, %d steps, sequence %d" % (n_seq, steps, b))
    g.close()


def test_a_new_upload_replaces_the_tile_ordered_copy():
    """The batched products read a second copy of the matrices; uploading a tensor again must not leave the old copy in use."""
    shape = (512, 1024, 1, 8, 8, 1008, 16, 1)
    g = l2j.Transformer(l2j.Config(*shape))
    rng = np.random.default_rng(3)
    x = rng.standard_normal((16, 512)).astype(np.float32)
    for seed in (1, 2):
        g.fill_synthetic(seed, 0.02)      # (uploads are legal until finalize; the product does not need a finalized context)
        got, _ = g.batch_matmul(TENSOR.WQ, 0, x, 512)
        want = x.astype(np.float64) @ dequantized(g, TENSOR.WQ, 0, 512, 512).T
        assert (np.abs(got - want).max(axis=1) / np.abs(want).max(axis=1)).max() < 5e-6, seed
    g.close()


def test_shapes_the_batched_path_does_not_take_are_an_error():
    g = l2j.Transformer(l2j.Config(288, 768, 1, 6, 6, 320, 16, 1))   # rows of 288 codes: groups straddle rows
    g.fill_synthetic(1, 0.02)
    g.finalize()
    with pytest.raises(L2JError) as e:
        g.decode_greedy_batch([np.array([5, 6], dtype=np.int32)], 8)
    assert e.value.code == -2
    with pytest.raises(L2JError):
        g.batch_matmul(TENSOR.WQ, 0, np.zeros((16, 288), dtype=np.float32), 288)
    assert len(g.decode_greedy(np.array([5, 6], dtype=np.int32), 8)[0]) > 0     # the context stays usable
    g.close()


def test_sequence_counts_other_than_16_and_32_are_an_error():
    g = l2j.Transformer(l2j.Config(512, 1024, 1, 8, 8, 1008, 16, 1))
    g.fill_synthetic(1, 0.02)
    g.finalize()
    for n_seq in (1, 8, 17, 48, 64):
        with pytest.raises(L2JError) as e:
            g.decode_greedy_batch([np.array([5], dtype=np.int32)], 4, n_seq=n_seq)
        assert e.value.code == -1
    g.close()


@pytest.mark.parametrize("n_seq,t,topp,vocab", [(16, 0.9, 0.9, 1008), (32, 1.0, 1.0, 1008), (32, 1.3, 0.6, 1008), (32, 1.0, 0.9, 32000),
                                                (16, 0.7, 1.0, 32000)])
def test_sampled_batch_gives_every_sequence_its_own_sampler(orc, n_seq, t, topp, vocab):
    """l2j_decode_sample_batch: sequence b must get what the reference's loop with a Sampler(seed b) gives it (J/Run.java:623-685,
    J/Sampler.java).  The oracle's sampler is fed the batched path's own logits of every step (they agree with the oracle's
    forward pass to rounding only, and a draw within that of a step of the cumulative sum would part two correct runs):
    every token identical; and the logits of a step must be those of the tokens sampled before it, which the
    single-sequence forward pass, fed the sampled tokens, confirms."""
    from tests.test_gpu_parity import make_pair
    shape = SHAPES[0][:5] + (vocab,) + SHAPES[0][6:]    # (32000: a sampling step takes 125 compute units, two of them run side by side)
    m, g = make_pair(orc, shape, seed=17, realistic=True)
    rng = np.random.default_rng(n_seq)
    steps = 28 if vocab < 10000 else 14
    prompts = [rng.integers(3, vocab, size=int(rng.integers(0, 7))).astype(np.int32) for _ in range(n_seq - 2)]   # (two run without one)
    seeds = rng.integers(-2**40, 2**40, size=n_seq).astype(np.int64)
    got, sec, logits = g.decode_sample_batch(prompts, steps, t, topp, seeds, n_seq=n_seq, want_logits=True)
    assert got.shape == (n_seq, steps) and sec > 0
    for b in range(n_seq):
        prompt = prompts[b] if b < len(prompts) else np.zeros(0, dtype=np.int32)
        s = orc.Sampler(int(seeds[b]), vocab)
        want = [int(prompt[pos]) if pos < len(prompt) else s.step(logits[pos, b], t, topp)[0] for pos in range(steps)]
        np.testing.assert_array_equal(got[b], np.array(want, dtype=np.int32), err_msg="sequence %d" % b)
    for b in (0, n_seq - 1):                                     # the sampled tokens are what the next step reads
        g.reset()
        tok = 1
        for pos in range(steps):
            lg = g.forward(tok, pos)
            assert rel_err(logits[pos, b], lg.astype(np.float64)) < 1e-5, (b, pos)
            tok = int(got[b, pos])
    again, _ = g.decode_sample_batch(prompts, steps, t, topp, seeds, n_seq=n_seq)      # the seeds restart generators and arrays
    np.testing.assert_array_equal(again, got)
    other, _ = g.decode_sample_batch(prompts, steps, t, topp, seeds + 1, n_seq=n_seq)
    assert not np.array_equal(other, got)
    greedy, _ = g.decode_greedy_batch(prompts, steps, n_seq=n_seq)
    cold, _ = g.decode_sample_batch(prompts, steps, 0.0, topp, seeds, n_seq=n_seq)     # temperature 0: Sampler.argmax
    np.testing.assert_array_equal(cold, greedy)
    g.close()


def test_sampled_batch_refuses_what_its_sampling_step_cannot_take():
    g = l2j.Transformer(l2j.Config(*SHAPES[3]))
    g.fill_synthetic(3, 0.02)
    g.finalize()
    p = [np.array([5, 6], dtype=np.int32)]
    with pytest.raises(L2JError):
        g.decode_sample_batch(p, 8, -1.0, 0.9, [1])
    with pytest.raises(L2JError):
        g.decode_sample_batch(p, 8, 1.0, 1.5, [1])
    g.set_option("sampler_scan", 0)
    with pytest.raises(L2JError, match="sampler_scan"):
        g.decode_sample_batch(p, 8, 1.0, 0.9, [1])
    g.set_option("sampler_scan", 1)
    g.set_option("sampler_wide", 0)                      # (the one-launch step of the single sequence: not what the batch takes)
    out, _ = g.decode_sample_batch(p, 8, 1.0, 0.9, [1])
    assert out.shape == (16, 8) and np.array_equal(out[0, :2], p[0])
    g.close()


def test_the_sampling_steps_of_the_batch_wait_for_nobody():
    """barrier_spins 0 makes every bounded wait between workgroups give up at once; the batch's sampling steps have none (a
    launch per stage, the sequences side by side in each): the tokens of a context with the default."""
    shape = SHAPES[0]
    outs = []
    for spins in (None, 0):
        g = l2j.Transformer(l2j.Config(*shape))
        g.fill_synthetic(5, 0.02)
        if spins is not None:
            g.set_option("barrier_spins", spins)
        g.finalize()
        out, _ = g.decode_sample_batch([np.array([9, 8, 7], dtype=np.int32)], 12, 1.0, 0.9, [3])
        outs.append(out)
        g.close()
    np.testing.assert_array_equal(outs[0], outs[1])


def test_release_batch_gives_the_memory_back_and_the_next_call_makes_it_again():
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = C.c_size_t(0), C.c_size_t(0)
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    shape = SHAPES[2]
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(11, 0.02)
    g.finalize()
    prompts = [np.array([5, 9, 13], dtype=np.int32), np.array([7], dtype=np.int32)]
    single, _ = g.decode_greedy(prompts[0], 24)
    g.reset()
    g.release_batch()                                  # (nothing to release yet: not an error)
    before = free_bytes()
    want, _ = g.decode_greedy_batch(prompts, 24)
    sampled, _ = g.decode_sample_batch(prompts, 24, 0.9, 0.9, [1, 2])
    tokens = np.concatenate([[1], prompts[0], np.arange(20, 40)]).astype(np.int32)
    logits, _ = g.prefill(tokens)
    held = before - free_bytes()
    assert held > 10 << 20                             # the copy of the matrices, caches, buffers, samplers
    g.release_batch()
    assert abs(free_bytes() - before) <= 4 << 20
    g.reset()
    again, _ = g.decode_greedy_batch(prompts, 24)
    np.testing.assert_array_equal(again, want)
    np.testing.assert_array_equal(g.decode_sample_batch(prompts, 24, 0.9, 0.9, [1, 2])[0], sampled)
    g.reset()
    np.testing.assert_array_equal(g.prefill(tokens)[0].view(np.uint32), logits.view(np.uint32))
    g.reset()
    np.testing.assert_array_equal(g.decode_greedy(prompts[0], 24)[0], single)   # the single-sequence path: untouched
    g.close()
