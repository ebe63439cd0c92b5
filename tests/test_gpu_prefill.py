"""l2j_prefill: the prompt positions of the token loop (J/Run.java:623-640, one Run.transformer call per position in the
reference) 32 at a time through the batched products.  It must leave in the KV cache, and return for the last position,
what l2j_forward position by position does (to rounding: the sums are formed in another order), and both must be what the
CPU oracle computes."""
import numpy as np
import pytest

import llama2j_amd as l2j
from llama2j_amd.binding import BUFFER, L2JError
from tests.test_gpu_batch import LOGIT_TOL, oracle_of, rel_err

pytestmark = pytest.mark.gpu

SHAPES = [
    (512, 1024, 4, 8, 8, 1008, 80, 1),      # head 64, shared classifier
    (512, 1024, 2, 8, 2, 1008, 72, 0),      # grouped-query attention: 8 heads on 2 kv heads
    (1024, 2816, 2, 8, 4, 2000, 96, 0),     # head 128, an odd number of groups per row
    (512, 768, 2, 2, 2, 512, 40, 1),        # head 256
]
CLOSE = 2e-5   # prefill against l2j_forward: relative to the largest value of what is compared


def model(shape, seed=9):
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(seed, 0.02)
    g.finalize()
    return g


def caches(g, shape):
    return [np.stack([g.read(which, layer) for layer in range(shape[2])]) for which in (BUFFER.KCACHE, BUFFER.VCACHE)]


@pytest.mark.parametrize("flash", [2, 0])    # the attention on the matrix cores at every position / at none (default: from position 64 on)
@pytest.mark.parametrize("shape", SHAPES)
def test_prefill_leaves_what_forward_position_by_position_leaves(orc, shape, flash):
    seq_len, kvd = shape[6], shape[0] // shape[3] * shape[4]
    rng = np.random.default_rng(shape[0] + shape[6])
    g = model(shape)
    g.set_option("prefill_flash", flash)
    m = oracle_of(orc, shape, 9)
    for n in (1, 31, 32, 33, seq_len):
        tokens = np.concatenate([[1], rng.integers(2, shape[5], size=n - 1)]).astype(np.int32)   # BOS first (J/Run.java:612)
        g.reset()
        for i, t in enumerate(tokens):
            want_logits = g.forward(int(t), i)
        want_k, want_v = caches(g, shape)
        g.reset()
        got_logits, sec = g.prefill(tokens)
        got_k, got_v = caches(g, shape)
        assert sec > 0
        assert rel_err(got_logits, want_logits.astype(np.float64)) < CLOSE, n
        for got, want in ((got_k, want_k), (got_v, want_v)):
            got, want = got.reshape(shape[2], seq_len, kvd), want.reshape(shape[2], seq_len, kvd)
            assert rel_err(got[:, :n], want[:, :n].astype(np.float64)) < CLOSE, n
            assert not got[:, n:].any(), n                      # rows past the last position: untouched
        # and the oracle, from the same tokens: the logits of the last position within the bar
        m.reset()
        for i, t in enumerate(tokens):
            oracle_logits = m.forward(int(t), i)
        assert rel_err(got_logits, oracle_logits.astype(np.float64)) < LOGIT_TOL, n
    m.close()


@pytest.mark.parametrize("shape", SHAPES[:2])
def test_prefill_goes_on_from_a_position_and_decode_goes_on_from_prefill(orc, shape):
    seq_len = shape[6]
    rng = np.random.default_rng(shape[6])
    g = model(shape)
    n1, n2, more = 17, 40, 8
    tokens = np.concatenate([[1], rng.integers(2, shape[5], size=n1 + n2 - 1)]).astype(np.int32)
    g.reset()
    whole, _ = g.prefill(tokens)
    k_whole, v_whole = caches(g, shape)
    g.reset()
    g.prefill(tokens[:n1], want_logits=False)
    parts, _ = g.prefill(tokens[n1:], pos0=n1)
    k_parts, v_parts = caches(g, shape)
    assert rel_err(parts, whole.astype(np.float64)) < CLOSE
    assert rel_err(k_parts, k_whole.astype(np.float64)) < CLOSE and rel_err(v_parts, v_whole.astype(np.float64)) < CLOSE
    # the single-sequence path continues on the cache prefill has left: the logits of the next positions against a run
    # that took every position through l2j_forward
    nxt = rng.integers(2, shape[5], size=more).astype(np.int32)
    after_prefill = [g.forward(int(t), n1 + n2 + i) for i, t in enumerate(nxt)]
    g.reset()
    for i, t in enumerate(np.concatenate([tokens, nxt])):
        lg = g.forward(int(t), i)
        if i >= n1 + n2:
            assert rel_err(after_prefill[i - n1 - n2], lg.astype(np.float64)) < CLOSE, i
    assert n1 + n2 + more <= seq_len


def test_prefill_refuses_what_it_cannot_take(orc):
    g = model(SHAPES[0])
    with pytest.raises(L2JError):
        g.prefill(np.array([1, 5000], dtype=np.int32))          # token id beyond the vocabulary
    with pytest.raises(L2JError):
        g.prefill(np.ones(4, dtype=np.int32), pos0=SHAPES[0][6] - 2)   # past seq_len
    small = l2j.Transformer(l2j.Config(64, 128, 2, 4, 4, 512, 32, 1))       # dim not in whole groups of 256
    small.fill_synthetic(3, 0.1)
    small.finalize()
    with pytest.raises(L2JError):
        small.prefill(np.array([1, 2, 3], dtype=np.int32))


@pytest.mark.parametrize("shape,n_prompt", [(SHAPES[0], 40), (SHAPES[1], 65), (SHAPES[2], 33)])
def test_decode_loops_with_option_prefill_give_the_tokens_they_give_without(orc, shape, n_prompt):
    """Option prefill: the loops take the first whole steps of 32 prompt positions through l2j_prefill and go on from there.
    Greedy against the CPU oracle's loop as well; sampled with the same seed."""
    steps = shape[6]
    prompt = orc.synth_prompt(5, n_prompt, shape[5])
    g = model(shape)
    want, _ = g.decode_greedy(prompt, steps)
    want_s, _ = g.decode_sample(prompt, steps, 0.9, 0.9, 11)
    g.set_option("prefill", 1)
    g.reset()
    got, sec = g.decode_greedy(prompt, steps)
    assert sec > 0
    np.testing.assert_array_equal(got, want)
    g.reset()
    got_s, _ = g.decode_sample(prompt, steps, 0.9, 0.9, 11)
    np.testing.assert_array_equal(got_s, want_s)
    m = oracle_of(orc, shape, 9)
    cpu, _, _ = m.generate_greedy(prompt, steps)
    np.testing.assert_array_equal(got[:len(cpu)], cpu)
    m.close()
    # a prompt id 1 among the first 32 ends the loop there, as without the option
    stop = prompt.copy()
    stop[7] = 1
    g.reset()
    got, _ = g.decode_greedy(stop, steps)
    assert len(got) == 8 and got[-1] == 1


@pytest.mark.parametrize("shape,n", [
    ((4096, 11008, 3, 32, 32, 32000, 48, 0), 45),      # the widths of Llama-2-7B (three layers of it)
    ((8192, 28672, 2, 64, 8, 32000, 40, 0), 37),       # the widths of Llama-2-70B: 64 heads on 8 kv heads
])
def test_prefill_at_the_published_widths(orc, shape, n):
    rng = np.random.default_rng(n)
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(21, 0.02)
    g.finalize()
    g.set_option("prefill_flash", 2)
    tokens = np.concatenate([[1], rng.integers(2, shape[5], size=n - 1)]).astype(np.int32)
    for i, t in enumerate(tokens):
        want = g.forward(int(t), i)
    g.reset()
    got, _ = g.prefill(tokens)
    assert rel_err(got, want.astype(np.float64)) < CLOSE
    g.close()
    m = oracle_of(orc, shape, 21)
    for i, t in enumerate(tokens):
        cpu = m.forward(int(t), i)
    worst = rel_err(got, cpu.astype(np.float64))
    print("prefill logits vs oracle at widths %s: max|d|/max|logit| = %.3g" % (shape[:2], worst), flush=True)
    assert worst < LOGIT_TOL
    m.close()


def test_prefill_and_the_batched_decode_share_their_buffers(orc):
    """Both run in the context's batch buffers (32 rows for prefill): calls of either kind in any order give what they give alone."""
    shape = SHAPES[1]
    g = model(shape)
    rng = np.random.default_rng(3)
    tokens = np.concatenate([[1], rng.integers(2, shape[5], size=44)]).astype(np.int32)
    prompts = [rng.integers(2, shape[5], size=3).astype(np.int32) for _ in range(16)]
    alone_logits, _ = g.prefill(tokens)
    alone_tokens, _ = g.decode_greedy_batch(prompts, 24, n_seq=16)        # (buffers for 16 sequences replace prefill's)
    g.reset()
    again_logits, _ = g.prefill(tokens)                                   # (and prefill's replace those)
    assert np.array_equal(again_logits.view(np.uint32), alone_logits.view(np.uint32))
    again_tokens, _ = g.decode_greedy_batch(prompts + prompts, 24, n_seq=32)
    np.testing.assert_array_equal(again_tokens[:16], alone_tokens)
    g.reset()
    third, _ = g.prefill(tokens)                                          # (in the buffers of the 32 sequences)
    assert np.array_equal(third.view(np.uint32), alone_logits.view(np.uint32))


def test_prefill_past_the_position_where_the_attention_changes_kernels(orc):
    """By default the attention of a step runs on the matrix cores from position 64 on, and from position 192 on the keys of a
    head are split over several workgroups: a prompt that crosses both, against position-by-position forwards and the oracle."""
    shape = (512, 1024, 2, 8, 2, 1008, 480, 0)
    rng = np.random.default_rng(640)
    g = model(shape)
    n = 470
    tokens = np.concatenate([[1], rng.integers(2, shape[5], size=n - 1)]).astype(np.int32)
    for i, t in enumerate(tokens):
        want = g.forward(int(t), i)
    want_k, want_v = caches(g, shape)
    g.reset()
    got, _ = g.prefill(tokens)
    got_k, got_v = caches(g, shape)
    assert rel_err(got, want.astype(np.float64)) < CLOSE
    assert rel_err(got_k, want_k.astype(np.float64)) < CLOSE and rel_err(got_v, want_v.astype(np.float64)) < CLOSE
    m = oracle_of(orc, shape, 9)
    for i, t in enumerate(tokens):
        cpu = m.forward(int(t), i)
    assert rel_err(got, cpu.astype(np.float64)) < LOGIT_TOL
    m.close()


@pytest.mark.parametrize("shape", SHAPES)
def test_the_keys_of_a_head_split_over_one_to_four_workgroups(shape):
    """Option prefill_split: as many workgroups share the keys of a head in the matrix-core attention, the last of them to finish
    merging what the others left (also where there are fewer tiles of 16 keys than workgroups): the logits and cache rows of
    position-by-position forwards, for every head size, and twice in a row (the counters of a launch are left at zero)."""
    seq_len = shape[6]
    rng = np.random.default_rng(seq_len)
    g = model(shape)
    g.set_option("prefill_flash", 2)
    tokens = np.concatenate([[1], rng.integers(2, shape[5], size=seq_len - 1)]).astype(np.int32)
    for i, t in enumerate(tokens):
        want = g.forward(int(t), i)
    want_k, want_v = caches(g, shape)
    for split in (4, 3, 2, 1, 4):
        g.set_option("prefill_split", split)
        g.reset()
        got, _ = g.prefill(tokens)
        got_k, got_v = caches(g, shape)
        assert rel_err(got, want.astype(np.float64)) < CLOSE, split
        assert rel_err(got_k, want_k.astype(np.float64)) < CLOSE and rel_err(got_v, want_v.astype(np.float64)) < CLOSE, split
    g.close()
