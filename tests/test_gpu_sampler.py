"""Device sampler (l2j_sampler_seed / l2j_sample / l2j_decode_sample) against the CPU oracle's restatement of
J/Sampler.java and J/Run.java:643-665, through the C ABI: the sampled tokens must be identical, the
probabilities left in the logits buffer equal to float32 rounding of the exponential."""
import numpy as np
import pytest

import llama2j_amd as l2j
from llama2j_amd.binding import BUFFER, L2JError

pytestmark = pytest.mark.gpu


def small_transformer(vocab, seed=3):
    g = l2j.Transformer(l2j.Config(32, 64, 1, 2, 2, vocab, 8, 1))
    g.fill_synthetic(seed, 0.1)
    g.finalize()
    return g


def logits_of(rng, n, kind):
    x = rng.standard_normal(n).astype(np.float32)
    if kind == "flat":
        return x * np.float32(0.05)
    if kind == "peaked":
        x = x * np.float32(4.0)
        x[rng.integers(0, n)] += np.float32(12.0)
        return x
    return x * np.float32(2.0)


def check_probabilities(got, want):
    # the only operation that may differ is the last bit of the double exponential before it is narrowed
    assert np.abs(got - want).max() <= 2e-7 * want.max(), np.abs(got - want).max()


# sampler_wide 1 (the default): the sampling step is one launch over many workgroups; 0: one launch per stage
WIDE = pytest.mark.parametrize("wide", ["1", "0"])


@WIDE
@pytest.mark.parametrize("vocab", [1003, 32000])
def test_plain_sampling_matches_oracle(orc, monkeypatch, vocab, wide):
    monkeypatch.setenv("L2J_SAMPLER_WIDE", wide)
    g = small_transformer(vocab)
    rng = np.random.default_rng(vocab)
    g.sampler_seed(77)
    o = orc.Sampler(77, vocab)
    for call, kind in enumerate(["mid", "flat", "peaked", "mid", "flat", "peaked"]):
        lg = logits_of(rng, vocab, kind)
        t = float(rng.choice([0.5, 0.9, 1.0, 1.7]))
        want, probs = o.step(lg, t, 1.0)                       # topp > 0.999: Sampler.sample
        assert g.sample(t, 1.0, logits=lg) == want, (call, kind)
        got = g.read(BUFFER.LOGITS)
        check_probabilities(got, probs)
        for coin in (0.0, 0.3, 0.99999994, float(np.float32(rng.random()))):
            assert g.sample(t, 1.0, logits=lg, coin=coin) == o.sample(got, coin=coin), (call, kind, coin)


@WIDE
@pytest.mark.parametrize("vocab", [1003, 32000])
def test_topp_sequence_matches_oracle_including_entries_of_earlier_calls(orc, monkeypatch, vocab, wide):
    monkeypatch.setenv("L2J_SAMPLER_WIDE", wide)
    g = small_transformer(vocab)
    rng = np.random.default_rng(vocab + 1)
    g.sampler_seed(-12345)
    o = orc.Sampler(-12345, vocab)
    kinds = ["flat", "peaked", "mid", "peaked", "flat", "mid", "peaked", "peaked", "flat", "mid"] * 2
    for call, kind in enumerate(kinds):
        lg = logits_of(rng, vocab, kind)
        t = float(rng.choice([0.7, 0.9, 1.0]))
        topp = float(rng.choice([0.5, 0.9, 0.95, 0.99]))
        want, probs = o.step(lg, t, topp)
        assert g.sample(t, topp, logits=lg) == want, (call, kind, topp)
        check_probabilities(g.read(BUFFER.LOGITS), probs)


@WIDE
@pytest.mark.parametrize("vocab", [255, 4097, 32000, 70001])
def test_topp_with_many_equal_probabilities_keeps_the_stable_order(orc, monkeypatch, vocab, wide):
    # logits on a coarse grid: thousands of equal probabilities, inside tiles, across tiles and across runs of the sort,
    # and among the entries that earlier calls left behind; Arrays.sort is stable, so their order is the array's
    monkeypatch.setenv("L2J_SAMPLER_WIDE", wide)
    g = small_transformer(vocab)
    rng = np.random.default_rng(vocab + 7)
    g.sampler_seed(3)
    o = orc.Sampler(3, vocab)
    for call in range(12):
        step = float(rng.choice([0.25, 0.5, 1.0]))
        lg = (np.round(rng.standard_normal(vocab) * 2.0 / step) * step).astype(np.float32)
        topp = float(rng.choice([0.3, 0.8, 0.95, 0.99]))
        want, probs = o.step(lg, 1.0, topp)
        assert g.sample(1.0, topp, logits=lg) == want, (call, step, topp)
        check_probabilities(g.read(BUFFER.LOGITS), probs)


@WIDE
@pytest.mark.parametrize("vocab", [2, 3, 64, 256, 257, 512, 4096, 8193])
def test_vocabularies_at_the_edges_of_slices_tiles_and_runs(orc, monkeypatch, vocab, wide):
    """A slice of the one-launch step and a tile of the sort hold 256 probabilities, a run 4096: vocabularies of exactly
    one, one more, and the smallest there are; top-p and plain calls mixed, so entries of earlier calls take part."""
    monkeypatch.setenv("L2J_SAMPLER_WIDE", wide)
    g = small_transformer(vocab)
    rng = np.random.default_rng(vocab * 7 + 1)
    g.sampler_seed(vocab)
    o = orc.Sampler(vocab, vocab)
    for call in range(10):
        lg = logits_of(rng, vocab, ("flat", "peaked", "mid")[call % 3])
        t = float(rng.choice([0.6, 0.9, 1.3]))
        topp = float(rng.choice([0.4, 0.9, 0.97, 1.0]))
        want, probs = o.step(lg, t, topp)
        assert g.sample(t, topp, logits=lg) == want, (call, topp)
        check_probabilities(g.read(BUFFER.LOGITS), probs)


def test_topp_worked_example_with_entries_of_an_earlier_call(orc):
    # the hand-worked case of the oracle's tests, on the device: eight tokens, padded with impossible ones
    vocab = 16
    g = small_transformer(vocab)
    g.sampler_seed(1)
    o = orc.Sampler(1, vocab)
    with np.errstate(divide="ignore"):
        u = np.log(np.array([0.125] * 8 + [0.0] * 8, dtype=np.float32))
        p = np.log(np.array([0.9, 0.04, 0.03, 0.01, 0.01, 0.005, 0.0025, 0.0025] + [0.0] * 8, dtype=np.float32))
    for lg, topp, coin in ((u, 0.5, 0.0), (p, 0.95, 0.95), (p, 0.95, 0.2), (u, 0.9, 0.7)):
        _, probs = o.step(lg, 1.0, 1.0)
        assert g.sample(1.0, topp, logits=lg, coin=coin) == o.sample_topp(probs, topp, coin=coin)


def running_sum_cases():
    rng = np.random.default_rng(11)
    n = 32000
    yield "uniform", rng.random(n)
    yield "flat softmax", np.exp(rng.standard_normal(n) * 0.05)
    yield "peaked softmax", np.exp(rng.standard_normal(n) * 6 - 20)
    yield "forty orders of magnitude", np.exp(rng.uniform(-80, 5, n))
    yield "sorted descending", np.sort(rng.random(n) / n)[::-1]
    yield "powers of two (ties)", np.ldexp(1.0, rng.integers(-30, 3, n))
    yield "3 * powers of two (ties)", 3 * np.ldexp(1.0, rng.integers(-30, 3, n))
    yield "halves", np.full(n, 0.5)
    yield "ones, then terms of half an ulp and of three quarters", np.concatenate(
        [np.ones(9000), np.full(9000, 2.0 ** -11), np.full(9000, 1.5 * 2.0 ** -11)])
    yield "denormals", np.concatenate([np.full(3000, 1e-45), np.full(3000, 1e-40), rng.random(3000) * 1e-38])
    yield "half of them zero", np.where(rng.random(n) < 0.5, 0.0, rng.random(n))
    yield "leading zeros", np.concatenate([np.zeros(5000), rng.random(5000)])
    yield "every term leaves the binade", np.ldexp(1.0, np.arange(-100, 100))
    yield "a large term late", np.concatenate([rng.random(20000) * 1e-3, [1e6], rng.random(5000)])
    for m in (1, 2, 31, 32, 33, 63, 64, 65, 1023, 1024, 1025, 3071, 3072, 3073, 1024 + 8192, 1024 + 8193, 36863, 36864):
        yield "n = %d" % m, rng.random(m)
    # sums that stay next to a power of two for thousands of terms, where a guessed binade is easily wrong
    for k in range(3):
        x = rng.standard_normal(n) * (1 + 3 * k)
        x[rng.integers(0, n)] += 8 + 4 * k
        e = np.exp((x - x.max()).astype(np.float32).astype(np.float64)).astype(np.float32)
        pr = e / np.cumsum(e, dtype=np.float32)[-1]
        yield "peaked exponentials %d" % k, e
        yield "peaked probabilities %d" % k, pr
        yield "peaked probabilities, sorted descending %d" % k, np.sort(pr)[::-1]
    yield "one, then tiny terms", np.concatenate([[1.0], np.full(n - 1, 1e-9)])
    yield "just below one, then terms of 3e-8", np.concatenate([rng.random(500) * 1e-3, [0.75], np.full(31000, 3e-8)])
    yield "an infinity", np.concatenate([rng.random(700), [np.inf], rng.random(700)])
    # more terms than fit in LDS: the sums are formed in device memory
    for m in (36865, 50257, 131072, 200003):
        yield "n = %d" % m, rng.random(m)
    yield "n = 151936, peaked", np.exp(rng.standard_normal(151936) * 5 - 12)


@pytest.mark.parametrize("scan", ["1", "0"])
def test_running_sums_are_the_sequential_float32_sums(orc, monkeypatch, scan):
    # numpy's cumsum adds one element after the other in float32: the order of the reference's loops
    monkeypatch.setenv("L2J_SAMPLER_SCAN", scan)
    g = small_transformer(64)
    for name, terms in running_sum_cases():
        with np.errstate(over="ignore", invalid="ignore"):
            terms = np.asarray(terms, dtype=np.float32)
            want = np.cumsum(terms, dtype=np.float32)
        got = g.running_sums(terms)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (name, int(np.argmax(got != want)))


def test_the_one_launch_step_forms_the_sequential_sums_and_finds_where_they_pass_a_limit(orc):
    """l2j_sum_probe asks the walk of the one-launch sampling step what the sampler asks it: the sum of all terms, and the
    first index whose running sum exceeds a limit with that sum; numpy's float32 cumsum is the reference's loop."""
    g = small_transformer(64)
    rng = np.random.default_rng(23)
    for name, terms in running_sum_cases():
        with np.errstate(over="ignore", invalid="ignore"):
            terms = np.asarray(terms, dtype=np.float32)
            if terms.size > 36864:
                continue
            c = np.cumsum(terms, dtype=np.float32)
            at = np.unique(np.concatenate([[0, terms.size - 1], rng.integers(0, terms.size, 150),
                                           np.flatnonzero(np.diff(np.frexp(c)[1]))[:40]]))   # (also where the sum changes binade)
            limits = np.concatenate([[0.0], c[at], np.nextafter(c[at], np.float32(-np.inf)), c[-1:] * 2 + 1]).astype(np.float32)
            limits = limits[np.isfinite(limits) & (limits >= 0)]
            idx, s, total = g.sum_probe(terms, limits)
            assert np.float32(total).view(np.uint32) == c[-1].view(np.uint32), (name, total, c[-1])
            for q, lim in enumerate(limits):
                over = np.flatnonzero(c > lim)
                want = int(over[0]) if over.size else -1
                assert idx[q] == want, (name, q, float(lim), int(idx[q]), want)
                if want >= 0:
                    assert s[q].view(np.uint32) == c[want].view(np.uint32), (name, q, float(lim), want)


@pytest.mark.parametrize("topp", [1.0, 0.9, 0.5])
def test_one_launch_and_launch_per_stage_pick_the_same_tokens(orc, monkeypatch, topp):
    vocab = 32000
    rng = np.random.default_rng(15)
    calls = [(logits_of(rng, vocab, kind), float(np.float32(rng.random()))) for kind in ("flat", "peaked", "mid", "peaked", "flat", "mid")]
    seen = []
    for wide in ("1", "0"):
        monkeypatch.setenv("L2J_SAMPLER_WIDE", wide)
        g = small_transformer(vocab)
        g.sampler_seed(4)
        out = []
        for lg, coin in calls:
            out.append((g.sample(0.9, topp, logits=lg, coin=coin), g.sample(0.9, topp, logits=lg), g.read(BUFFER.LOGITS).view(np.uint32)))
        seen.append(out)
    for a, b in zip(*seen):
        assert a[0] == b[0] and a[1] == b[1] and np.array_equal(a[2], b[2])


@pytest.mark.parametrize("topp", [1.0, 0.9])
def test_scanned_and_single_lane_sums_pick_the_same_tokens(orc, monkeypatch, topp):
    vocab = 32000
    g = small_transformer(vocab)
    rng = np.random.default_rng(5)
    for kind in ("flat", "peaked", "mid"):
        lg = logits_of(rng, vocab, kind)
        for coin in [0.0, 0.99999994] + [float(np.float32(c)) for c in rng.random(6)]:
            picks, probs = [], []
            for scan in ("1", "0"):
                monkeypatch.setenv("L2J_SAMPLER_SCAN", scan)
                g.sampler_seed(9)                    # (top-p keeps entries of earlier calls: the same history for both)
                picks.append(g.sample(0.9, topp, logits=lg, coin=coin))
                probs.append(g.read(BUFFER.LOGITS))
            assert picks[0] == picks[1], (kind, coin)
            assert np.array_equal(probs[0].view(np.uint32), probs[1].view(np.uint32)), kind


def test_temperature_zero_is_first_max_and_nan_is_an_error(orc):
    vocab = 1003
    g = small_transformer(vocab)
    lg = np.zeros(vocab, dtype=np.float32)
    lg[[17, 500, 900]] = 3.0
    assert g.sample(0.0, 0.9, logits=lg) == 17
    lg[5] = np.nan
    with pytest.raises(L2JError):
        g.sample(0.9, 0.9, logits=lg)
    lg[5] = 0.0
    assert g.sample(0.9, 0.9, logits=lg, coin=0.0) in (17, 500, 900)   # the context stays usable
    with pytest.raises(L2JError):                                      # flat distribution, topp 0: no candidate
        g.sample(1.0, 0.0, logits=np.zeros(vocab, dtype=np.float32))
    assert g.sample(1.0, 0.0, logits=lg, coin=0.9) == 17               # ties keep index order; cumulative > 0 at once


def test_a_wait_of_the_one_launch_step_that_runs_out_is_an_error_and_the_context_falls_back(orc):
    """barrier_spins 0: the first workgroup to reach a grid barrier gives up at once (every kernel still runs to its end).
    The call fails, the context then samples with one launch per stage, and a newly seeded sampler gives the oracle's tokens."""
    vocab = 1003
    g = l2j.Transformer(l2j.Config(32, 64, 1, 2, 2, vocab, 8, 1))
    g.fill_synthetic(3, 0.1)
    g.set_option("barrier_spins", 0)
    g.finalize()
    assert g.get_option("sampler_wide") == 1
    rng = np.random.default_rng(4)
    lg = logits_of(rng, vocab, "mid")
    g.sampler_seed(6)
    with pytest.raises(L2JError):
        g.sample(0.9, 0.9, logits=lg)
    assert g.get_option("sampler_wide") == 0
    g.sampler_seed(6)
    o = orc.Sampler(6, vocab)
    for topp in (0.9, 1.0, 0.5):
        want, probs = o.step(lg, 0.9, topp)
        assert g.sample(0.9, topp, logits=lg) == want
        check_probabilities(g.read(BUFFER.LOGITS), probs)


def test_largest_vocabulary_the_sampler_takes(orc):
    vocab = 36864
    g = small_transformer(vocab)
    rng = np.random.default_rng(8)
    g.sampler_seed(5)
    o = orc.Sampler(5, vocab)
    for kind, topp in (("flat", 0.9), ("peaked", 0.95), ("mid", 1.0), ("flat", 1.0)):
        lg = logits_of(rng, vocab, kind)
        want, probs = o.step(lg, 0.9, topp)
        assert g.sample(0.9, topp, logits=lg) == want, (kind, topp)
        check_probabilities(g.read(BUFFER.LOGITS), probs)


@pytest.mark.parametrize("vocab", [36865, 50257, 70001, 131072])
def test_vocabularies_beyond_the_lds(orc, vocab):
    """Above 36864 entries the probabilities stay in device memory and the sort merges sixteen runs at a time (70001: a
    short last run at the second level; 131072: two full levels); the tokens are still the reference's."""
    g = small_transformer(vocab)
    rng = np.random.default_rng(vocab)
    g.sampler_seed(11)
    o = orc.Sampler(11, vocab)
    for kind, topp in (("flat", 0.9), ("peaked", 0.95), ("mid", 1.0), ("peaked", 0.5), ("flat", 1.0), ("mid", 0.99)):
        lg = logits_of(rng, vocab, kind)
        want, probs = o.step(lg, 0.9, topp)
        assert g.sample(0.9, topp, logits=lg) == want, (kind, topp)
        check_probabilities(g.read(BUFFER.LOGITS), probs)


@pytest.mark.parametrize("shape,steps,t,topp", [
    ((64, 128, 2, 4, 4, 512, 64, 1), 64, 1.0, 0.9),
    ((64, 128, 2, 4, 2, 512, 64, 0), 64, 0.9, 1.0),
    ((288, 768, 6, 6, 6, 32000, 256, 1), 72, 0.9, 0.9),
])
def test_decode_sample_matches_oracle_loop(orc, shape, steps, t, topp):
    """The device loop against the reference's loop with the oracle's sampler fed the logits of l2j_forward:
    every token must be identical.  (Against the all-CPU loop the tokens agree until a cumulative probability
    lands within the forward pass's 1e-7 logit difference of topp or of the draw -- once in 1e2 (vocabulary 32000,
    flat distribution) to 1e4 steps -- after which two correct samplers legitimately part ways; only the first
    sampled tokens are asserted there.)"""
    from tests.test_gpu_parity import make_pair
    m, g = make_pair(orc, shape, seed=31, realistic=True)
    prompt = orc.synth_prompt(31, 5, shape[5])
    got, sec = g.decode_sample(prompt, steps, t, topp, 2024)
    assert np.array_equal(got[:5], prompt) and sec > 0

    g.reset()
    s = orc.Sampler(2024, shape[5])
    tok, want = 1, []
    for pos in range(len(got)):                               # J/Run.java:623-685 driven from the host
        lg = g.forward(tok, pos)
        nxt = int(prompt[pos]) if pos < len(prompt) else s.step(lg, t, topp)[0]
        want.append(nxt)
        if nxt == 1:
            break
        tok = nxt
    assert np.array_equal(got, np.array(want, dtype=np.int32)), (got, want)

    cpu, _ = m.generate(prompt, steps, t, topp, 2024)
    assert np.array_equal(got[:8], cpu[:8])

    g.reset()
    again, _ = g.decode_sample(prompt, steps, t, topp, 2024)
    assert np.array_equal(again, got)                         # the seed restarts the generator and the array
    g.reset()
    greedy, _ = g.decode_greedy(prompt, steps)
    g.reset()
    same, _ = g.decode_sample(prompt, steps, 0.0, topp, 2024)
    assert np.array_equal(same, greedy)
