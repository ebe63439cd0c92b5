"""Pins the CPU oracle's sampler (J/Sampler.java, K/FindMax.java, J/Run.java:643-665) without the
reference running: published values of java.util.Random, numpy's sequential float32 cumsum, a
restatement of the ProbIndex object array with Python objects and Python's stable sort, and cases
worked by hand from the Java source (including the reference's whole-array sort, which lets entries
of an earlier call take part in a later one)."""
import numpy as np
import pytest


# ---------------------------------------------------------------- java.util.Random

def test_java_random_published_sequences(orc):
    # the first nextInt() values of new Random(42) and new Random(0), as printed by any JVM
    s = orc.Sampler(42, 4)
    assert [s.next_bits(32) for _ in range(4)] == [-1170105035, 234785527, -1360544799, 205897768]
    s = orc.Sampler(0, 4)
    assert [s.next_bits(32) for _ in range(4)] == [-1155484576, -723955400, 1033096058, -1690734402]


def test_java_random_next_float(orc):
    # nextFloat() = next(24) / 2^24: the top 24 of the 32 bits that nextInt() would have returned
    s = orc.Sampler(42, 4)
    f = s.next_float()
    assert f == np.float32(((-1170105035) & 0xFFFFFFFF) >> 8) / np.float32(1 << 24)
    assert repr(float(np.float32(f)))[:9] == "0.7275636"      # new Random(42).nextFloat() prints 0.7275637
    t = orc.Sampler(42, 4)
    t.next_bits(32)
    assert s.next_bits(32) == t.next_bits(32)                  # one draw advanced the state once
    for seed in (1, -7, 2**40 + 3, -2**62):
        s = orc.Sampler(seed, 4)
        v = [s.next_float() for _ in range(1000)]
        assert 0.0 <= min(v) and max(v) < 1.0
        assert all(x * (1 << 24) == int(x * (1 << 24)) for x in v)
        assert 0.45 < np.mean(v) < 0.55


# ---------------------------------------------------------------- FindMax, sample

def test_find_max(orc):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(1000).astype(np.float32)
    assert orc.find_max(x) == x.max()
    assert orc.find_max(np.array([-3.0], dtype=np.float32)) == -3.0
    assert orc.find_max(np.array([-3.0, -1.0, -2.0], dtype=np.float32)) == -1.0


def first_below(cdf, r):
    hit = np.nonzero(np.float32(r) < cdf)[0]
    return int(hit[0]) if hit.size else cdf.size - 1


@pytest.mark.parametrize("n", [1, 2, 7, 1000, 32000])
def test_sample_against_sequential_float32_cumsum(orc, n):
    rng = np.random.default_rng(n)
    p = rng.random(n).astype(np.float32)
    p /= p.sum(dtype=np.float32)
    cdf = np.cumsum(p, dtype=np.float32)      # accumulate runs left to right in float32
    s = orc.Sampler(1, n)
    for r in list(rng.random(50).astype(np.float32)) + [0.0, float(cdf[-1]), 0.99999994]:
        assert s.sample(p, coin=float(r)) == first_below(cdf, r)
    # the generator variant takes exactly one nextFloat per call
    a, b = orc.Sampler(9, n), orc.Sampler(9, n)
    for _ in range(5):
        assert a.sample(p) == first_below(cdf, b.next_float())


def test_sample_skips_zero_probabilities_and_falls_back_to_last(orc):
    p = np.array([0.0, 0.0, 0.5, 0.0, 0.25], dtype=np.float32)
    s = orc.Sampler(1, 5)
    assert s.sample(p, coin=0.0) == 2          # 0 < 0 is false twice
    assert s.sample(p, coin=0.5) == 4          # 0.5 < 0.5 is false, and for index 3 too
    assert s.sample(p, coin=0.75) == 4         # nothing exceeds the draw: n - 1


# ---------------------------------------------------------------- sample_topp

class ProbIndex:
    def __init__(self):
        self.prob = np.float32(0.0)
        self.index = 0


class PySampler:
    """J/Sampler.java:76-120 with Python objects: the list keeps its objects between calls and the whole
    list is sorted (sorted() is stable, like Arrays.sort on objects)."""

    def __init__(self, n):
        self.a = [ProbIndex() for _ in range(n)]

    def sample_topp(self, probs, topp, coin):
        n = len(probs)
        topp = np.float32(topp)
        cutoff = (np.float32(1.0) - topp) / np.float32(n - 1)
        n0 = 0
        for i in range(n):
            if probs[i] >= cutoff:
                self.a[n0].index = i
                self.a[n0].prob = probs[i]
                n0 += 1
        self.a = sorted(self.a, key=lambda e: -float(e.prob))
        cum = np.float32(0.0)
        last = n0 - 1
        for i in range(n0):
            cum = np.float32(cum + self.a[i].prob)
            if cum > topp:
                last = i
                break
        r = np.float32(np.float32(coin) * cum)
        cdf = np.float32(0.0)
        for i in range(last + 1):
            cdf = np.float32(cdf + self.a[i].prob)
            if r < cdf:
                return self.a[i].index
        return self.a[last].index


def test_topp_worked_example_first_call(orc):
    # distinct probabilities, first call of a sampler: plain nucleus sampling
    p = np.array([0.05, 0.4, 0.1, 0.25, 0.2], dtype=np.float32)
    s = orc.Sampler(1, 5)
    # cutoff = 0.3 / 4 = 0.075: index 0 is dropped; order 1 (0.4), 3 (0.25), 4 (0.2), 2 (0.1);
    # cumulative 0.4, 0.65, 0.85 > 0.7 -> three entries, r = coin * 0.85
    assert s.sample_topp(p, 0.7, coin=0.0) == 1
    assert s.sample_topp(p, 0.7, coin=0.46) == 1      # r = 0.391 < 0.4
    assert s.sample_topp(p, 0.7, coin=0.48) == 3      # r = 0.408
    assert s.sample_topp(p, 0.7, coin=0.77) == 4      # r = 0.6545 >= 0.65
    assert s.sample_topp(p, 0.7, coin=0.99999994) == 4


def test_topp_entries_of_an_earlier_call_take_part(orc):
    # Worked by hand from J/Sampler.java:87-119.  Call 1: eight equal probabilities, all candidates.
    # Call 2: five candidates overwrite slots 0..4; slots 5..7 still hold (0.125, 5), (0.125, 6), (0.125, 7)
    # and the sort of the whole array puts them right after the 0.9: cumulative 0.9, 1.025 > 0.95, so the
    # list is cut after two entries and a draw of 0.95 (r = 0.97375) returns token 5 of the earlier call.
    s = orc.Sampler(1, 8)
    u = np.full(8, 0.125, dtype=np.float32)
    assert s.sample_topp(u, 0.5, coin=0.0) == 0
    p = np.array([0.9, 0.04, 0.03, 0.01, 0.01, 0.005, 0.0025, 0.0025], dtype=np.float32)
    assert s.sample_topp(p, 0.95, coin=0.95) == 5
    # a fresh sampler has no such entries: cumulative 0.9, 0.94, 0.97 -> r = 0.9215 -> token 1
    assert orc.Sampler(1, 8).sample_topp(p, 0.95, coin=0.95) == 1


def test_topp_ties_keep_index_order(orc):
    p = np.array([0.2, 0.3, 0.2, 0.3], dtype=np.float32)
    s = orc.Sampler(1, 4)
    # order 1, 3, 0, 2; cumulative 0.3, 0.6, 0.8, 1.0 > 0.9 -> all four, r = coin * 1.0
    got = [s.sample_topp(p, 0.9, coin=c) for c in (0.1, 0.4, 0.7, 0.9)]
    assert got == [1, 3, 0, 2]


@pytest.mark.parametrize("n,scale", [(50, 1.0), (50, 6.0), (2000, 3.0)])
def test_topp_against_object_list_restatement_over_many_calls(orc, n, scale):
    rng = np.random.default_rng(n + int(scale))
    s, py = orc.Sampler(1, n), PySampler(n)
    for call in range(40):
        logits = (rng.standard_normal(n) * scale * rng.choice([0.3, 1.0, 2.0])).astype(np.float32)
        p = np.exp(logits - logits.max()).astype(np.float32)
        p /= p.sum(dtype=np.float32)
        topp = float(rng.choice([0.5, 0.8, 0.9, 0.95]))
        coin = float(np.float32(rng.random()))
        assert s.sample_topp(p, topp, coin=coin) == py.sample_topp(p, topp, coin), call


def test_topp_nan_is_an_error(orc):
    p = np.array([0.5, np.nan, 0.5], dtype=np.float32)
    assert orc.Sampler(1, 3).sample_topp(p, 0.9, coin=0.5) == -1


def test_topp_without_candidates_is_an_error(orc):
    # topp 0: cutoff = 1 / (n - 1), above every probability of a flat distribution -> probIndex[-1] in the reference
    p = np.full(4, 0.25, dtype=np.float32)
    assert orc.Sampler(1, 4).sample_topp(p, 0.0, coin=0.5) == -2
    assert orc.Sampler(1, 4).sample_topp(np.array([0.4, 0.2, 0.2, 0.2], dtype=np.float32), 0.0, coin=0.5) == 0


# ---------------------------------------------------------------- the step of J/Run.java:643-665

def test_step_softmax_and_branches(orc):
    rng = np.random.default_rng(5)
    n = 500
    logits = (rng.standard_normal(n) * 3).astype(np.float32)
    s = orc.Sampler(3, n)
    nxt, after = s.step(logits, 0.0, 0.9)
    assert nxt == int(np.argmax(logits)) and np.array_equal(after, logits)     # temperature 0: untouched
    t = np.float32(0.8)
    ref = np.exp((logits / t).astype(np.float64) - float((logits / t).max()))
    ref /= ref.sum()
    a, b = orc.Sampler(3, n), orc.Sampler(3, n)
    nxt, after = a.step(logits, float(t), 1.0)                                  # topp > 0.999: plain sampling
    assert np.abs(after - ref).max() < 1e-6 and abs(float(after.sum(dtype=np.float64)) - 1) < 1e-5
    assert nxt == first_below(np.cumsum(after, dtype=np.float32), b.next_float())
    a, b = orc.Sampler(4, n), orc.Sampler(4, n)
    nxt, after2 = a.step(logits, float(t), 0.9)
    assert np.array_equal(after, after2)
    assert nxt == PySampler(n).sample_topp(after2, 0.9, b.next_float())


def test_generate_with_temperature_zero_is_greedy(orc):
    shape = dict(dim=64, hidden_dim=128, n_layers=2, n_heads=4, n_kv_heads=4, vocab_size=96, seq_len=24,
                 shared_weights=1)
    m = orc.Model(**shape)
    m.fill_synth(3, 0.5)
    prompt = orc.synth_prompt(3, 3, 96)
    want, _, _ = m.generate_greedy(prompt, 20)
    m.reset()
    got, _ = m.generate(prompt, 20, 0.0, 0.9, 1234)
    assert np.array_equal(got, want)
    m.reset()
    a, _ = m.generate(prompt, 20, 1.0, 0.9, 1234)
    m.reset()
    b, _ = m.generate(prompt, 20, 1.0, 0.9, 1234)
    assert np.array_equal(a, b) and np.array_equal(a[:3], prompt)
