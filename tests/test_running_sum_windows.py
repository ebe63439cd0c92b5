"""The arithmetic behind the device sampler's running sums (llama2j_amd/csrc/sampler_kernels.hpp, chain_scan), restated in
Python integers and checked on the CPU: inside a binade of the running sum a float32 addition of a non-negative term is
an integer addition whose increment depends only on the parity of the sum before it, and the term that leaves the binade
is added with a real float32 addition.  The sums must equal numpy's sequential float32 cumsum bit for bit.  (The GPU
routine itself is compared with the same cumsum in tests/test_gpu_sampler.py.)"""
import struct

import numpy as np
import pytest

f32 = np.float32
BIG = 1 << 25


def bits(x):
    return struct.unpack("<I", struct.pack("<f", float(x)))[0]


def window(s):
    """(E, S): s = S * 2^(E - 23), E >= -126"""
    b = bits(s)
    ef, m = (b >> 23) & 0xFF, b & 0x7FFFFF
    return (-126, m) if ef == 0 else (ef - 127, m | (1 << 23))


def increments(e, E):
    """what a term adds to the integer sum in the binade E when the sum before it is even / odd"""
    b = bits(e)
    ef, m = (b >> 23) & 0xFF, b & 0x7FFFFF
    if ef == 0xFF:
        return BIG, BIG
    Ee, M = (-126, m) if ef == 0 else (ef - 127, m | (1 << 23))
    d = E - Ee
    if M == 0 or d >= 25:
        return 0, 0
    if d < 0:
        return BIG, BIG
    if d == 0:
        return M, M
    a, rem, half = M >> d, M & ((1 << d) - 1), 1 << (d - 1)
    if rem != half:
        return (a, a) if rem < half else (a + 1, a + 1)
    return a + (a & 1), a + ((a + 1) & 1)          # a tie goes to the even sum


def value(S, E):
    return f32(np.ldexp(np.float64(S), E - 23))


def compose(x, y):
    """increments of a run of terms followed by another run"""
    return x[0] + y[x[0] & 1], x[1] + y[(1 + x[1]) & 1]


def running_sums(p, tile=64):
    out, s, i, n = [], f32(0.0), 0, len(p)
    while i < n:
        if s == 0:
            s = f32(p[i]); out.append(s); i += 1
            continue
        E, S = window(s)
        run = [increments(x, E) for x in p[i:i + tile]]
        # the prefix compositions, as a scan would form them
        pre, acc = [], (0, 0)
        for inc in run:
            acc = compose(acc, inc)
            pre.append(acc)
        sums = [S + q[S & 1] for q in pre]
        cross = next((k for k, v in enumerate(sums) if v >= 1 << 24), None)
        upto = len(run) if cross is None else cross
        out.extend(value(v, E) for v in sums[:upto])
        i += upto
        s = out[-1] if upto else s
        if cross is not None:                       # the term that leaves the binade: a real addition
            s = f32(s + f32(p[i])); out.append(s); i += 1
    return np.array(out, dtype=np.float32)


def cases():
    rng = np.random.default_rng(0)
    n = 3000
    yield "uniform", rng.random(n)
    yield "peaked softmax", np.exp(rng.standard_normal(n) * 6 - 20)
    yield "forty orders of magnitude", np.exp(rng.uniform(-80, 5, n))
    yield "sorted descending", np.sort(rng.random(n) / n)[::-1]
    yield "powers of two", np.ldexp(1.0, rng.integers(-30, 3, n))
    yield "3 * powers of two", 3 * np.ldexp(1.0, rng.integers(-30, 3, n))
    yield "halves", np.full(n, 0.5)
    yield "half and three quarters of an ulp", np.concatenate([np.ones(900), np.full(900, 2.0 ** -14), np.full(900, 1.5 * 2.0 ** -14)])
    yield "denormals", np.concatenate([np.full(500, 1e-45), np.full(500, 1e-40), rng.random(500) * 1e-38])
    yield "zeros", np.where(rng.random(n) < 0.5, 0.0, rng.random(n))
    yield "every term leaves the binade", np.ldexp(1.0, np.arange(-100, 100))


@pytest.mark.parametrize("name,terms", list(cases()), ids=[c[0] for c in cases()])
def test_binade_sums_equal_the_sequential_float32_sums(name, terms):
    terms = np.asarray(terms, dtype=np.float32)
    want = np.cumsum(terms, dtype=np.float32)       # one addition after the other, in float32
    got = running_sums(terms)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), int(np.argmax(got != want))
