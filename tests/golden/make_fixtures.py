"""Writes the committed fixtures of tests/golden/: a tiny llama2.c v0 checkpoint, its ten .quant caches
and the oracle's logits / greedy tokens for it.  Run from the repository root:
    python tests/golden/make_fixtures.py
The reference itself holds no fixtures (no src/test) and cannot run here (Java, no JVM), so the expected
values come from the CPU oracle, which the other tests pin independently."""
import os
import struct
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as orc  # noqa: E402

CFG = (32, 48, 2, 4, 2, 40, 12)   # dim hidden layers heads kv_heads vocab seq_len; unshared classifier


def main():
    dim, hidden, L, H, kvH, vocab, seq = CFG
    rng = np.random.default_rng(2024)
    kvd = dim * kvH // H
    sizes = [L * dim, L * dim * dim, L * dim * kvd, L * dim * kvd, L * dim * dim, L * dim, L * dim * hidden,
             L * hidden * dim, L * dim * hidden, dim]
    tens = [(rng.standard_normal(n) * 0.08).astype(np.float32) for n in sizes]
    for i in (0, 5, 9):
        tens[i] += 1.0
    emb = (rng.standard_normal(vocab * dim) * 0.08).astype(np.float32)
    wcls = (rng.standard_normal(vocab * dim) * 0.08).astype(np.float32)
    path = os.path.join(HERE, "tiny.bin")
    for f in os.listdir(HERE):
        if f.endswith(".quant"):
            os.remove(os.path.join(HERE, f))
    with open(path, "wb") as f:
        f.write(struct.pack("<7i", dim, hidden, L, H, kvH, -vocab, seq))
        f.write(emb.tobytes())
        for t in tens:
            f.write(t.tobytes())
        f.write(np.zeros(seq * (dim // H), "<f4").tobytes())  # freq_cis_real, freq_cis_imag (skipped by the loader)
        f.write(wcls.tobytes())
    m = orc.Model.load(path, write_caches=True)
    prompt = np.array([5, 17, 3], np.int32)
    toks, logits, _ = m.generate_greedy(prompt, seq, want_logits=True)
    np.savez(os.path.join(HERE, "expected.npz"), prompt=prompt, tokens=toks, logits=logits)
    print("wrote", path, os.path.getsize(path), "bytes;", len(toks), "steps")


if __name__ == "__main__":
    main()
