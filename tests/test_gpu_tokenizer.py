"""The tokenizer tests that need no file of the reference, run once more under the `gpu` marker: the same host code of
libllama2j_hip.so (J/Tokenizer.java:102-163, 189-208), exercised on the GPU box beside the kernels it feeds."""
import pytest

from tests import test_tokenizer as T
from tests.test_tokenizer import tiny  # noqa: F401  (the module-scoped fixture)

pytestmark = pytest.mark.gpu


def test_merges_worked_by_hand(tiny):  # noqa: F811
    T.test_merges_worked_by_hand(tiny)


def test_byte_fallback_above_0x7f_fails_as_in_the_reference(tiny):  # noqa: F811
    T.test_byte_fallback_above_0x7f_fails_as_in_the_reference(tiny)


def test_decode_rules(tiny):  # noqa: F811
    T.test_decode_rules(tiny)


def test_library_equals_restatement_on_random_prompts(tiny):  # noqa: F811
    T.test_library_equals_restatement_on_random_prompts(tiny)


def test_open_errors(tmp_path):
    T.test_open_errors(tmp_path)


def test_encoded_prompt_drives_a_decode(tiny, orc):  # noqa: F811
    """Prompt string -> ids -> greedy decode on the GPU -> text, the path of J/Run.java:607-609, 611-680, against the
    oracle's tokenizer restatement and CPU forward on the same ids."""
    import numpy as np
    import llama2j_amd as l2j
    lib_tok, ref_tok = tiny
    ids = lib_tok.bpe_encode("abc bc a")
    assert list(ids) == list(ref_tok.bpe_encode("abc bc a"))
    vocab = len(T.TINY)
    shape = (64, 128, 2, 4, 4, vocab, 32, 1)
    m = orc.Model(dim=shape[0], hidden_dim=shape[1], n_layers=shape[2], n_heads=shape[3], n_kv_heads=shape[4],
                  vocab_size=vocab, seq_len=shape[6], shared_weights=1)
    m.fill_synth(21, 0.05)
    g = l2j.Transformer(l2j.Config(*shape))
    g.fill_synthetic(21, 0.05)
    g.finalize()
    want, _, _ = m.generate_greedy(ids, 24)
    got, _ = g.decode_greedy(ids, 24)
    np.testing.assert_array_equal(got, want)
    tok, text_lib, text_ref = 1, [], []
    for nxt in got:
        text_lib.append(lib_tok.bpe_decode(tok, int(nxt)))
        text_ref.append(ref_tok.bpe_decode(tok, int(nxt)))
        tok = int(nxt)
    assert text_lib == text_ref
    m.close(); g.close()
