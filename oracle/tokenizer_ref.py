"""TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.

Restatement of the reference's tokenizer (J/Tokenizer.java, J/ = src/main/java/com/lastbot/llama2j/) with Java's
string semantics spelled out: a string is a tuple of UTF-16 code units, compareTo is the lexicographic order of
those tuples, Arrays.binarySearch takes the probes it takes.  Pure Python; only tests import it.

Pinned (tests/test_tokenizer.py) by token ids of the Llama-2 vocabulary that are public knowledge
("Hello world" = 15043, 3186; "Once upon a time" = 9038, 2501, 263, 931; token 13 = "<0x0A>" = newline) when the
reference's tokenizer.bin is at hand, and by merges worked by hand on a tiny vocabulary.
"""
import struct


def units(s):
    """Java String of a Python str: UTF-16 code units."""
    b = s.encode("utf-16-le", "surrogatepass")
    return tuple(struct.unpack("<%dH" % (len(b) // 2), b))


def to_str(u):
    """String.getBytes(UTF_8) then back: pairs of surrogates are one character, an unpaired surrogate becomes '?'."""
    out, i = [], 0
    while i < len(u):
        c = u[i]
        if 0xD800 <= c <= 0xDBFF and i + 1 < len(u) and 0xDC00 <= u[i + 1] <= 0xDFFF:
            out.append(chr(0x10000 + ((c - 0xD800) << 10) + (u[i + 1] - 0xDC00)))
            i += 2
            continue
        out.append("?" if 0xD800 <= c <= 0xDFFF else chr(c))
        i += 1
    return "".join(out)


class JavaIndexError(Exception):
    """Where the reference throws ArrayIndexOutOfBoundsException / StringIndexOutOfBoundsException."""


class Tokenizer:
    def __init__(self, path, vocab_size):
        # J/Tokenizer.java:61-90
        self.vocab, self.scores = [], []
        with open(path, "rb") as f:
            f.read(4)                                   # max_token_length, ignored (:70)
            for _ in range(vocab_size):
                score, n = struct.unpack("<fi", f.read(8))
                self.scores.append(score)
                self.vocab.append(units(f.read(n).decode("utf-8")))
        self.sorted_vocab = sorted(range(vocab_size), key=lambda i: self.vocab[i])   # stable, as Arrays.sort (:85)

    def lookup(self, key):
        # :47-56 : Arrays.binarySearch on the sorted TokenIndex array
        low, high = 0, len(self.sorted_vocab) - 1
        while low <= high:
            mid = (low + high) >> 1
            v = self.vocab[self.sorted_vocab[mid]]
            if v < key:
                low = mid + 1
            elif v > key:
                high = mid - 1
            else:
                return self.sorted_vocab[mid]
        return -1

    def lookup_char(self, c):
        # :92-100 : first vocabulary entry that is exactly this one char
        for i, v in enumerate(self.vocab):
            if len(v) == 1 and v[0] == c:
                return i
        return -1

    def bpe_encode(self, prompt):
        # :102-163
        tokens = [self.lookup(units(" "))]
        for c in units(prompt):
            i = self.lookup_char(c)
            if i != -1:
                tokens.append(i)
            else:
                for b in to_str((c,)).encode("utf-8"):
                    tokens.append((b - 256 if b > 127 else b) + 3)      # Java bytes are signed (:123-125)
        while True:
            best_score, best_id, best_idx = -1e10, -1, -1   # -1e10f is exact in float32
            for i in range(len(tokens) - 1):
                for t in (tokens[i], tokens[i + 1]):
                    if t < 0 or t >= len(self.vocab):
                        raise JavaIndexError(t)
                j = self.lookup(self.vocab[tokens[i]] + self.vocab[tokens[i + 1]])
                if j != -1 and self.scores[j] > best_score:
                    best_score, best_id, best_idx = self.scores[j], j, i
            if best_idx == -1:
                break
            tokens[best_idx] = best_id
            del tokens[best_idx + 1]
        return tokens

    def bpe_decode(self, token, nxt):
        # :189-208
        piece = self.vocab[nxt]
        if token == 1:
            if not piece:
                raise JavaIndexError(0)
            if piece[0] == 0x20:
                piece = piece[1:]
        s = "".join(chr(c) for c in piece)               # lone surrogates stay as they are for the pattern match
        hexdigits = "0123456789abcdefABCDEF"
        if s.startswith("<0x") and s.endswith(">") and len(s) >= 4 and all(ch in hexdigits for ch in s[3:-1]):
            if len(s) == 4:
                return None                              # Integer.parseInt("") throws
            value = int(s[3:-1], 16)
            if value > 0x7FFFFFFF:
                return None
            c = value & 0xFF
            if c != 0x0A and (c <= 0x1F or 0x7F <= c <= 0x9F):
                return None
            return chr(c)
        return to_str(piece)
