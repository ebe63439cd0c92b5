"""ctypes binding of libllama2j_hip.so and the host-side mirror of llama2j's Java classes.

Reference classes mirrored (J/ = src/main/java/com/lastbot/llama2j/ in the reference):
  Config             J/Config.java:6-14
  Quant              J/Quant.java (encode / decode / size helpers / extension)
  Transformer        J/TransformerWeights.java + J/RunState.java + Run.transformer (J/Run.java:44-51)
  Sampler.argmax     J/Sampler.java:46-57
Errors become exceptions carrying the library's message, as the reference turns CUDA errors into
RuntimeException (J/ContextCUDA.java:296-304).
"""
import atexit
import ctypes as C
import os
import subprocess
import weakref

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

F_EXACT_SILU = 1


class TENSOR:
    TOK_EMB, RMS_ATT, WQ, WK, WV, WO, RMS_FFN, W1, W2, W3, RMS_FINAL, WCLS = range(12)
    QUANT = (RMS_ATT, WQ, WK, WV, WO, RMS_FFN, W1, W2, W3, RMS_FINAL)


class BUFFER:
    X, XB, XB2, HB, Q, K, V, LOGITS, KCACHE, VCACHE = range(10)


class KERNEL:
    QKV, ATTENTION, WO, W13, W2, CLASSIFIER, TOKEN = range(7)
    NAMES = ("qkv", "attention", "wo", "w13", "w2", "classifier", "token")


class L2JError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("llama2j_hip error %d: %s" % (code, msg))
        self.code = code


class Config(C.Structure):
    """J/Config.java:6-14 plus shared_weights (J/Run.java:572), the quantization constants
    (J/Run.java:27-28), the device ordinal and flags."""
    _fields_ = [(n, C.c_int32) for n in
                ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len",
                 "shared_weights", "group_size", "bits", "device")] + [("flags", C.c_uint32)]

    def __init__(self, dim=0, hidden_dim=0, n_layers=0, n_heads=0, n_kv_heads=0, vocab_size=0, seq_len=0,
                 shared_weights=1, group_size=256, bits=8, device=0, flags=0):
        super().__init__(dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len, shared_weights,
                         group_size, bits, device, flags)

    @property
    def head_size(self):
        return self.dim // self.n_heads

    @property
    def kv_dim(self):
        return self.dim * self.n_kv_heads // self.n_heads

    def __repr__(self):
        return "Config{" + ", ".join("%s=%d" % (n, getattr(self, n)) for n, _ in self._fields_[:7]) + "}"


def lib_path():
    """The in-tree library; L2J_LIB_PATH selects another build of the same ABI (kernel experiments)."""
    return os.environ.get("L2J_LIB_PATH") or os.path.join(_HERE, "libllama2j_hip.so")


def build_library():
    """Compile libllama2j_hip.so for gfx950 with hipcc (about ten seconds)."""
    subprocess.check_call(["sh", os.path.join(_HERE, "csrc", "build.sh")])


_lib = None

_SIGNATURES = None


def _signatures():
    vp, u8p, fp, i32p = C.c_void_p, C.POINTER(C.c_uint8), C.POINTER(C.c_float), C.POINTER(C.c_int32)
    cfgp = C.POINTER(Config)
    return {
        "l2j_create": (C.c_int, [cfgp, C.POINTER(vp)]),
        "l2j_destroy": (None, [vp]),
        "l2j_last_error": (C.c_char_p, []),
        "l2j_ctx_last_error": (C.c_int, [vp, C.c_char_p, C.c_int32]),
        "l2j_set_option": (C.c_int, [vp, C.c_char_p, C.c_int32]),
        "l2j_get_option": (C.c_int, [vp, C.c_char_p, i32p]),
        "l2j_device_count": (C.c_int, []),
        "l2j_upload_quant": (C.c_int, [vp, C.c_int, u8p, C.c_uint64]),
        "l2j_upload_quant_layer": (C.c_int, [vp, C.c_int, C.c_int, u8p, C.c_uint64]),
        "l2j_upload_f32": (C.c_int, [vp, C.c_int, fp, C.c_uint64]),
        "l2j_upload_f32_quantize": (C.c_int, [vp, C.c_int, C.c_uint64, fp, C.c_uint64]),
        "l2j_read_quant": (C.c_int, [vp, C.c_int, C.c_uint64, C.c_uint64, u8p]),
        "l2j_fill_synthetic": (C.c_int, [vp, C.c_uint64, C.c_float]),
        "l2j_finalize": (C.c_int, [vp]),
        "l2j_reset": (C.c_int, [vp]),
        "l2j_forward": (C.c_int, [vp, C.c_int32, C.c_int32, fp]),
        "l2j_forward_argmax": (C.c_int, [vp, C.c_int32, C.c_int32, i32p]),
        "l2j_forward_taps": (C.c_int, [vp, C.c_int32, C.c_int32, fp]),
        "l2j_decode_greedy": (C.c_int, [vp, i32p, C.c_int32, C.c_int32, i32p, i32p, C.POINTER(C.c_double)]),
        "l2j_sampler_seed": (C.c_int, [vp, C.c_int64]),
        "l2j_sample": (C.c_int, [vp, fp, C.c_float, C.c_float, C.c_float, i32p]),
        "l2j_running_sums": (C.c_int, [vp, fp, C.c_int32, fp]),
        "l2j_running_sums_noalloc": (C.c_int, [vp, fp, C.c_int32, fp]),
        "l2j_sum_probe": (C.c_int, [vp, fp, C.c_int32, fp, C.c_int32, i32p, fp, fp]),
        "l2j_prefill": (C.c_int, [vp, i32p, C.c_int32, C.c_int32, fp, C.POINTER(C.c_double)]),
        "l2j_decode_sample": (C.c_int, [vp, i32p, C.c_int32, C.c_int32, C.c_float, C.c_float, C.c_int64, i32p, i32p,
                                        C.POINTER(C.c_double)]),
        "l2j_read": (C.c_int, [vp, C.c_int, C.c_int, C.c_uint64, fp, C.c_uint64]),
        "l2j_write_kv": (C.c_int, [vp, C.c_int, C.c_int32, C.c_int32, fp, fp]),
        "l2j_sync": (C.c_int, [vp]),
        "l2j_time_kernel": (C.c_int, [vp, C.c_int, C.c_int32, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_uint64)]),
        "l2j_calibration_copy": (C.c_int, [vp, C.c_uint64, C.c_int32]),
        "l2j_decode_greedy_batch": (C.c_int, [vp, i32p, i32p, C.c_int32, C.c_int32, C.c_int32, i32p, C.POINTER(C.c_double)]),
        "l2j_decode_greedy_batch_logits": (C.c_int, [vp, i32p, i32p, C.c_int32, C.c_int32, C.c_int32, i32p, fp]),
        "l2j_release_batch": (C.c_int, [vp]),
        "l2j_decode_sample_batch": (C.c_int, [vp, i32p, i32p, C.c_int32, C.c_int32, C.c_int32, C.c_float, C.c_float,
                                              C.POINTER(C.c_int64), i32p, C.POINTER(C.c_double), fp]),
        "l2j_batch_matmul": (C.c_int, [vp, C.c_int, C.c_int, fp, fp, C.c_int32, C.c_int32, C.POINTER(C.c_double)]),
        "l2j_bytes_per_token": (C.c_uint64, [cfgp, C.c_int32]),
        "l2j_quant_nbytes": (C.c_uint64, [C.c_uint64]),
        "l2j_quant_encode": (C.c_int, [fp, C.c_uint64, u8p]),
        "l2j_quant_decode": (C.c_int, [u8p, C.c_uint64, C.c_uint64, fp]),
        "l2j_write_quant_file": (C.c_int, [C.c_char_p, u8p, C.c_uint64]),
        "l2j_read_quant_file": (C.c_int64, [C.c_char_p, u8p, C.c_uint64]),
        "l2j_quant_cache_path": (C.c_int, [C.c_char_p, C.c_int, C.c_char_p, C.c_int]),
        "l2j_read_checkpoint_header": (C.c_int, [C.c_char_p, cfgp]),
        "l2j_load_checkpoint": (C.c_int, [C.c_char_p, C.c_int, C.c_uint32, C.c_int, C.POINTER(vp)]),
        "l2j_get_config": (C.c_int, [vp, cfgp]),
        "l2j_tokenizer_open": (C.c_int, [C.c_char_p, C.c_int32, C.POINTER(vp)]),
        "l2j_tokenizer_close": (None, [vp]),
        "l2j_bpe_encode": (C.c_int, [vp, C.c_char_p, i32p, C.c_int32, i32p]),
        "l2j_bpe_decode": (C.c_int, [vp, C.c_int32, C.c_int32, C.c_char_p, C.c_int32, i32p]),
    }


def lib():
    """Loads the built library.  Raises if it was not built: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise FileNotFoundError(path + " is missing: run llama2j_amd/csrc/build.sh (or __graft_entry__.build())")
    L = C.CDLL(path)
    for name, (res, args) in _signatures().items():
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args
    _lib = L
    return L


def _check(rc):
    if rc < 0:
        raise L2JError(rc, lib().l2j_last_error().decode(errors="replace"))
    return rc


def _fp(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u8(a):
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def _i32(a):
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_int32))


class Quant:
    """J/Quant.java: group min/max linear 8-bit codec (host side)."""

    def __init__(self, groupSize=256, bits=8):
        if groupSize != 256 or bits != 8:
            raise ValueError("only Quant(256, 8) is implemented (J/Run.java:27-28)")
        self.groupSize, self.bits = groupSize, bits

    def encodedBytesPerGroup(self):
        return self.groupSize * self.bits // 8 + 8

    def numberOfBytesByFloatSize(self, floatSize):
        return int(lib().l2j_quant_nbytes(floatSize))

    def encode(self, values):
        x = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        out = np.empty(self.numberOfBytesByFloatSize(x.size), dtype=np.uint8)
        _check(lib().l2j_quant_encode(_fp(x), x.size, _u8(out)))
        return out

    def decode(self, encoded, floatIndex, size):
        enc = np.ascontiguousarray(encoded, dtype=np.uint8)
        out = np.empty(size, dtype=np.float32)
        _check(lib().l2j_quant_decode(_u8(enc), floatIndex, size, _fp(out)))
        return out

    def extension(self):
        return "_%d_%d.quant" % (self.groupSize, self.bits)

    @staticmethod
    def write_file(path, encoded):
        enc = np.ascontiguousarray(encoded, dtype=np.uint8)
        _check(lib().l2j_write_quant_file(os.fsencode(path), _u8(enc), enc.size))

    @staticmethod
    def read_file(path, expected_bytes):
        out = np.empty(expected_bytes, dtype=np.uint8)
        n = lib().l2j_read_quant_file(os.fsencode(path), _u8(out), out.size)
        _check(n)
        return out[:n]

    @staticmethod
    def cache_path(bin_path, tensor):
        buf = C.create_string_buffer(4096)
        _check(lib().l2j_quant_cache_path(os.fsencode(bin_path), tensor, buf, 4096))
        return os.fsdecode(buf.value)


class Sampler:
    """J/Sampler.java:46-57; the device computes the same first-max inside the forward.  The sampling methods
    of the reference run on the device through Transformer.sampler_seed / sample / decode_sample."""

    @staticmethod
    def argmax(logits):
        return int(np.argmax(np.asarray(logits)))  # numpy also returns the first maximum


class Tokenizer:
    """J/Tokenizer.java: tokenizer.bin reader, bpe_encode, bpe_decode (host code inside the library)."""

    def __init__(self, tokenizerFilePath, vocabSize):
        h = C.c_void_p()
        _check(lib().l2j_tokenizer_open(os.fsencode(tokenizerFilePath), vocabSize, C.byref(h)))
        self._h = h

    def bpe_encode(self, prompt):
        raw = prompt.encode("utf-8", "surrogatepass") if isinstance(prompt, str) else bytes(prompt)
        cap = 2 * len(raw) + 2
        out = np.zeros(cap, dtype=np.int32)
        n = C.c_int32(0)
        _check(lib().l2j_bpe_encode(self._h, raw, _i32(out), cap, C.byref(n)))
        return out[:n.value].copy()

    def bpe_decode(self, token, next):
        buf = C.create_string_buffer(1 << 16)
        n = C.c_int32(0)
        _check(lib().l2j_bpe_decode(self._h, token, next, buf, len(buf), C.byref(n)))
        return None if n.value < 0 else buf.raw[:n.value].decode("utf-8")

    def close(self):
        if getattr(self, "_h", None):
            lib().l2j_tokenizer_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_live = weakref.WeakSet()


@atexit.register
def _close_live():
    """Contexts still open at interpreter exit are destroyed here, while the HIP runtime is still whole: graph,
    events, buffers and stream go before any library's own exit handlers run."""
    for t in list(_live):
        t.close()


class Transformer:
    """Weights + run state + forward on the GPU (TransformerWeights, RunState, Run.transformer)."""

    def __init__(self, config=None, _handle=None, options=None):
        """options: {name: int} passed to l2j_set_option before anything else (launch shapes, see the header)."""
        L = lib()
        if _handle is None:
            h = C.c_void_p()
            _check(L.l2j_create(C.byref(config), C.byref(h)))
            _handle = h
        self._h = _handle
        _live.add(self)
        self.config = Config()
        self._check(L.l2j_get_config(self._h, C.byref(self.config)))
        for k, v in (options or {}).items():
            self.set_option(k, v)

    def _check(self, rc):
        """Negative return codes become L2JError with the context's own error text (l2j_ctx_last_error: right
        whatever thread made the failing call)."""
        if rc < 0:
            buf = C.create_string_buffer(1024)
            n = lib().l2j_ctx_last_error(self._h, buf, len(buf)) if self._h else -1
            raise L2JError(rc, buf.value.decode(errors="replace") if n >= 0 else lib().l2j_last_error().decode(errors="replace"))
        return rc

    def last_error(self):
        buf = C.create_string_buffer(1024)
        self._check(lib().l2j_ctx_last_error(self._h, buf, len(buf)))
        return buf.value.decode(errors="replace")

    def get_option(self, name):
        v = C.c_int32(0)
        self._check(lib().l2j_get_option(self._h, name.encode(), C.byref(v)))
        return v.value

    def set_option(self, name, value):
        self._check(lib().l2j_set_option(self._h, name.encode(), int(value)))

    @classmethod
    def from_checkpoint(cls, bin_path, device=0, flags=0, write_caches=True):
        """= new TransformerWeights(context, reader, ...) + new RunState (J/Run.java:561-593)."""
        h = C.c_void_p()
        _check(lib().l2j_load_checkpoint(os.fsencode(bin_path), device, flags, 1 if write_caches else 0, C.byref(h)))
        return cls(_handle=h)

    def close(self):
        if getattr(self, "_h", None):
            lib().l2j_destroy(self._h)
            self._h = None
            _live.discard(self)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # ---- load phase
    def upload_quant(self, tensor, ref_bytes):
        b = np.ascontiguousarray(ref_bytes, dtype=np.uint8)
        self._check(lib().l2j_upload_quant(self._h, tensor, _u8(b), b.size))

    def upload_quant_layer(self, tensor, layer, ref_bytes):
        b = np.ascontiguousarray(ref_bytes, dtype=np.uint8)
        self._check(lib().l2j_upload_quant_layer(self._h, tensor, layer, _u8(b), b.size))

    def upload_f32(self, tensor, values):
        v = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        self._check(lib().l2j_upload_f32(self._h, tensor, _fp(v), v.size))

    def upload_f32_quantize(self, tensor, values, first=0):
        v = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
        self._check(lib().l2j_upload_f32_quantize(self._h, tensor, first, _fp(v), v.size))

    def read_quant(self, tensor, group0, ngroups):
        out = np.empty(ngroups * 264, dtype=np.uint8)
        self._check(lib().l2j_read_quant(self._h, tensor, group0, ngroups, _u8(out)))
        return out

    def fill_synthetic(self, seed, sigma=0.02):
        self._check(lib().l2j_fill_synthetic(self._h, seed, C.c_float(sigma)))

    def finalize(self):
        self._check(lib().l2j_finalize(self._h))

    def reset(self):
        self._check(lib().l2j_reset(self._h))

    # ---- forward
    def forward(self, token, pos, want_logits=True):
        """Run.transformer(token, pos, ...) + the logits copy (J/Run.java:625-632)."""
        logits = np.empty(self.config.vocab_size, dtype=np.float32) if want_logits else None
        self._check(lib().l2j_forward(self._h, token, pos, _fp(logits) if want_logits else None))
        return logits

    def prefill(self, tokens, pos0=0, want_logits=True):
        """forward(tokens[i], pos0 + i) for every i, 32 positions per step on the matrix cores: (logits of the last
        position or None, device seconds)."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.empty(self.config.vocab_size, dtype=np.float32) if want_logits else None
        sec = C.c_double(0.0)
        self._check(lib().l2j_prefill(self._h, tokens.ctypes.data_as(C.POINTER(C.c_int32)), tokens.size, pos0,
                                      _fp(logits) if want_logits else None, C.byref(sec)))
        return logits, sec.value

    def forward_argmax(self, token, pos):
        nxt = C.c_int32(-1)
        self._check(lib().l2j_forward_argmax(self._h, token, pos, C.byref(nxt)))
        return nxt.value

    def forward_taps(self, token, pos):
        logits = np.empty(self.config.vocab_size, dtype=np.float32)
        self._check(lib().l2j_forward_taps(self._h, token, pos, _fp(logits)))
        return logits

    def decode_greedy(self, prompt, steps):
        """The token loop of Run.main at temperature 0 (J/Run.java:611-685)."""
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        cap = self.config.seq_len if steps <= 0 or steps > self.config.seq_len else steps
        out = np.zeros(cap, dtype=np.int32)
        n = C.c_int32(0)
        sec = C.c_double(0.0)
        self._check(lib().l2j_decode_greedy(self._h, _i32(p), p.size, steps, _i32(out), C.byref(n), C.byref(sec)))
        return out[:n.value], sec.value

    def sampler_seed(self, rng_seed):
        """new Sampler(rngSeed, vocab_size) (J/Sampler.java:24-31): java.util.Random(seed), empty ProbIndex array."""
        self._check(lib().l2j_sampler_seed(self._h, rng_seed))

    def sample(self, temperature, topp, logits=None, coin=None):
        """The sampling step of J/Run.java:643-665 on the device.  logits: an array to sample from instead of the
        last forward's; coin: the caller's Random.nextFloat() instead of the context's generator."""
        nxt = C.c_int32(0)
        lp = None
        if logits is not None:
            logits = np.ascontiguousarray(logits, dtype=np.float32)
            if logits.size != self.config.vocab_size:
                raise ValueError("logits must hold vocab_size floats")
            lp = _fp(logits)
        self._check(lib().l2j_sample(self._h, lp, temperature, topp, -1.0 if coin is None else coin, C.byref(nxt)))
        return nxt.value

    def running_sums_noalloc(self, terms):
        """running_sums through the entry point that allocates nothing (the terms pass through a fixed device buffer
        of the library: at most 36864)."""
        terms = np.ascontiguousarray(terms, dtype=np.float32)
        out = np.empty_like(terms)
        self._check(lib().l2j_running_sums_noalloc(self._h, _fp(terms), terms.size, _fp(out)))
        return out

    def decode_greedy_batch(self, prompts, steps, n_seq=None, want_logits=False):
        """Sixteen or thirty-two greedy token loops at once (l2j_decode_greedy_batch).  prompts: up to n_seq id sequences
        (missing ones run without a prompt; n_seq defaults to 16, or 32 for more than sixteen prompts); returns (tokens of
        shape (n_seq, steps), seconds after the first step), or with want_logits (tokens, logits of shape (steps, n_seq,
        vocab_size)) through l2j_decode_greedy_batch_logits."""
        if n_seq is None:
            n_seq = 16 if len(prompts) <= 16 else 32
        assert len(prompts) <= n_seq
        stride = max([len(p) for p in prompts] + [1])
        ids = np.zeros((n_seq, stride), dtype=np.int32)
        n = np.zeros(n_seq, dtype=np.int32)
        for b, p in enumerate(prompts):
            ids[b, :len(p)] = p
            n[b] = len(p)
        out = np.zeros((n_seq, steps), dtype=np.int32)
        if want_logits:
            logits = np.empty((steps, n_seq, self.config.vocab_size), dtype=np.float32)
            self._check(lib().l2j_decode_greedy_batch_logits(self._h, _i32(ids), _i32(n), n_seq, stride, steps, _i32(out), _fp(logits)))
            return out, logits
        sec = C.c_double(0.0)
        self._check(lib().l2j_decode_greedy_batch(self._h, _i32(ids), _i32(n), n_seq, stride, steps, _i32(out), C.byref(sec)))
        return out, sec.value

    @staticmethod
    def until_bos(tokens):
        """The rows of decode_greedy_batch / decode_sample_batch as Run.main's loop would have left them: each cut behind its
        first token 1, where the reference's loop stops (J/Run.java:670-672); the batch runs every sequence to the last step."""
        out = []
        for row in np.asarray(tokens):
            ones = np.flatnonzero(row == 1)
            out.append(row[:ones[0] + 1] if ones.size else row)
        return out

    def release_batch(self):
        """Frees what the calls for several sequences at once keep on the device (l2j_release_batch)."""
        self._check(lib().l2j_release_batch(self._h))

    def decode_sample_batch(self, prompts, steps, temperature, topp, rng_seeds, n_seq=None, want_logits=False):
        """decode_greedy_batch with a sampler per sequence (l2j_decode_sample_batch): sequence b samples its unforced
        tokens from a sampler seeded with rng_seeds[b].  Returns (tokens, seconds after the first step), with want_logits
        (tokens, seconds, logits of every step before sampling, of shape (steps, n_seq, vocab_size))."""
        if n_seq is None:
            n_seq = 16 if len(prompts) <= 16 else 32
        assert len(prompts) <= n_seq
        seeds = np.zeros(n_seq, dtype=np.int64)
        seeds[:len(rng_seeds)] = rng_seeds
        stride = max([len(p) for p in prompts] + [1])
        ids = np.zeros((n_seq, stride), dtype=np.int32)
        n = np.zeros(n_seq, dtype=np.int32)
        for b, p in enumerate(prompts):
            ids[b, :len(p)] = p
            n[b] = len(p)
        out = np.zeros((n_seq, steps), dtype=np.int32)
        logits = np.empty((steps, n_seq, self.config.vocab_size), dtype=np.float32) if want_logits else None
        sec = C.c_double(0.0)
        self._check(lib().l2j_decode_sample_batch(self._h, _i32(ids), _i32(n), n_seq, stride, steps, temperature, topp,
                                                  seeds.ctypes.data_as(C.POINTER(C.c_int64)), _i32(out), C.byref(sec),
                                                  _fp(logits) if want_logits else None))
        return (out, sec.value, logits) if want_logits else (out, sec.value)

    def batch_matmul(self, tensor, layer, x, rows, groups_per_slice=2, rounds=1):
        """y[b] = W x[b] for sixteen activation vectors against one layer's matrix of a quantized tensor, by the
        matrix-core kernel of the batched path; returns (y of shape (16, rows), mean microseconds per launch)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        assert x.ndim == 2 and x.shape[0] == 16
        y = np.empty((16, rows), dtype=np.float32)
        us = C.c_double(0.0)
        self._check(lib().l2j_batch_matmul(self._h, int(tensor), layer, _fp(x), _fp(y), groups_per_slice, rounds, C.byref(us)))
        return y, us.value

    def running_sums(self, terms):
        """The float32 sums terms[0] + ... + terms[i] formed one addition after the other (the order of the reference's
        softmax denominator and cdf loops), by the routine the device sampler uses."""
        terms = np.ascontiguousarray(terms, dtype=np.float32)
        out = np.empty_like(terms)
        self._check(lib().l2j_running_sums(self._h, _fp(terms), terms.size, _fp(out)))
        return out

    def sum_probe(self, terms, limits):
        """The sequential float32 sum of the terms as the one-launch sampling step forms it: (index, sum, total) with
        index[q] the first i whose running sum exceeds limits[q] (-1: none), sum[q] that running sum, total the sum of
        all terms."""
        terms = np.ascontiguousarray(terms, dtype=np.float32)
        limits = np.ascontiguousarray(limits, dtype=np.float32)
        idx = np.empty(max(limits.size, 1), dtype=np.int32)
        at = np.empty(max(limits.size, 1), dtype=np.float32)
        total = np.empty(1, dtype=np.float32)
        self._check(lib().l2j_sum_probe(self._h, _fp(terms), terms.size, _fp(limits), limits.size,
                                        idx.ctypes.data_as(C.POINTER(C.c_int32)), _fp(at), _fp(total)))
        return idx[:limits.size], at[:limits.size], float(total[0])

    def decode_sample(self, prompt, steps, temperature, topp, rng_seed):
        """The token loop of Run.main with its sampler (J/Run.java:611-685)."""
        p = np.ascontiguousarray(prompt, dtype=np.int32)
        cap = self.config.seq_len if steps <= 0 or steps > self.config.seq_len else steps
        out = np.zeros(cap, dtype=np.int32)
        n = C.c_int32(0)
        sec = C.c_double(0.0)
        self._check(lib().l2j_decode_sample(self._h, _i32(p), p.size, steps, temperature, topp, rng_seed, _i32(out),
                                       C.byref(n), C.byref(sec)))
        return out[:n.value], sec.value

    def read(self, which, layer=-1, off=0, n=None):
        c = self.config
        if n is None:
            n = {BUFFER.HB: c.hidden_dim, BUFFER.K: c.kv_dim, BUFFER.V: c.kv_dim, BUFFER.LOGITS: c.vocab_size,
                 BUFFER.KCACHE: c.seq_len * c.kv_dim, BUFFER.VCACHE: c.seq_len * c.kv_dim}.get(which, c.dim) - off
        out = np.empty(n, dtype=np.float32)
        self._check(lib().l2j_read(self._h, which, layer, off, _fp(out), n))
        return out

    def write_kv(self, layer, pos0, k, v):
        k = np.ascontiguousarray(k, dtype=np.float32).reshape(-1)
        v = np.ascontiguousarray(v, dtype=np.float32).reshape(-1)
        assert k.size == v.size and k.size % self.config.kv_dim == 0
        self._check(lib().l2j_write_kv(self._h, layer, pos0, k.size // self.config.kv_dim, _fp(k), _fp(v)))

    def sync(self):
        self._check(lib().l2j_sync(self._h))

    def time_kernel(self, kernel_class, pos, rounds=3):
        us = C.c_double(0)
        b = C.c_uint64(0)
        self._check(lib().l2j_time_kernel(self._h, kernel_class, pos, rounds, C.byref(us), C.byref(b)))
        return us.value, b.value

    def calibration_copy(self, nbytes, rounds=3):
        self._check(lib().l2j_calibration_copy(self._h, nbytes, rounds))

    def bytes_per_token(self, pos):
        return int(lib().l2j_bytes_per_token(C.byref(self.config), pos))
