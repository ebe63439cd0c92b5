"""TEST INFRASTRUCTURE - ctypes binding of the CPU oracle (oracle/liboracle.so).

Only tests, the smoke check and the cpu_baseline leg of the benchmark import this.
The HIP library and the llama2j_amd package never do.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

GROUP_SIZE = 256
GROUP_BYTES = 264

T_RMS_ATT, T_WQ, T_WK, T_WV, T_WO, T_RMS_FFN, T_W1, T_W2, T_W3, T_RMS_FINAL = range(10)
T_COUNT = 10
TAP_Q, TAP_K, TAP_V, TAP_ATT_OUT, TAP_X_ATT, TAP_HB, TAP_X_FFN = range(7)
B_X, B_XB, B_XB2, B_HB, B_HB2, B_Q, B_K, B_V, B_ATT, B_LOGITS, B_KCACHE, B_VCACHE, B_TMP1 = range(13)


class Config(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len",
                 "shared_weights")]


def build():
    """Compile liboracle.so with gcc (a few seconds)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    fp = C.POINTER(C.c_float)
    u8p = C.POINTER(C.c_uint8)
    i32p = C.POINTER(C.c_int32)
    vp = C.c_void_p
    sig = {
        "orc_quant_nbytes": (C.c_int64, [C.c_int64]),
        "orc_quant_encode": (None, [fp, C.c_int64, u8p]),
        "orc_quant_decode": (None, [u8p, C.c_int64, C.c_int64, fp]),
        "orc_rms": (None, [fp, fp, C.c_int]),
        "orc_wns_i8": (None, [fp, fp, u8p, C.c_int64, fp, C.c_int]),
        "orc_matmul_i8": (None, [fp, fp, u8p, C.c_int64, C.c_int, C.c_int]),
        "orc_matmul_i8_aligned": (None, [fp, fp, u8p, C.c_int64, C.c_int, C.c_int]),
        "orc_matmul_i8_unaligned": (None, [fp, fp, u8p, C.c_int64, C.c_int, C.c_int]),
        "orc_matmul_f32": (None, [fp, fp, fp, C.c_int64, C.c_int, C.c_int]),
        "orc_rope_table": (None, [fp, fp, C.c_int, C.c_int, C.c_int]),
        "orc_rope": (None, [fp, fp, fp, fp, C.c_int, C.c_int, C.c_int]),
        "orc_attention_loop": (None, [fp, fp, fp, fp, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_int,
                                      C.c_int, C.c_int]),
        "orc_exp_sum_normalize": (None, [fp, fp, C.c_int, C.c_int64, C.c_int]),
        "orc_accum_weighted_value": (None, [fp, fp, fp, C.c_int, C.c_int, C.c_int64, C.c_int, C.c_int,
                                            C.c_int64]),
        "orc_accum": (None, [fp, fp, C.c_int]),
        "orc_silu_table": (None, [fp]),
        "orc_silu_lookup": (C.c_float, [fp, C.c_float]),
        "orc_silu": (None, [fp, fp, fp, C.c_int]),
        "orc_argmax": (C.c_int, [fp, C.c_int]),
        "orc_model_new": (vp, [C.POINTER(Config)]),
        "orc_model_free": (None, [vp]),
        "orc_tensor_floats": (C.c_int64, [C.POINTER(Config), C.c_int]),
        "orc_tensor_name": (C.c_char_p, [C.c_int]),
        "orc_model_set_quant": (C.c_int, [vp, C.c_int, u8p, C.c_int64]),
        "orc_model_set_emb": (C.c_int, [vp, fp, C.c_int64]),
        "orc_model_set_wcls": (C.c_int, [vp, fp, C.c_int64]),
        "orc_model_quant_ptr": (u8p, [vp, C.c_int]),
        "orc_model_emb_ptr": (fp, [vp]),
        "orc_model_wcls_ptr": (fp, [vp]),
        "orc_model_buffer": (fp, [vp, C.c_int]),
        "orc_model_reset": (None, [vp]),
        "orc_model_enable_taps": (C.c_int, [vp]),
        "orc_model_tap": (fp, [vp, C.c_int, C.c_int]),
        "orc_forward": (None, [vp, C.c_int, C.c_int]),
        "orc_forward_layers": (None, [vp, C.c_int, C.c_int, C.c_int]),
        "orc_generate_greedy": (C.c_int, [vp, i32p, C.c_int, C.c_int, i32p, fp, C.POINTER(C.c_double)]),
        "orc_find_max": (None, [fp, C.c_int, fp, C.c_int64, C.c_int]),
        "orc_sampler_new": (vp, [C.c_int64, C.c_int]),
        "orc_sampler_free": (None, [vp]),
        "orc_sampler_next_bits": (C.c_int32, [vp, C.c_int]),
        "orc_sampler_next_float": (C.c_float, [vp]),
        "orc_sample": (C.c_int, [vp, fp, C.c_int]),
        "orc_sample_topp": (C.c_int, [vp, fp, C.c_int, C.c_float]),
        "orc_sample_coin": (C.c_int, [fp, C.c_int, C.c_float]),
        "orc_sample_topp_coin": (C.c_int, [vp, fp, C.c_int, C.c_float, C.c_float]),
        "orc_sample_step": (C.c_int, [vp, fp, C.c_int, C.c_float, C.c_float]),
        "orc_generate": (C.c_int, [vp, i32p, C.c_int, C.c_int, C.c_float, C.c_float, C.c_int64, i32p,
                                   C.POINTER(C.c_double)]),
        "orc_write_quant_file": (C.c_int, [C.c_char_p, u8p, C.c_int64]),
        "orc_read_quant_file": (C.c_int64, [C.c_char_p, u8p, C.c_int64]),
        "orc_load_checkpoint": (vp, [C.c_char_p, C.c_int, C.c_char_p, C.c_int]),
        "orc_synth_fill": (None, [C.c_uint64, C.c_uint32, C.c_int64, C.c_int64, C.c_float, fp]),
        "orc_model_fill_synth": (None, [vp, C.c_uint64, C.c_float]),
        "orc_synth_prompt": (None, [C.c_uint64, C.c_int, C.c_int, i32p]),
        "orc_num_threads": (C.c_int, []),
    }
    for name, (res, args) in sig.items():
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args
    _lib = L
    return L


def _fp(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u8(a):
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def _i32(a):
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_int32))


# ---- sampling ----------------------------------------------------------------------------
class Sampler:
    """J/Sampler.java: java.util.Random(seed) + the ProbIndex array that outlives a call."""

    def __init__(self, rng_seed, vocab_size):
        self.n = vocab_size
        self.h = lib().orc_sampler_new(rng_seed, vocab_size)
        if not self.h:
            raise MemoryError("orc_sampler_new")

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_sampler_free(self.h)
            self.h = None

    def next_bits(self, bits):
        return lib().orc_sampler_next_bits(self.h, bits)

    def next_float(self):
        return lib().orc_sampler_next_float(self.h)

    def sample(self, probs, coin=None):
        probs = np.ascontiguousarray(probs, dtype=np.float32)
        if coin is None:
            return lib().orc_sample(self.h, _fp(probs), probs.size)
        return lib().orc_sample_coin(_fp(probs), probs.size, coin)

    def sample_topp(self, probs, topp, coin=None):
        probs = np.ascontiguousarray(probs, dtype=np.float32)
        if coin is None:
            return lib().orc_sample_topp(self.h, _fp(probs), probs.size, topp)
        return lib().orc_sample_topp_coin(self.h, _fp(probs), probs.size, topp, coin)

    def step(self, logits, temperature, topp):
        """J/Run.java:643-665 on a copy; returns (next, the array after the step)."""
        a = np.array(logits, dtype=np.float32, copy=True)
        nxt = lib().orc_sample_step(self.h, _fp(a), a.size, temperature, topp)
        return nxt, a


def find_max(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(1, dtype=np.float32)
    lib().orc_find_max(_fp(out), 0, _fp(x), 0, x.size)
    return float(out[0])


# ---- codec -------------------------------------------------------------------------------

def quant_nbytes(n):
    return lib().orc_quant_nbytes(n)


def quant_encode(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(quant_nbytes(x.size), dtype=np.uint8)
    lib().orc_quant_encode(_fp(x), x.size, _u8(out))
    return out


def quant_decode(enc, float_index, size):
    out = np.empty(size, dtype=np.float32)
    lib().orc_quant_decode(_u8(enc), float_index, size, _fp(out))
    return out


# ---- ops ---------------------------------------------------------------------------------

def rms(x):
    s = np.zeros(1, dtype=np.float32)
    lib().orc_rms(_fp(s), _fp(x), x.size)
    return s


def wns_i8(x, enc, weight_index, ss):
    out = np.empty_like(x)
    lib().orc_wns_i8(_fp(out), _fp(x), _u8(enc), weight_index, _fp(ss), x.size)
    return out


def matmul_i8(x, enc, weight_index, n, d, variant=""):
    out = np.empty(d, dtype=np.float32)
    f = getattr(lib(), "orc_matmul_i8" + variant)
    f(_fp(out), _fp(x), _u8(enc), weight_index, n, d)
    return out


def matmul_f32(x, w, weight_index, n, d):
    out = np.empty(d, dtype=np.float32)
    lib().orc_matmul_f32(_fp(out), _fp(x), _fp(w), weight_index, n, d)
    return out


def rope_table(dim, head_size, seq_len):
    c = np.empty((dim // 2) * seq_len, dtype=np.float32)
    s = np.empty_like(c)
    lib().orc_rope_table(_fp(c), _fp(s), dim, head_size, seq_len)
    return c, s


def rope(q, k, cos_t, sin_t, pos, dim, kv_dim):
    lib().orc_rope(_fp(q), _fp(k), _fp(cos_t), _fp(sin_t), pos, dim, kv_dim)


def silu_table():
    t = np.empty(8192, dtype=np.float32)
    lib().orc_silu_table(_fp(t))
    return t


def silu_lookup(table, v):
    return float(lib().orc_silu_lookup(_fp(table), C.c_float(v)))


def silu(hb, hb2, table):
    lib().orc_silu(_fp(hb), _fp(hb2), _fp(table), hb.size)


def argmax(logits):
    return lib().orc_argmax(_fp(logits), logits.size)


def synth_fill(seed, stream, first, n, sigma=0.02):
    out = np.empty(n, dtype=np.float32)
    lib().orc_synth_fill(seed, stream, first, n, C.c_float(sigma), _fp(out))
    return out


def synth_prompt(seed, n, vocab):
    out = np.empty(n, dtype=np.int32)
    lib().orc_synth_prompt(seed, n, vocab, _i32(out))
    return out


# ---- model -------------------------------------------------------------------------------

class Model:
    """Owns an orc_model; numpy views expose its tensors and activation buffers."""

    def __init__(self, cfg=None, handle=None, **kw):
        L = lib()
        if handle is None:
            if cfg is None:
                cfg = Config(**kw)
            handle = L.orc_model_new(C.byref(cfg))
            if not handle:
                raise MemoryError("orc_model_new failed")
        self.h = handle
        self.cfg = cfg
        self.head_size = cfg.dim // cfg.n_heads
        self.kv_dim = cfg.dim * cfg.n_kv_heads // cfg.n_heads

    @classmethod
    def load(cls, bin_path, write_caches=True):
        L = lib()
        err = C.create_string_buffer(512)
        h = L.orc_load_checkpoint(bin_path.encode(), 1 if write_caches else 0, err, 512)
        if not h:
            raise RuntimeError(err.value.decode())
        # read the header again for the config
        hdr = np.fromfile(bin_path, dtype="<i4", count=7)
        cfg = Config(int(hdr[0]), int(hdr[1]), int(hdr[2]), int(hdr[3]), int(hdr[4]), abs(int(hdr[5])),
                     int(hdr[6]), 1 if hdr[5] > 0 else 0)
        return cls(cfg=cfg, handle=h)

    def close(self):
        if self.h:
            lib().orc_model_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def tensor_floats(self, t):
        return lib().orc_tensor_floats(C.byref(self.cfg), t)

    def quant(self, t):
        n = quant_nbytes(self.tensor_floats(t))
        p = lib().orc_model_quant_ptr(self.h, t)
        return np.ctypeslib.as_array(p, shape=(n,))

    def emb(self):
        return np.ctypeslib.as_array(lib().orc_model_emb_ptr(self.h), shape=(self.cfg.vocab_size * self.cfg.dim,))

    def wcls(self):
        return np.ctypeslib.as_array(lib().orc_model_wcls_ptr(self.h), shape=(self.cfg.vocab_size * self.cfg.dim,))

    def set_quant(self, t, b):
        b = np.ascontiguousarray(b, dtype=np.uint8)
        rc = lib().orc_model_set_quant(self.h, t, _u8(b), b.size)
        if rc:
            raise ValueError("set_quant rc=%d" % rc)

    def buffer(self, which):
        c = self.cfg
        n = {B_X: c.dim, B_XB: c.dim, B_XB2: c.dim, B_HB: c.hidden_dim, B_HB2: c.hidden_dim, B_Q: c.dim,
             B_K: self.kv_dim, B_V: self.kv_dim, B_ATT: c.n_heads * c.seq_len, B_LOGITS: c.vocab_size,
             B_KCACHE: c.n_layers * c.seq_len * self.kv_dim, B_VCACHE: c.n_layers * c.seq_len * self.kv_dim,
             B_TMP1: max(c.dim, c.vocab_size) * 4}[which]
        return np.ctypeslib.as_array(lib().orc_model_buffer(self.h, which), shape=(n,))

    def enable_taps(self):
        if lib().orc_model_enable_taps(self.h):
            raise MemoryError("taps")

    def tap(self, which, layer):
        n = self.cfg.hidden_dim if which == TAP_HB else self.kv_dim if which in (TAP_K, TAP_V) else self.cfg.dim
        return np.ctypeslib.as_array(lib().orc_model_tap(self.h, which, layer), shape=(n,))

    def fill_synth(self, seed, sigma=0.02):
        lib().orc_model_fill_synth(self.h, seed, C.c_float(sigma))

    def reset(self):
        lib().orc_model_reset(self.h)

    def forward(self, token, pos):
        lib().orc_forward(self.h, token, pos)
        return self.buffer(B_LOGITS)

    def forward_layers(self, token, pos, n_layers):
        lib().orc_forward_layers(self.h, token, pos, n_layers)

    def generate_greedy(self, prompt, steps, want_logits=False):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        cap = self.cfg.seq_len if steps <= 0 or steps > self.cfg.seq_len else steps
        out = np.zeros(cap, dtype=np.int32)
        logits = np.zeros((cap, self.cfg.vocab_size), dtype=np.float32) if want_logits else None
        sec = C.c_double(0)
        n = lib().orc_generate_greedy(self.h, _i32(prompt), prompt.size, steps, _i32(out),
                                      _fp(logits) if want_logits else None, C.byref(sec))
        return out[:n], (logits[:n] if want_logits else None), sec.value

    def generate(self, prompt, steps, temperature, topp, rng_seed):
        """J/Run.java:611-685 with the sampler of J/Run.java:620."""
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        cap = self.cfg.seq_len if steps <= 0 or steps > self.cfg.seq_len else steps
        out = np.zeros(cap, dtype=np.int32)
        sec = C.c_double(0)
        n = lib().orc_generate(self.h, _i32(prompt), prompt.size, steps, temperature, topp, rng_seed,
                               _i32(out), C.byref(sec))
        return out[:n], sec.value
