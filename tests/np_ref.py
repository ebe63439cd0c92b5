"""Independent numpy checks for the oracle: a byte-level parser of the quant format and a
textbook float64 Llama-2 forward.  Shares no code with oracle/ or with the HIP library."""
import numpy as np


def parse_quant(enc):
    """264-byte groups: big-endian fp32 min, max, then 256 unsigned codes."""
    g = np.asarray(enc, dtype=np.uint8).reshape(-1, 264)
    mn = g[:, 0:4].copy().view(">f4").astype(np.float32).reshape(-1)
    mx = g[:, 4:8].copy().view(">f4").astype(np.float32).reshape(-1)
    return mn, mx, g[:, 8:]


def dequant64(enc, n):
    """Mathematical value of every weight, float64: min + code/255*(max-min)."""
    mn, mx, codes = parse_quant(enc)
    w = mn.astype(np.float64)[:, None] + codes.astype(np.float64) / 255.0 * (mx.astype(np.float64) - mn.astype(np.float64))[:, None]
    return w.reshape(-1)[:n]


def silu_lut64(v):
    """The reference's 8192-entry sigmoid table with linear interpolation (index step 819, not 819.2)."""
    i = np.arange(8192)
    table = (1.0 / (1.0 + np.exp(-((i / 8192.0) * 10.0 - 5.0)))).astype(np.float32).astype(np.float64)
    v = np.asarray(v, dtype=np.float64)
    p = (v + 5.0) * 819.0
    idx = np.clip(p.astype(np.int64), 0, 8190)
    interp = table[idx] + (p - idx) * (table[idx + 1] - table[idx])
    exact = 1.0 / (1.0 + np.exp(-v))
    return np.where((p > 0) & (p < 8191), interp, exact)


def sigmoid64(v):
    return 1.0 / (1.0 + np.exp(-np.asarray(v, dtype=np.float64)))


class TextbookLlama:
    """Plain float64 Llama-2 decoder (RMSNorm, interleaved-pair RoPE, softmax attention, SwiGLU)."""

    def __init__(self, cfg, tensors, emb, wcls, sigmoid=silu_lut64):
        self.c = cfg
        self.t = tensors  # dict name -> float64 flat arrays (dequantized)
        self.emb = np.asarray(emb, dtype=np.float64).reshape(cfg["vocab_size"], cfg["dim"])
        self.wcls = np.asarray(wcls, dtype=np.float64).reshape(cfg["vocab_size"], cfg["dim"])
        self.sigmoid = sigmoid
        L, S = cfg["n_layers"], cfg["seq_len"]
        self.kv_dim = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
        self.K = np.zeros((L, S, self.kv_dim))
        self.V = np.zeros((L, S, self.kv_dim))

    @staticmethod
    def rmsnorm(x, w):
        return w * (x / np.sqrt(np.mean(x * x) + 1e-5))

    def rope(self, v, pos, hs):
        out = v.copy()
        i = np.arange(0, v.size, 2)
        theta = 10000.0 ** (-((i % hs) / hs))
        ang = pos * theta
        out[0::2] = v[0::2] * np.cos(ang) - v[1::2] * np.sin(ang)
        out[1::2] = v[0::2] * np.sin(ang) + v[1::2] * np.cos(ang)
        return out

    def forward(self, token, pos):
        c = self.c
        dim, hid, H = c["dim"], c["hidden_dim"], c["n_heads"]
        hs = dim // H
        kv_dim = self.kv_dim
        kv_mul = H // c["n_kv_heads"]
        x = self.emb[token].copy()
        for l in range(c["n_layers"]):
            xb = self.rmsnorm(x, self.t["rms_att"][l * dim:(l + 1) * dim])
            wq = self.t["wq"][l * dim * dim:(l + 1) * dim * dim].reshape(dim, dim)
            wk = self.t["wk"][l * dim * kv_dim:(l + 1) * dim * kv_dim].reshape(kv_dim, dim)
            wv = self.t["wv"][l * dim * kv_dim:(l + 1) * dim * kv_dim].reshape(kv_dim, dim)
            q = self.rope(wq @ xb, pos, hs)
            k = self.rope(wk @ xb, pos, hs)
            v = wv @ xb
            self.K[l, pos] = k
            self.V[l, pos] = v
            att_out = np.zeros(dim)
            for h in range(H):
                kh = (h // kv_mul) * hs
                s = self.K[l, :pos + 1, kh:kh + hs] @ q[h * hs:(h + 1) * hs] / np.sqrt(hs)
                p = np.exp(s - s.max())
                p /= p.sum()
                att_out[h * hs:(h + 1) * hs] = p @ self.V[l, :pos + 1, kh:kh + hs]
            wo = self.t["wo"][l * dim * dim:(l + 1) * dim * dim].reshape(dim, dim)
            x = x + wo @ att_out
            xb = self.rmsnorm(x, self.t["rms_ffn"][l * dim:(l + 1) * dim])
            w1 = self.t["w1"][l * dim * hid:(l + 1) * dim * hid].reshape(hid, dim)
            w3 = self.t["w3"][l * dim * hid:(l + 1) * dim * hid].reshape(hid, dim)
            w2 = self.t["w2"][l * dim * hid:(l + 1) * dim * hid].reshape(dim, hid)
            h1 = w1 @ xb
            h3 = w3 @ xb
            x = x + w2 @ (h1 * self.sigmoid(h1) * h3)
        x = self.rmsnorm(x, self.t["rms_final"][:dim])
        return self.wcls @ x
