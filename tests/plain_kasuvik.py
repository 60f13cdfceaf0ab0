"""A plain, slow implementation of the Kasuvik decoder in NumPy float64, one function per mechanism,
written from the design's equations and sharing no code with the package.  Tests compare the engine
with it; it reads a configuration as the dictionary config.json holds and tensors by their checkpoint
names.

Notation: T tokens of one sequence, positions 0 .. T-1; W x means ``x @ W.T`` for a stored [out, in].
"""
import json
import struct

import numpy as np


# ----------------------------------------------------------------------------------- files
def read_safetensors(path):
    """name -> float64 (or int64) array; bfloat16 is widened exactly."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        raw, shape = data[lo:hi], info["shape"]
        if info["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif info["dtype"] == "F32":
            a = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif info["dtype"] == "I32":
            a = np.frombuffer(raw, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {info['dtype']}")
        out[name] = a.reshape(shape)
    return out


# ------------------------------------------------------------------------------ elementwise
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w None: no weight)."""
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * w


def embedding(table, tokens, scale):
    return table[np.asarray(tokens)] * scale


def short_conv(u, w, bias=None):
    """Causal convolution over time per channel.  u [T, C], w [C, taps]: the last column multiplies the
    current token, zeros stand before the sequence's start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), u], 0)
    y = np.zeros((T, C))
    for j in range(taps):
        y += padded[j:j + T] * w[:, j]
    return y if bias is None else y + bias


def rotate_interleaved(x, positions, dims, base):
    """x [T, heads, dim]: the pairs (2i, 2i+1), i < dims/2, are turned by the angle p * base^(-2i/dims);
    entries from ``dims`` on pass."""
    out = x.copy()
    i = np.arange(dims // 2)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * base ** (-2.0 * i / dims)      # [T, dims/2]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# --------------------------------------------------------------------------------- attention
def window_pool_attention(q, k, v, scale, temp, window, pool):
    """q [T, H, d], k [T, G, d], v [T, G, dv] as the cache holds them.  Query i sees the tokens j with
    0 <= i - j < window and, beside them, one mean key and mean value for every block of ``pool`` tokens
    b*pool .. b*pool + pool - 1 that ends at or before i - window; one softmax over both."""
    T, H, d = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    nblocks = T // pool
    kp = k[:nblocks * pool].reshape(nblocks, pool, G, d).mean(1) if nblocks else np.zeros((0, G, d))
    vp = v[:nblocks * pool].reshape(nblocks, pool, G, -1).mean(1) if nblocks else np.zeros((0, G, v.shape[2]))
    for i in range(T):
        lo = max(0, i - window + 1)
        seen = sum(1 for b in range(nblocks) if b * pool + pool - 1 <= i - window)
        for h in range(H):
            g = h // (H // G)
            keys = np.concatenate([kp[:seen, g], k[lo:i + 1, g]], 0)
            vals = np.concatenate([vp[:seen, g], v[lo:i + 1, g]], 0)
            s = keys @ q[i, h] * scale * temp[h]
            p = np.exp(s - s.max())
            out[i, h] = (p / p.sum()) @ vals
    return out


def conv_attention(h, t, pre, c):
    """The left half of a ``parallel`` mixer: projections with biases, a short convolution on q, k and v,
    rotation of q and k, attention over the window and the pooled blocks, output projection."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    proj = {}
    for n in ("q", "k", "v"):
        u = h @ t[pre + n].T + t[pre + n + ".b"]
        proj[n] = short_conv(u, t[pre + n + ".conv"])
    pos = np.arange(T)
    q = rotate_interleaved(proj["q"].reshape(T, H, d), pos, c["rot"]["dims"], c["rot"]["base"])
    k = rotate_interleaved(proj["k"].reshape(T, G, d), pos, c["rot"]["dims"], c["rot"]["base"])
    v = proj["v"].reshape(T, G, dv)
    o = window_pool_attention(q, k, v, c["scale"], t[pre + "temp"], c["mask"]["size"], c["mask"]["pool"])
    return o.reshape(T, H * dv) @ t[pre + "o"].T


# ----------------------------------------------------------------------------- selective scan
def selective_scan(x, dt, A, B, C, D):
    """x, dt [T, c]; A [c, n]; B, C [T, n]; D [c].  S <- exp(dt A) S + dt x B;  y = S C + D x."""
    T, ch = x.shape
    S = np.zeros_like(A)
    y = np.zeros((T, ch))
    for i in range(T):
        S = np.exp(dt[i][:, None] * A) * S + (dt[i] * x[i])[:, None] * B[i][None, :]
        y[i] = S @ C[i] + D * x[i]
    return y


def mamba(h, t, pre, c):
    """The right half of a ``parallel`` mixer."""
    inner, n, r = c["inner"], c["state"], c["dt_rank"]
    xz = h @ t[pre + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(short_conv(x, t[pre + "conv"], t[pre + "conv.b"]))
    p = x @ t[pre + "x"].T
    dt, B, C = p[:, :r], p[:, r:r + n], p[:, r + n:r + 2 * n]
    dt = softplus(dt @ t[pre + "dt"].T + t[pre + "dt.b"])
    y = selective_scan(x, dt, -np.exp(t[pre + "A_log"]), B, C, t[pre + "D"])
    return (y * silu(z)) @ t[pre + "o"].T


def parallel_mixer(h, t, pre, c, eps):
    left = conv_attention(h, t, pre + "left.", c["left"])
    right = mamba(h, t, pre + "right.", c["right"])
    return 0.5 * (rms_norm(left, t[pre + "left.out"], eps) + rms_norm(right, t[pre + "right.out"], eps))


# --------------------------------------------------------------------------------- delta rule
def delta_rule(r, k, v, w, a):
    """All [T, heads, d].  With u = k / sqrt(|k|^2 + 1e-6):
    S_t = diag(w_t) S_{t-1} - (a_t * u_t) (u_t^T S_{t-1}) + k_t v_t^T;  o_t = S_t^T r_t."""
    T, H, d = k.shape
    out = np.zeros((T, H, v.shape[2]))
    for hd in range(H):
        S = np.zeros((d, v.shape[2]))
        for i in range(T):
            u = k[i, hd] / np.sqrt(np.sum(k[i, hd] ** 2) + 1e-6)
            S = w[i, hd][:, None] * S - np.outer(a[i, hd] * u, u @ S) + np.outer(k[i, hd], v[i, hd])
            out[i, hd] = S.T @ r[i, hd]
    return out


def general_delta(h, t, pre, c, eps):
    T = h.shape[0]
    H, d = c["heads"], c["dim"]
    r = (h @ t[pre + "r"].T).reshape(T, H, d)
    k = (h @ t[pre + "k"].T).reshape(T, H, d)
    v = (h @ t[pre + "v"].T).reshape(T, H, d)
    w = np.exp(-np.exp(-0.5) * sigmoid(np.tanh(h @ t[pre + "w1"].T) @ t[pre + "w2"].T + t[pre + "w0"])).reshape(T, H, d)
    a = sigmoid(h @ t[pre + "a"].T + t[pre + "a.b"]).reshape(T, H, d)
    o = rms_norm(delta_rule(r, k, v, w, a), None, eps).reshape(T, H * d)
    o = o * t[pre + "norm"] * sigmoid(h @ t[pre + "g"].T)
    return o @ t[pre + "o"].T


# ------------------------------------------------------------------------------ feed-forward
def dense_ff(h, t, pre):
    return (np.maximum(h @ t[pre + "gate"].T, 0.0) * (h @ t[pre + "up"].T)) @ t[pre + "down"].T


# ----------------------------------------------------------------------------------- a model
def hidden_states(cfg, t, tokens, after_layer=None):
    """The residual stream after the last layer [T, width]; ``after_layer`` (a list) receives it after every layer."""
    eps = cfg["norm"]["eps"]
    x = embedding(t["embed"], tokens, cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm(x, t[p + "norm1"], eps)
        if layer["type"] == "parallel":
            m = parallel_mixer(h, t, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "general_delta":
            m = general_delta(h, t, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(m, t[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(layer["mlp"]["kind"])
            f = dense_ff(rms_norm(x, t[p + "norm2"], eps), t, p + "mlp.")
            x = x + rms_norm(f, t[p + "norm2b"], eps)
        if after_layer is not None:
            after_layer.append(x.copy())
    return x


def logits(cfg, t, tokens, after_layer=None):
    x = hidden_states(cfg, t, tokens, after_layer)
    return rms_norm(x, t["final.norm"], cfg["norm"]["eps"]) @ t["head"].T
