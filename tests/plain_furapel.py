"""A plain, slow implementation of the Furapel decoder in NumPy float64, one function per mechanism, written
from the design's equations and sharing no code with the package.  Tests compare the engine with it; it reads a
configuration as the dictionary config.json holds and tensors by their checkpoint names.

Notation: T tokens of one sequence at positions 0 .. T-1; a stored matrix W is [out, in] and "W x" is
``x @ W.T``.  A layer is x <- x + mixer(n1(x)) + ff(n2(x)) with n(x) = tanh(alpha x) * w + b; a stretch of layers
may run several times in a row, each pass led in by x <- W_in [x ; x0] (x0: the scaled embedding).
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


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def dynamic_tanh(x, alpha, w, b):
    """tanh(alpha x) * w + b: a norm without statistics."""
    return np.tanh(float(alpha) * x) * w + b


def softmax(z):
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


# ---------------------------------------------------------------------------------- rotation
def yarn_frequencies(dims, base, scaling=None):
    """(frequency of every pair [dims/2], factor on cos and sin).  Plain: f_i = base^(-2i/dims), factor 1.
    With scaling (factor s, original length L, fast and slow turn counts): pair i keeps f_i where it turns fast and
    takes f_i / s where it turns slowly, with a linear ramp between the pairs at which a length of L holds
    ``fast`` and ``slow`` turns; cos and sin grow by 0.1 ln s + 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    s, L = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):
        return dims * np.log(L / (2.0 * np.pi * turns)) / (2.0 * np.log(base))

    lo = max(np.floor(pair_of(float(scaling["fast"]))), 0.0)
    hi = min(np.ceil(pair_of(float(scaling["slow"]))), dims - 1.0)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s * ramp + f * (1.0 - ramp), 0.1 * np.log(s) + 1.0


def rotate_half(x, positions, dims, freqs, factor):
    """x [T, heads, dim]: entry i < dims/2 is paired with entry i + dims/2 and the pair is turned by
    position * freqs[i]; entries from ``dims`` on pass."""
    if not dims:
        return x.copy()
    half = dims // 2
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    c, s = (np.cos(ang) * factor)[:, None, :], (np.sin(ang) * factor)[:, None, :]
    out = x.copy()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


# --------------------------------------------------------------------------------- attention
def visible(T, window=0):
    """[T, T] bool: query i sees key j when j <= i and, with a window, i - j < window."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    ok = j <= i
    return ok & (i - j < window) if window else ok


def attend(q, k, v, scale, window=0):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; query head h reads key head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    mask = visible(T, window)
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        z = (q[:, h] @ k[:, g].T) * scale
        z = np.where(mask, z, -np.inf)
        out[:, h] = softmax(z) @ v[:, g]
    return out


def gated_attention(h, w, pre, m, positions=None):
    """Grouped-query attention with a rotation on part of each head and one sigmoid gate per head and token."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = np.arange(T) if positions is None else positions
    q = (h @ w[pre + "q"].T).reshape(T, H, d)
    k = (h @ w[pre + "k"].T).reshape(T, G, d)
    v = (h @ w[pre + "v"].T).reshape(T, G, dv)
    rot = m.get("rot") or {}
    dims = rot.get("dims", 0)
    if dims:
        f, factor = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
        q, k = rotate_half(q, positions, dims, f, factor), rotate_half(k, positions, dims, f, factor)
    o = attend(q, k, v, m["scale"], 0)
    gate = sigmoid(h @ w[pre + "g"].T)                      # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def latent_attention(h, w, pre, m, eps):
    """Keys and values of every head are made from one small normed vector per token; no positions; a window."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, d)
    c = unit_rms(h @ w[pre + "dkv"].T, eps) * w[pre + "dkv.norm"]
    k = (c @ w[pre + "uk"].T).reshape(T, H, d)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    o = attend(q, k, v, m["scale"], m["mask"]["size"])
    return o.reshape(T, H * dv) @ w[pre + "o"].T


# --------------------------------------------------------------------------- matrix memory
def soft_cap(z, cap):
    return cap * np.tanh(z / cap)


def matrix_memory(q, k, v, log_in, log_keep, state=None):
    """One head, token by token.  q, k [T, d] (q already scaled), v [T, dv], log_in, log_keep [T].
    state = (S [d, dv], n [d], m) or None for (0, 0, 0).  Returns (o [T, dv], state)."""
    T, d = k.shape
    S, n, m = (np.zeros((d, v.shape[1])), np.zeros(d), 0.0) if state is None else state
    out = np.zeros((T, v.shape[1]))
    for t in range(T):
        m_new = max(log_keep[t] + m, log_in[t])
        keep, take = np.exp(log_keep[t] + m - m_new), np.exp(log_in[t] - m_new)
        S = keep * S + take * np.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        out[t] = (S.T @ q[t]) / (max(abs(n @ q[t]), np.exp(-m)) + 1e-6)
    return out, (S, n, m)


def mlstm(h, w, pre, m, eps):
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, d)
    v = (h @ w[pre + "v"].T).reshape(T, H, dv)
    log_in = soft_cap(h @ w[pre + "i"].T + w[pre + "i.b"], cap)                 # [T, H]
    log_keep = log_sigmoid(soft_cap(h @ w[pre + "f"].T + w[pre + "f.b"], cap))
    o = np.zeros((T, H, dv))
    for a in range(H):
        o[:, a], _ = matrix_memory(q[:, a], k[:, a], v[:, a], log_in[:, a], log_keep[:, a])
    o = unit_rms(o, eps).reshape(T, H * dv) * w[pre + "norm"]
    o = o * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


# ------------------------------------------------------------------------------ feed-forward
def route(h, w_router, top):
    """-> (chosen experts [T, top], their weights [T, top]): softmax over all experts, the ``top`` largest,
    weights as they are."""
    s = softmax(h @ w_router.T)
    order = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return order, np.take_along_axis(s, order, axis=-1)


def expert(h, up, down):
    return np.maximum(h @ up.T, 0.0) ** 2 @ down.T


def mixture(h, w, pre, mlp):
    T = h.shape[0]
    chosen, weight = route(h, w[pre + "router"], mlp["router"]["top"])
    out = np.zeros((T, w[pre + "e0.down"].shape[0]))
    for t in range(T):
        for e, g in zip(chosen[t], weight[t]):
            out[t] += g * expert(h[t], w[pre + f"e{e}.up"], w[pre + f"e{e}.down"])
    return out


# ----------------------------------------------------------------------------------- model
def layer_runs(raw):
    """[(layer index, leads a pass?)] in the order the layers run."""
    n = len(raw["layers"])
    loop = raw.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def norm_of(w, name, x):
    return dynamic_tanh(x, w[name + ".alpha"], w[name], w[name + ".b"])


def forward(raw, w, tokens, trace=None):
    """Logits [T, vocab] of one sequence; ``trace``: a list that receives the stream after every layer run."""
    eps = raw["norm"]["eps"]
    x0 = w["embed"][np.asarray(tokens)] * raw["embedding"]["scale"]
    x = x0.copy()
    for i, leads in layer_runs(raw):
        L, p = raw["layers"][i], f"l{i}."
        if leads:
            x = np.concatenate([x, x0], axis=-1) @ w["loop.in"].T
        h = norm_of(w, p + "norm1", x)
        kind, m = L["type"], L["mixer"]
        if kind == "attention":
            y = gated_attention(h, w, p + "mix.", m)
        elif kind == "latent_attention":
            y = latent_attention(h, w, p + "mix.", m, eps)
        elif kind == "mlstm":
            y = mlstm(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(kind)
        if L.get("mlp"):
            y = y + mixture(norm_of(w, p + "norm2", x), w, p + "mlp.", L["mlp"])
        x = x + y
        if trace is not None:
            trace.append(x.copy())
    return norm_of(w, "final.norm", x) @ w["head"].T * raw.get("logit_scale", 1.0)
