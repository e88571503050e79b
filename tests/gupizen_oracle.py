"""Plain, slow float64 restatement of the Gupizen design that zig_gpt2_amd/lm.py serves.

One function per mechanism, numpy only, written from the design's equations; it shares no code with the product path
(zig_gpt2_amd/ is not imported).  Weights are a dict name -> numpy array with the checkpoint's tensor names, the
configuration is the dict of config.json.

Notation: x residual stream [T, W]; h a sublayer's input; positions count from 0 per sequence;
rms(v) = sqrt(mean(v^2) + eps).  Every function that carries something from token to token takes the state the tokens
before left (None: the start of a sequence) and returns the new one.
"""
import math

import numpy as np

F = np.float64


def rms_unit(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def norm_around_zero(v, w, eps):
    return rms_unit(v, eps) * (1.0 + w)


def norm_plain(v, w, eps):
    return rms_unit(v, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


# ----------------------------------------------------------------------------------------------- causal convolution over time
def causal_conv(v, w, tail):
    """v [T, C], w [C, taps] (last column multiplies the current token), tail: the taps - 1 inputs before v (None: zeros).
    Returns (conv [T, C], new tail)."""
    taps = w.shape[1]
    T, C = v.shape
    before = np.zeros((taps - 1, C), F) if tail is None else tail
    full = np.concatenate([before, v], axis=0)
    out = np.zeros((T, C), F)
    for j in range(taps):
        out += full[j:j + T] * w[:, j][None, :]
    return out, full[full.shape[0] - (taps - 1):].copy()


# ----------------------------------------------------------------------------------------------- rotary positions
def band_scaled_frequencies(rot):
    """base^(-2i/dims), then the wavelength bands: short waves stay, long waves are slowed by `factor`, a blend between."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], F)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = f.copy()
        for i, fi in enumerate(f):
            wave = 2.0 * math.pi / fi
            if wave < orig / high:
                out[i] = fi
            elif wave > orig / low:
                out[i] = fi / factor
            else:
                s = (orig / wave - low) / (high - low)
                out[i] = (1.0 - s) * fi / factor + s * fi
        f = out
    return f


def angles(positions, freq):
    """32-bit products of position and frequency, as the product path forms them."""
    return (np.asarray(positions, np.float32)[:, None] * freq.astype(np.float32)[None, :]).astype(F)


def turn_pairs(v, ang, dims):
    """v [T, heads, n]: entries (2i, 2i+1) for 2i < dims turn by ang[t, i]; the rest pass."""
    out = v.copy()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ----------------------------------------------------------------------------------------------- windowed attention with sink
def window_attention_weights(q, k, m, sink, talk, q_pos, k_pos):
    """Softmax weights [heads, queries, keys]: scaled scores inside the window, exp(sink) in the denominator only, then the
    heads' weights mixed by `talk`."""
    H, G = int(m["heads"]), int(m["kv_heads"])
    rep = H // G
    s = np.einsum("thd,nhd->htn", q, np.repeat(k, rep, axis=1)) * float(m["scale"])
    dist = np.asarray(q_pos)[:, None] - np.asarray(k_pos)[None, :]
    ok = dist >= 0
    if m.get("mask") and m["mask"].get("size"):
        ok &= dist < int(m["mask"]["size"])
    s = np.where(ok[None], s, -np.inf)
    top = np.maximum(s.max(axis=-1, keepdims=True), sink[:, None, None])
    e = np.exp(s - top)
    a = e / (e.sum(axis=-1, keepdims=True) + np.exp(sink[:, None, None] - top))
    return np.einsum("hg,gtn->htn", talk, a)


def window_attention(h, w, p, m, positions, cache):
    """The left branch.  cache: (rotated keys [n, G, dim], rotated values [n, G, vdim]) of the tokens before, or None."""
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    rot = m["rot"]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, G, D)
    v = (h @ w[p + "v"].T).reshape(T, G, V)
    ang = angles(positions, band_scaled_frequencies(rot))
    q, k = turn_pairs(q, ang, int(rot["dims"])), turn_pairs(k, ang, int(rot["dims"]))
    vfreq = np.array([float(rot["base"]) ** (-2.0 * i / V) for i in range(V // 2)], F)
    vang = angles(positions, vfreq)
    v = turn_pairs(v, vang, V)
    if cache is not None:
        k, v = np.concatenate([cache[0], k]), np.concatenate([cache[1], v])
    n = k.shape[0]
    a = window_attention_weights(q, k, m, w[p + "sink"], w[p + "talk"], positions, np.arange(n))
    o = np.einsum("htn,nhv->thv", a, np.repeat(v, H // G, axis=1))
    o = turn_pairs(o, -vang, V)
    return o.reshape(T, H * V) @ w[p + "o"].T, (k, v)


# ----------------------------------------------------------------------------------------------- gated linear recurrent unit
def recurrent_unit(h, w, p, m, state):
    """The right branch.  state: (S [width], conv tail) or None."""
    NB = int(m["blocks"])
    T = h.shape[0]
    S, tail = (None, None) if state is None else state
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u, tail = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], tail)
    u = u + w[p + "conv.b"]
    C = u.shape[1]
    B = C // NB
    ub = u.reshape(T, NB, B)
    r = sigmoid(np.einsum("boi,tbi->tbo", w[p + "ra"], ub) + w[p + "ra.b"]).reshape(T, C)
    i = sigmoid(np.einsum("boi,tbi->tbo", w[p + "ri"], ub) + w[p + "ri.b"]).reshape(T, C)
    a = np.exp(-8.0 * r * softplus(w[p + "lam"]))
    S = np.zeros(C, F) if S is None else S.copy()
    out = np.zeros((T, C), F)
    for t in range(T):
        S = a[t] * S + np.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[p + "o"].T, (S, tail)


def parallel_mixer(h, w, p, m, eps, positions, state):
    state = state or {"left": None, "right": None}
    left, state["left"] = window_attention(h, w, p + "left.", m["left"], positions, state["left"])
    right, state["right"] = recurrent_unit(h, w, p + "right.", m["right"], state["right"])
    return 0.5 * (norm_plain(left, w[p + "left.out"], eps) + norm_plain(right, w[p + "right.out"], eps)), state


# ----------------------------------------------------------------------------------------------- gated delta rule
def delta_step(S, q, k, v, beta, g):
    """One token of one head: S [dim, vdim]; decay of the key rows, the delta write, the read-out after the write."""
    S = g[:, None] * S
    u = beta * (v - S.T @ k)
    S = S + np.outer(k, u)
    return S, S.T @ q


def channel_delta(h, w, p, m, eps, state):
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    state = state or {"S": np.zeros((H, D, V), F), "q": None, "k": None, "v": None}
    proj = {}
    for name in ("q", "k", "v"):
        c, state[name] = causal_conv(h @ w[p + name].T, w[p + name + ".conv"], state[name])
        proj[name] = silu(c)
    q = proj["q"].reshape(T, G, D)
    k = proj["k"].reshape(T, G, D)
    v = proj["v"].reshape(T, H, V)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[p + "b"].T)
    g = np.exp(-np.exp(w[p + "A_log"])[None, :, None] * softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, D))
    S = state["S"].copy()
    o = np.zeros((T, H, V), F)
    for t in range(T):
        for hh in range(H):
            kv = hh // (H // G)
            S[hh], o[t, hh] = delta_step(S[hh], q[t, kv], k[t, kv], v[t, hh], beta[t, hh], g[t, hh])
    state["S"] = S
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, V)
    o = norm_plain(o, w[p + "norm"], eps) * gate
    return o.reshape(T, H * V) @ w[p + "o"].T, state


# ----------------------------------------------------------------------------------------------- experts
def route_top_logits(h, w, p, top):
    """(chosen experts [T, top], weights [T, top]): the largest logits win (lowest index on a tie), softmax over the chosen."""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    pick = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, pick, axis=-1)
    e = np.exp(zc - zc.max(axis=-1, keepdims=True))
    return pick, e / e.sum(axis=-1, keepdims=True)


def experts_ff(h, w, p, mlp):
    pick, wt = route_top_logits(h, w, p, int(mlp["router"]["top"]))
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]), F)
    for t in range(h.shape[0]):
        for e, g in zip(pick[t], wt[t]):
            q = f"{p}e{int(e)}."
            out[t] += g * (gelu_erf(h[t] @ w[q + "up"].T) @ w[q + "down"].T)
    return out


# ----------------------------------------------------------------------------------------------- the model
def layer_runs(config):
    """(layer index, add the embedding output in front) for every layer run, in execution order."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop or int(loop["times"]) <= 1:
        return [(i, False) for i in range(n)]
    a, b, k = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for t in range(k):
        runs += [(i, t > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


class Model:
    def __init__(self, config, weights):
        self.config = config
        self.w = {k: np.asarray(v).astype(F) for k, v in weights.items()}
        self.eps = float(config["norm"]["eps"])
        self.runs = layer_runs(config)

    def new_state(self):
        return {"pos": 0, "runs": [{"canon1": None, "canon2": None, "mix": None} for _ in self.runs]}

    def forward(self, tokens, state=None, want_layers=False):
        """tokens: the next tokens of one sequence; state as left by earlier calls (None: a new sequence).
        Returns (logits [T, vocab], state[, residual stream after every layer run [runs, T, W]])."""
        w, eps = self.w, self.eps
        state = state or self.new_state()
        T = len(tokens)
        positions = np.arange(state["pos"], state["pos"] + T)
        x = w["embed"][np.asarray(tokens, np.int64)] * float((self.config.get("embedding") or {}).get("scale", 1.0))
        x0 = x.copy()
        trace = []
        for st, (li, readd) in zip(state["runs"], self.runs):
            lay, p = self.config["layers"][li], f"l{li}."
            if readd:
                x = x + x0
            h = norm_around_zero(x, w[p + "norm1"], eps)
            c, st["canon1"] = causal_conv(h, w[p + "canon1"], st["canon1"])
            h = h + c
            if lay["type"] == "parallel":
                y, st["mix"] = parallel_mixer(h, w, p + "mix.", lay["mixer"], eps, positions, st["mix"])
            elif lay["type"] == "channel_delta":
                y, st["mix"] = channel_delta(h, w, p + "mix.", lay["mixer"], eps, st["mix"])
            else:
                raise ValueError(lay["type"])
            x = x + norm_around_zero(y, w[p + "norm1b"], eps)
            if lay.get("mlp"):
                g = norm_around_zero(x, w[p + "norm2"], eps)
                c, st["canon2"] = causal_conv(g, w[p + "canon2"], st["canon2"])
                x = x + norm_around_zero(experts_ff(g + c, w, p + "mlp.", lay["mlp"]), w[p + "norm2b"], eps)
            trace.append(x.copy())
        state["pos"] += T
        logits = norm_around_zero(x, w["final.norm"], eps) @ w["embed"].T
        return (logits, state, np.stack(trace)) if want_layers else (logits, state)
