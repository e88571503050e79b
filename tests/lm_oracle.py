"""Plain, slow float64 restatement of the layered language models (Tokosun design) that zig_gpt2_amd/lm.py serves.

One function per mechanism, numpy only, written from the design's equations; it shares no code with the product path
(zig_gpt2_amd/ is not imported).  Weights are a dict name -> numpy array with the checkpoint's tensor names, the
configuration is the dict of config.json.

Notation: x residual stream [T, W]; h a sublayer's input; positions count from 0 per sequence; rms(v) = sqrt(mean(v^2) + eps).
"""
import math

import numpy as np

F = np.float64


def rms_unit(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def norm_around_zero(v, w, eps):
    """The layer norms and the final norm: the stored weight is an offset from one."""
    return rms_unit(v, eps) * (1.0 + w)


def norm_plain(v, w, eps):
    return rms_unit(v, eps) * w


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def token_shift(h, mu, prev):
    """h [T, W] -> mix of every row with its predecessor (prev, or zeros, in front of row 0).  Returns (mixed, last row of h)."""
    before = np.concatenate([(np.zeros_like(h[:1]) if prev is None else prev[None]), h[:-1]], axis=0)
    return h + (before - h) * mu, h[-1].copy()


# ----------------------------------------------------------------------------------------------- rotary positions
def rotary_tables(rot, positions):
    """cos / sin [T, dims/2] with the YaRN frequency blend and amplitude, angles as 32-bit products like the product path."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)], F)
    amp = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def corr(t):
            return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

        lo = max(math.floor(corr(float(sc["fast"]))), 0)
        hi = min(math.ceil(corr(float(sc["slow"]))), dims - 1)
        ramp = np.clip((np.arange(half, dtype=F) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    ang = (np.asarray(positions, np.float32)[:, None] * f.astype(np.float32)[None, :]).astype(F)
    return np.cos(ang) * amp, np.sin(ang) * amp


def rotate_pairs(v, cos, sin, dims):
    """v [T, ..., n]: the first `dims` entries are rotated as interleaved pairs (2i, 2i+1), the rest pass."""
    out = v.copy()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    shape = (cos.shape[0],) + (1,) * (v.ndim - 2) + (cos.shape[1],)
    c, s = cos.reshape(shape), sin.reshape(shape)
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ----------------------------------------------------------------------------------------------- mixers
def hgrn2(h, w, p, m, eps, state):
    """Gated linear recurrence; state [heads, dim, vdim] or None.  Returns (out [T, W], new state)."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ w[p + "q"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, V)
    low = w[p + "lower"].astype(F)
    f = (low + (1.0 - low) * sigmoid(h @ w[p + "f"].T + w[p + "f.b"])).reshape(T, H, D)
    S = np.zeros((H, D, V), F) if state is None else state.copy()
    o = np.zeros((T, H, V), F)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = norm_plain(o, w[p + "norm"], eps).reshape(T, H * V)
    return o @ w[p + "o"].T, S


def latent_attention(h, w, p, m, eps, positions, cache):
    """Attention through a low-rank latent; cache = (latents [n, kv_rank], rotated keys [n, rot_dim]) of the tokens before, or
    None.  Keys and values are rebuilt from the latents of all tokens seen so far.  Returns (out, new cache)."""
    H, D, R, V, KR = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    cq = norm_plain(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(T, H, D + R)
    kv = h @ w[p + "dkv"].T
    c = norm_plain(kv[:, :KR], w[p + "dkv.norm"], eps)
    cos, sin = rotary_tables(m["rot"], positions)
    dims = int(m["rot"]["dims"])
    kr = rotate_pairs(kv[:, KR:], cos, sin, dims)
    qr = rotate_pairs(q[:, :, D:], cos, sin, dims)
    if cache is not None:
        c_all, kr_all = np.concatenate([cache[0], c]), np.concatenate([cache[1], kr])
    else:
        c_all, kr_all = c, kr
    n = c_all.shape[0]
    k = (c_all @ w[p + "uk"].T).reshape(n, H, D)
    val = (c_all @ w[p + "uv"].T).reshape(n, H, V)
    s = (np.einsum("thd,nhd->htn", q[:, :, :D], k) + np.einsum("thr,nr->htn", qr, kr_all)) * float(m["scale"])
    key_pos = np.arange(n)[None, :]
    q_pos = (n - T + np.arange(T))[:, None]
    s = np.where(key_pos <= q_pos, s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    a = e / e.sum(axis=-1, keepdims=True)
    o = np.einsum("htn,nhv->thv", a, val).reshape(T, H * V)
    return o @ w[p + "o"].T, (c_all, kr_all)


def attention_weights(h, w, p, m, eps, positions):
    """The softmax weights [heads, queries, keys] of latent_attention for a whole sequence (tests look at where they peak)."""
    H, D, R, KR = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    T = h.shape[0]
    q = (norm_plain(h @ w[p + "dq"].T, w[p + "dq.norm"], eps) @ w[p + "uq"].T).reshape(T, H, D + R)
    kv = h @ w[p + "dkv"].T
    c = norm_plain(kv[:, :KR], w[p + "dkv.norm"], eps)
    cos, sin = rotary_tables(m["rot"], positions)
    dims = int(m["rot"]["dims"])
    kr, qr = rotate_pairs(kv[:, KR:], cos, sin, dims), rotate_pairs(q[:, :, D:], cos, sin, dims)
    k = (c @ w[p + "uk"].T).reshape(T, H, D)
    s = (np.einsum("thd,nhd->htn", q[:, :, :D], k) + np.einsum("thr,nr->htn", qr, kr)) * float(m["scale"])
    s = np.where(np.arange(T)[None, :] <= np.arange(T)[:, None], s, -np.inf)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


# ----------------------------------------------------------------------------------------------- feed-forward
def dense_ff(h, w, p):
    u = np.maximum(h @ w[p + "up"].T, 0.0)
    return (u * u) @ w[p + "down"].T


def route(h, w, p, top):
    """(chosen experts [T, top], their weights [T, top]): softmax scores; the choice adds the correction, the weight does not."""
    z = h @ w[p + "router"].T
    z = z - z.max(axis=-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(axis=-1, keepdims=True)
    pick = np.argsort(-(s + w[p + "correction"]), axis=-1, kind="stable")[:, :top]
    return pick, np.take_along_axis(s, pick, axis=-1)


def moe_ff(h, w, p, mlp):
    top = int(mlp["router"]["top"])
    pick, wt = route(h, w, p, top)
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]), F)
    for t in range(h.shape[0]):
        for e, g in zip(pick[t], wt[t]):
            q = f"{p}e{int(e)}."
            out[t] += g * ((silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


# ----------------------------------------------------------------------------------------------- the model
def layer_runs(config):
    """Indices of config['layers'] in execution order: the looped span repeated in a row, every pass with its own state."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, k = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * k + list(range(b, n))


class Model:
    def __init__(self, config, weights):
        self.config = config
        self.w = {k: np.asarray(v).astype(F) for k, v in weights.items()}
        self.eps = float(config["norm"]["eps"])
        self.runs = layer_runs(config)

    def new_state(self):
        return {"pos": 0, "runs": [{"shift": None, "mix": None} for _ in self.runs]}

    def forward(self, tokens, state=None, want_layers=False):
        """tokens: the next tokens of one sequence; state as left by earlier calls (None: a new sequence).
        Returns (logits [T, vocab], state[, residual stream after every layer run [runs, T, W]])."""
        w, eps = self.w, self.eps
        state = state or self.new_state()
        T = len(tokens)
        positions = np.arange(state["pos"], state["pos"] + T)
        x = w["embed"][np.asarray(tokens, np.int64)]
        trace = []
        for st, li in zip(state["runs"], self.runs):
            lay, p = self.config["layers"][li], f"l{li}."
            h = norm_around_zero(x, w[p + "norm1"], eps)
            h, st["shift"] = token_shift(h, w[p + "shift"], st["shift"])
            if lay["type"] == "hgrn2":
                y, st["mix"] = hgrn2(h, w, p + "mix.", lay["mixer"], eps, st["mix"])
            elif lay["type"] == "latent_attention":
                y, st["mix"] = latent_attention(h, w, p + "mix.", lay["mixer"], eps, positions, st["mix"])
            else:
                raise ValueError(lay["type"])
            x = x + norm_around_zero(y, w[p + "norm1b"], eps)
            if lay.get("mlp"):
                g = norm_around_zero(x, w[p + "norm2"], eps)
                y = dense_ff(g, w, p + "mlp.") if lay["mlp"]["kind"] == "dense" else moe_ff(g, w, p + "mlp.", lay["mlp"])
                x = x + norm_around_zero(y, w[p + "norm2b"], eps)
            trace.append(x.copy())
        state["pos"] += T
        logits = norm_around_zero(x, w["final.norm"], eps) @ w["head"].T
        return (logits, state, np.stack(trace)) if want_layers else (logits, state)
