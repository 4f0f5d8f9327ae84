"""Plain, slow restatement of the Kosusun design in float64 numpy: one function per mechanism, whole sequences at once, no cache
carried between calls.  It shares no code with the product path (csrc/gl3_hybrid*.h, csrc/gl3_hy*_kernels.h) and is the yardstick of
tests/test_kosusun*.py.

Notation: T tokens at positions 0 .. T - 1, W model width, h the [T, W] normed input of a layer, weights as [out, in] matrices applied
as h @ M.T.  A mixer's weights are a dict keyed by the tensor's name behind the mixer's prefix ("q", "k.b", "sink", "norm", ...).

The design: x_0 = embed[token] * embedding.scale; every layer is x <- x + residual_mult * (mixer(h) + ff(h)) with ONE norm
h = x / rms(x) * norm1; logits = head (x / rms(x) * final.norm) * logit_scale.  Layer type "parallel" = left_scale * attention +
right_scale * retention, layer type "mlstm" = a matrix memory with exponential gates.
"""
from __future__ import annotations

import numpy as np


def bf16_round(a):
    """float32 values that bfloat16 holds exactly (round to nearest even)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def frequencies(rot):
    n = rot["dims"]
    return rot["base"] ** (-2.0 * np.arange(n // 2) / n) / (rot.get("scaling") or {}).get("factor", 1.0)


def turn(x, pos, rot, interleaved):
    """Rotary turn of the first rot.dims entries of the last axis by pos * frequency; the rest pass.  Pairs are (2 i, 2 i + 1) when
    interleaved, else (i, i + dims / 2).  x: [T, heads, D], pos: [T]."""
    if not rot:
        return x
    n, f = rot["dims"], frequencies(rot)
    a = pos[:, None, None] * f
    c, s = np.cos(a), np.sin(a)
    out = x.copy()
    if interleaved:
        u, v = x[..., 0:n:2], x[..., 1:n:2]
        out[..., 0:n:2], out[..., 1:n:2] = u * c - v * s, v * c + u * s
    else:
        u, v = x[..., :n // 2], x[..., n // 2:n]
        out[..., :n // 2], out[..., n // 2:n] = u * c - v * s, v * c + u * s
    return out


def window_lo(i, size):
    """First position the window of query i holds."""
    return max(0, i - size + 1)


def blocks_seen(i, size, pool, shift=0):
    """Number of pooled blocks query i sees: block b (positions b pool .. b pool + pool - 1) counts when its last position is at most
    i - size (+ shift, a knob for the tests' sensitivity checks)."""
    if not pool:
        return 0
    return max(0, (i - size + shift + 1) // pool)


def pooled_window_attention(h, p, c, eps, size_delta=0, pool_shift=0):
    """Grouped-query attention: biased q / k / v, RMS norm with weights over the whole q and the whole k projection, interleaved rotary
    pairs, a window of mask.size positions, one averaged key / value per finished block of mask.pool positions behind the window (see
    blocks_seen), a learned sink logit per head in the denominator."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    mask = c.get("mask") or {}
    size, pool = mask.get("size", 1 << 30) + size_delta, mask.get("pool", 0)
    pos = np.arange(T, dtype=np.float64)
    q = unit_rms(h @ p["q"].T + p["q.b"], eps) * p["q.norm"]
    k = unit_rms(h @ p["k"].T + p["k.b"], eps) * p["k.norm"]
    v = (h @ p["v"].T + p["v.b"]).reshape(T, G, V)
    q = turn(q.reshape(T, H, D), pos, c.get("rot"), True)
    k = turn(k.reshape(T, G, D), pos, c.get("rot"), True)
    nblocks = T // pool if pool else 0                       # complete blocks: their pooled key / value is the mean of the block's rows
    pk = k[:nblocks * pool].reshape(nblocks, pool, G, D).mean(axis=1) if nblocks else np.zeros((0, G, D))
    pv = v[:nblocks * pool].reshape(nblocks, pool, G, V).mean(axis=1) if nblocks else np.zeros((0, G, V))
    out = np.zeros((T, H, V))
    per = H // G
    for i in range(T):
        lo, nb = window_lo(i, size), blocks_seen(i, size, pool, pool_shift)
        for g in range(G):
            keys = np.concatenate([pk[:nb, g], k[lo:i + 1, g]])
            vals = np.concatenate([pv[:nb, g], v[lo:i + 1, g]])
            hs = slice(g * per, (g + 1) * per)
            s = q[i, hs] @ keys.T * c["scale"]                # [heads of the group, keys]
            z = p["sink"][hs]
            m = np.maximum(s.max(axis=1), z)
            e = np.exp(s - m[:, None])
            out[i, hs] = (e @ vals) / (e.sum(axis=1) + np.exp(z - m))[:, None]
    return out.reshape(T, H * V) @ p["o"].T


def retention(h, p, c, eps):
    """S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head; q / k turned in half-split pairs, k times dim^(-1/2) afterwards; every
    head's o divided by its root mean square, times silu(W_g h)."""
    T = h.shape[0]
    H, D, V = c["heads"], c["dim"], c["vdim"]
    pos = np.arange(T, dtype=np.float64)
    q = turn((h @ p["q"].T).reshape(T, H, D), pos, c.get("rot"), False)
    k = turn((h @ p["k"].T).reshape(T, H, D), pos, c.get("rot"), False) * D ** -0.5
    v = (h @ p["v"].T).reshape(T, H, V)
    decay = np.asarray(c["decay"], np.float64)
    S = np.zeros((H, D, V))
    o = np.zeros((T, H, V))
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    g = h @ p["g"].T
    return (unit_rms(o, eps).reshape(T, H * V) * g * sigmoid(g)) @ p["o"].T


def mlstm(h, p, c, eps):
    """Matrix memory with exponential gating: log gates i = cap tanh(z_i / cap), f = logsigmoid(cap tanh(z_f / cap)); running maximum
    m_t = max(f + m_(t-1), i) from m = 0; S and n decay by e^(f + m_(t-1) - m_t) and take e^(i - m_t) k v^T / k;
    o = S^T q / (max(|n . q|, e^(-m_t)) + 1e-6), q scaled by dim^(-1/2); unit-RMS heads times a weight, times sigmoid(W_g h)."""
    T = h.shape[0]
    H, D, V, cap = c["heads"], c["dim"], c["vdim"], c["gate_cap"]
    q = (h @ p["q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ p["k"].T).reshape(T, H, D)
    v = (h @ p["v"].T).reshape(T, H, V)
    ig = cap * np.tanh((h @ p["i"].T + p["i.b"]) / cap)
    fg = -np.logaddexp(0.0, -cap * np.tanh((h @ p["f"].T + p["f.b"]) / cap))
    S, n, m = np.zeros((H, D, V)), np.zeros((H, D)), np.zeros(H)
    o = np.zeros((T, H, V))
    for t in range(T):
        m_new = np.maximum(fg[t] + m, ig[t])
        a, b = np.exp(fg[t] + m - m_new), np.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        m = m_new
        den = np.maximum(np.abs(np.sum(n * q[t], axis=-1)), np.exp(-m)) + 1e-6
        o[t] = np.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
    return (unit_rms(o, eps).reshape(T, H * V) * p["norm"] * sigmoid(h @ p["g"].T)) @ p["o"].T


def dense_ff(h, p):
    return (gelu_tanh(h @ p["gate"].T) * (h @ p["up"].T)) @ p["down"].T


def sub(w, prefix):
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def forward(cfg, w, tokens, taps=None, **attn_knobs):
    """Logits [T, vocab] of a whole sequence; taps (a list) receives the residual after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i, layer in enumerate(cfg["layers"]):
        pre, mx = "l%d." % i, layer["mixer"]
        h = unit_rms(x, eps) * w[pre + "norm1"]
        if layer["type"] == "parallel":
            y = mx.get("left_scale", 1.0) * pooled_window_attention(h, sub(w, pre + "mix.left."), mx["left"], eps, **attn_knobs)
            y = y + mx.get("right_scale", 1.0) * retention(h, sub(w, pre + "mix.right."), mx["right"], eps)
        else:
            y = mlstm(h, sub(w, pre + "mix."), mx, eps)
        if layer.get("mlp"):
            y = y + dense_ff(h, sub(w, pre + "mlp."))
        x = x + cfg.get("residual_mult", 1.0) * y
        if taps is not None:
            taps.append(x.copy())
    head = w["head"] if "head" in w else w["embed"]
    return (unit_rms(x, eps) * w["final.norm"]) @ head.T * cfg.get("logit_scale", 1.0)


# ---- shapes and random weights ---------------------------------------------------------------------------------------------------------
def tensor_shapes(cfg, tied=False):
    """{tensor name: shape} in file order."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W)}
    for i, layer in enumerate(cfg["layers"]):
        p, mx, ff = "l%d." % i, layer["mixer"], layer.get("mlp")
        out[p + "norm1"] = (W,)
        if layer["type"] == "parallel":
            a, r = mx["left"], mx["right"]
            q = p + "mix.left."
            out.update({q + "q": (a["heads"] * a["dim"], W), q + "q.b": (a["heads"] * a["dim"],), q + "k": (a["kv_heads"] * a["dim"], W),
                        q + "k.b": (a["kv_heads"] * a["dim"],), q + "v": (a["kv_heads"] * a["vdim"], W), q + "v.b": (a["kv_heads"] * a["vdim"],),
                        q + "q.norm": (a["heads"] * a["dim"],), q + "k.norm": (a["kv_heads"] * a["dim"],), q + "sink": (a["heads"],),
                        q + "o": (W, a["heads"] * a["vdim"])})
            q = p + "mix.right."
            out.update({q + "q": (r["heads"] * r["dim"], W), q + "k": (r["heads"] * r["dim"], W), q + "v": (r["heads"] * r["vdim"], W),
                        q + "g": (r["heads"] * r["vdim"], W), q + "o": (W, r["heads"] * r["vdim"])})
        else:
            q = p + "mix."
            out.update({q + "q": (mx["heads"] * mx["dim"], W), q + "k": (mx["heads"] * mx["dim"], W), q + "v": (mx["heads"] * mx["vdim"], W),
                        q + "g": (mx["heads"] * mx["vdim"], W), q + "o": (W, mx["heads"] * mx["vdim"]), q + "norm": (mx["heads"] * mx["vdim"],),
                        q + "i": (mx["heads"], W), q + "i.b": (mx["heads"],), q + "f": (mx["heads"], W), q + "f.b": (mx["heads"],)})
        if ff:
            out.update({p + "mlp.gate": (ff["ff"], W), p + "mlp.up": (ff["ff"], W), p + "mlp.down": (W, ff["ff"])})
    out["final.norm"] = (W,)
    if not tied:
        out["head"] = (V, W)
    return out


def leaf_of(name):
    """Tensor name without the layer and mixer prefixes: "l3.mix.left.q.b" -> "q.b"."""
    if name in ("embed", "head", "final.norm"):
        return name
    rest = name.split(".", 1)[1]
    for pre in ("mix.left.", "mix.right.", "mix.", "mlp."):
        if rest.startswith(pre):
            return rest[len(pre):]
    return rest


def random_weights(cfg, seed, tied=False):
    """bfloat16-representable float32 weights: matrices ~ N(0, 1 / fan_in), gate projections larger (so that gates move), norm weights
    around one, biases and sinks of order one, forget-gate biases positive (a memory that keeps most of its past)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shp in tensor_shapes(cfg, tied).items():
        leaf = leaf_of(name)
        if leaf in ("norm1", "final.norm", "q.norm", "k.norm", "norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shp)
        elif leaf == "embed":
            a = rng.standard_normal(shp) / cfg.get("embedding", {}).get("scale", 1.0)
        elif leaf in ("q.b", "k.b", "v.b"):
            a = 0.3 * rng.standard_normal(shp)
        elif leaf == "sink":
            a = rng.standard_normal(shp)
        elif leaf in ("i", "f"):
            a = 3.0 * rng.standard_normal(shp) / np.sqrt(shp[-1])
        elif leaf == "i.b":
            a = rng.standard_normal(shp)
        elif leaf == "f.b":
            a = 2.0 + rng.standard_normal(shp)
        else:
            a = rng.standard_normal(shp) / np.sqrt(shp[-1])
        out[name] = bf16_round(a)
    return out


def to_f64(w):
    return {k: np.asarray(v, np.float64) for k, v in w.items()}
