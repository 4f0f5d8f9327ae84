"""Plain, slow restatement of the Kugadra design in float64 numpy: one function per mechanism, whole sequences at once, no cache
carried between calls.  It shares no code with the product path (csrc/gl3_hybrid*.h, csrc/gl3_hy*_kernels.h) and is the yardstick of
tests/test_kugadra*.py.

Notation: T tokens at positions 0 .. T - 1, W model width, h the [T, W] normed input of a sublayer, weights as [out, in] matrices
applied as h @ M.T.  A mixer's weights are a dict keyed by the tensor's name behind "<layer>.mix." ("q", "dq.norm", ...), a
feed-forward's by the name behind "<layer>.mlp." ("up", "e3.gate", "shared.down", "router", "correction").

The design: x_0 = embed[token] * embedding.scale; every layer is
    x <- x + rms_norm(mixer(rms_norm(x, norm1)), norm1b);   x <- x + rms_norm(ff(rms_norm(x, norm2)), norm2b)
(the second line only where the layer has a feed-forward); logits = cap * tanh(embed (rms_norm(x, final.norm)) / cap).
Mixers: "lightning" (a matrix memory with a fixed decay per head behind silu-activated q / k / v, one norm over all heads, sigmoid
gate) and "latent_attention" (queries through a normed latent, keys and values expanded from a cached normed latent, one rotated key
part shared by all heads with YaRN-scaled frequencies, softmax, one sigmoid gate per head; a layer may read another layer's cache).
"""
from __future__ import annotations

import math

import numpy as np


def bf16_round(a):
    """float32 values that bfloat16 holds exactly (round to nearest even)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w = None: no weight)."""
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


# ---- lightning ------------------------------------------------------------------------------------------------------------------
def decayed_memory(q, k, v, decay, state=None):
    """Per head S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t from S = 0 (or `state`).  q, k: [T, H, D], v: [T, H, V], decay: [H].
    Returns o [T, H, V] and the last state [H, D, V]."""
    T, H, D = q.shape
    V = v.shape[2]
    S = np.zeros((H, D, V)) if state is None else state.copy()
    o = np.zeros((T, H, V))
    g = np.asarray(decay, np.float64)[:, None, None]
    for t in range(T):
        S = g * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    return o, S


def lightning(h, p, c, eps):
    """q, k = silu(W h) as [heads, dim], v = silu(W_v h) as [heads, vdim]; the decayed memory per head; the heads side by side go
    through ONE rms norm with the weight `norm`, times sigmoid(W_g h), through W_o."""
    T = h.shape[0]
    H, D, V = c["heads"], c["dim"], c["vdim"]
    q = silu(h @ p["q"].T).reshape(T, H, D)
    k = silu(h @ p["k"].T).reshape(T, H, D)
    v = silu(h @ p["v"].T).reshape(T, H, V)
    o, _ = decayed_memory(q, k, v, c["decay"])
    o = rms_norm(o.reshape(T, H * V), p["norm"], eps) * sigmoid(h @ p["g"].T)
    return o @ p["o"].T


# ---- rotary positions with YaRN-scaled frequencies ------------------------------------------------------------------------------
def yarn_frequencies(rot):
    """Frequencies [dims / 2] and the multiplier of cos and sin.  Without rot.scaling: base^(-2 i / dims) and 1."""
    n, base = rot["dims"], float(rot["base"])
    i = np.arange(n // 2, dtype=np.float64)
    f = base ** (-2.0 * i / n)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def where(turns):          # the (fractional) pair index whose wavelength makes `turns` turns over the original length
        return n * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(float(sc["fast"]))), 0)
    hi = min(math.ceil(where(float(sc["slow"]))), n - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn(x, pos, rot):
    """Rotary turn of the first rot.dims entries of the last axis, entry i paired with entry i + dims / 2; the rest pass.
    x: [T, heads, D], pos: [T]."""
    n = rot["dims"]
    f, mul = yarn_frequencies(rot)
    a = np.asarray(pos, np.float64)[:, None, None] * f
    c, s = np.cos(a) * mul, np.sin(a) * mul
    out = x.copy()
    u, v = x[..., :n // 2], x[..., n // 2:n]
    out[..., :n // 2], out[..., n // 2:n] = u * c - v * s, v * c + u * s
    return out


# ---- latent attention -----------------------------------------------------------------------------------------------------------
def latent_cache(h, p, c, eps):
    """What a latent-attention layer caches per token: the normed latent [T, kv_rank] and the rotated key part [T, rot_dim]."""
    R, P = c["kv_rank"], c["rot_dim"]
    T = h.shape[0]
    z = h @ p["dkv"].T
    lat = rms_norm(z[:, :R], p["dkv.norm"], eps)
    kr = turn(z[:, None, R:R + P], np.arange(T), c["rot"])[:, 0]
    return lat, kr


def latent_attention(h, p, c, eps, cache=None):
    """Queries q = W_uq rms_norm(W_dq h) as [heads, dim + rot_dim] (the last rot_dim entries turn); keys [W_uk c | shared rotated part],
    values W_uv c, from this layer's cache or the one handed in (`cache`: a layer with kv_from); causal softmax of scale * q . k; one
    sigmoid gate per head; W_o."""
    T = h.shape[0]
    H, D, P, V, R = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    lat, kr = cache if cache is not None else latent_cache(h, p, c, eps)
    cq = rms_norm(h @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).reshape(T, H, D + P)
    qn, qr = q[..., :D], turn(q[..., D:], np.arange(T), c["rot"])
    kn = (lat @ p["uk"].T).reshape(T, H, D)
    v = (lat @ p["uv"].T).reshape(T, H, V)
    s = (np.einsum("ihd,jhd->hij", qn, kn) + np.einsum("ihd,jd->hij", qr, kr)) * c["scale"]
    s = np.where(np.tril(np.ones((T, T), bool))[None], s, -np.inf)
    w = np.exp(s - s.max(axis=-1, keepdims=True))
    w = w / w.sum(axis=-1, keepdims=True)
    o = np.einsum("hij,jhv->ihv", w, v) * sigmoid(h @ p["g"].T)[:, :, None]
    return o.reshape(T, H * V) @ p["o"].T


# ---- feed-forward -----------------------------------------------------------------------------------------------------------------
def dense_ff(h, p):
    """W_down relu(W_up h)^2."""
    return np.square(np.maximum(h @ p["up"].T, 0.0)) @ p["down"].T


def gated_expert(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h, p, c):
    """Chosen experts [T, top] and their weights: scores = softmax(W_router h); the `top` largest of scores + correction are chosen
    (lowest index wins a tie); weights = the chosen scores (without the correction) / (their sum + 1e-20) * router.scale."""
    z = h @ p["router"].T
    s = np.exp(z - z.max(axis=-1, keepdims=True))
    s = s / s.sum(axis=-1, keepdims=True)
    top = c["router"]["top"]
    choice = np.argsort(-(s + p["correction"]), axis=-1, kind="stable")[:, :top]
    w = np.take_along_axis(s, choice, axis=-1)
    w = w / (w.sum(axis=-1, keepdims=True) + 1e-20) * c["router"]["scale"]
    return choice, w


def moe_ff(h, p, c):
    choice, w = route(h, p, c)
    out = np.zeros((h.shape[0], p["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, we in zip(choice[t], w[t]):
            out[t] += we * gated_expert(h[t:t + 1], p[f"e{e}.gate"], p[f"e{e}.up"], p[f"e{e}.down"])[0]
    if c.get("shared"):
        out = out + gated_expert(h, p["shared.gate"], p["shared.up"], p["shared.down"])
    return out


# ---- the model --------------------------------------------------------------------------------------------------------------------
def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, round_router_input=False):
    """Logits [T, vocab] and the residual stream after every layer [layers, T, W] of one sequence.  weights: name -> float64 array."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    x = weights["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    taps, caches = [], {}
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m, c = sub(weights, pre + "mix."), layer["mixer"]
        h = rms_norm(x, weights[pre + "norm1"], eps)
        if layer["type"] == "lightning":
            y = lightning(h, m, c, eps)
        elif layer["type"] == "latent_attention":
            if c.get("kv_from") is None:
                caches[i] = latent_cache(h, m, c, eps)
                y = latent_attention(h, m, c, eps, caches[i])
            else:
                y = latent_attention(h, m, c, eps, caches[c["kv_from"]])
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, weights[pre + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp:
            f = sub(weights, pre + "mlp.")
            h = rms_norm(x, weights[pre + "norm2"], eps)
            y = dense_ff(h, f) if mlp["kind"] == "dense" else moe_ff(h, f, mlp)
            x = x + rms_norm(y, weights[pre + "norm2b"], eps)
        taps.append(x.copy())
    z = rms_norm(x, weights["final.norm"], eps) @ weights["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * np.tanh(z / cap)
    return z, np.stack(taps)
