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


ROUND_INPUTS = False          # set by forward(round_inputs=True)


def inp(x):
    """The input of a matrix product: as it is, or (ROUND_INPUTS) rounded to bfloat16 as a bfloat16 plan rounds it.  The products of the
    cached latents with the key / value expansions are float32 in every plan and are not rounded."""
    return np.asarray(bf16_round(x), np.float64) if ROUND_INPUTS else x


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
    h = inp(h)
    q = silu(h @ p["q"].T).reshape(T, H, D)
    k = silu(h @ p["k"].T).reshape(T, H, D)
    v = silu(h @ p["v"].T).reshape(T, H, V)
    o, _ = decayed_memory(q, k, v, c["decay"])
    o = rms_norm(o.reshape(T, H * V), p["norm"], eps) * sigmoid(h @ p["g"].T)
    return inp(o) @ p["o"].T


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
    R, P = c["kv_rank"], c.get("rot_dim", 0)
    T = h.shape[0]
    z = inp(h) @ p["dkv"].T
    lat = rms_norm(z[:, :R], p["dkv.norm"], eps)
    kr = turn(z[:, None, R:R + P], np.arange(T), c["rot"])[:, 0] if P else z[:, R:R]
    return lat, kr


def latent_attention(h, p, c, eps, cache=None, causal_shift=0, drop_keys=()):
    """Queries q = W_uq rms_norm(W_dq h) as [heads, dim + rot_dim] (the last rot_dim entries turn); keys [W_uk c | shared rotated part],
    values W_uv c, from this layer's cache or the one handed in (`cache`: a layer with kv_from); causal softmax of scale * q . k; one
    sigmoid gate per head; W_o.  causal_shift and drop_keys are knobs for the tests' sensitivity checks: query i sees j <= i + shift
    (always itself), and the listed keys are hidden from later queries."""
    T = h.shape[0]
    H, D, P, V, R = c["heads"], c["dim"], c.get("rot_dim", 0), c["vdim"], c["kv_rank"]
    lat, kr = cache if cache is not None else latent_cache(h, p, c, eps)
    h = inp(h)
    cq = rms_norm(h @ p["dq"].T, p["dq.norm"], eps)
    q = (inp(cq) @ p["uq"].T).reshape(T, H, D + P)
    qn, qr = q[..., :D], (turn(q[..., D:], np.arange(T), c["rot"]) if P else q[..., D:])
    kn = (lat @ p["uk"].T).reshape(T, H, D)
    v = (lat @ p["uv"].T).reshape(T, H, V)
    s = (np.einsum("ihd,jhd->hij", qn, kn) + np.einsum("ihd,jd->hij", qr, kr)) * c["scale"]
    seen = np.tril(np.ones((T, T), bool), causal_shift) | np.eye(T, dtype=bool)
    for j in drop_keys:
        seen[j + 1:, j] = False
    s = np.where(seen[None], s, -np.inf)
    w = np.exp(s - s.max(axis=-1, keepdims=True))
    w = w / w.sum(axis=-1, keepdims=True)
    o = np.einsum("hij,jhv->ihv", w, v) * sigmoid(h @ p["g"].T)[:, :, None]
    return inp(o.reshape(T, H * V)) @ p["o"].T


# ---- feed-forward -----------------------------------------------------------------------------------------------------------------
def dense_ff(h, p):
    """W_down relu(W_up h)^2."""
    return inp(np.square(np.maximum(inp(h) @ p["up"].T, 0.0))) @ p["down"].T


def gated_expert(h, gate, up, down):
    h = inp(h)
    return inp(silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h, p, c):
    """Chosen experts [T, top] and their weights: scores = softmax(W_router h); the `top` largest of scores + correction are chosen
    (lowest index wins a tie); weights = the chosen scores (without the correction) / (their sum + 1e-20) * router.scale."""
    z = inp(h) @ p["router"].T
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


def forward(cfg, weights, tokens, taps=None, round_inputs=False, **knobs):
    """Logits [T, vocab] of one sequence; taps (a list) receives the residual stream [T, W] after every layer.  weights: name -> float64
    array.  round_inputs: every matrix product's input is rounded to bfloat16 first (see inp).  knobs go to every latent attention."""
    global ROUND_INPUTS
    ROUND_INPUTS = round_inputs
    try:
        return _forward(cfg, weights, tokens, taps, knobs)
    finally:
        ROUND_INPUTS = False


def _forward(cfg, weights, tokens, taps, knobs):
    eps = cfg["norm"]["eps"]
    x = weights["embed"][np.asarray(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    caches = {}
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m, c = sub(weights, pre + "mix."), layer["mixer"]
        h = rms_norm(x, weights[pre + "norm1"], eps)
        if layer["type"] == "lightning":
            y = lightning(h, m, c, eps)
        elif layer["type"] == "latent_attention":
            if c.get("kv_from") is None:
                caches[i] = latent_cache(h, m, c, eps)
                y = latent_attention(h, m, c, eps, caches[i], **knobs)
            else:
                y = latent_attention(h, m, c, eps, caches[c["kv_from"]], **knobs)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, weights[pre + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp:
            f = sub(weights, pre + "mlp.")
            h = rms_norm(x, weights[pre + "norm2"], eps)
            y = dense_ff(h, f) if mlp["kind"] == "dense" else moe_ff(h, f, mlp)
            x = x + rms_norm(y, weights[pre + "norm2b"], eps)
        if taps is not None:
            taps.append(x.copy())
    z = inp(rms_norm(x, weights["final.norm"], eps)) @ weights["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * np.tanh(z / cap)
    return z


# ---- random models for the tests ----------------------------------------------------------------------------------------------------
def tensor_shapes(cfg):
    """{tensor name: shape} of a configuration, in file order."""
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, ff = "l%d." % i, layer["mixer"], layer.get("mlp")
        out.update({p + "norm1": (W,), p + "norm1b": (W,)})
        od = m["heads"] * m["vdim"]
        if layer["type"] == "lightning":
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (m["heads"] * m["dim"], W), p + "mix.v": (od, W), p + "mix.g": (od, W),
                        p + "mix.o": (W, od), p + "mix.norm": (od,)})
        else:
            P = m.get("rot_dim", 0)
            out.update({p + "mix.dq": (m["q_rank"], W), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (m["heads"] * (m["dim"] + P), m["q_rank"])})
            if m.get("kv_from") is None:
                out.update({p + "mix.dkv": (m["kv_rank"] + P, W), p + "mix.dkv.norm": (m["kv_rank"],)})
            out.update({p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (od, m["kv_rank"]), p + "mix.g": (m["heads"], W), p + "mix.o": (W, od)})
        if ff:
            out.update({p + "norm2": (W,), p + "norm2b": (W,)})
            if ff["kind"] == "dense":
                out.update({p + "mlp.up": (ff["ff"], W), p + "mlp.down": (W, ff["ff"])})
            else:
                f = ff["expert"]["ff"]
                for e in range(ff["router"]["experts"]):
                    out.update({p + "mlp.e%d.gate" % e: (f, W), p + "mlp.e%d.up" % e: (f, W), p + "mlp.e%d.down" % e: (W, f)})
                out.update({p + "mlp.router": (ff["router"]["experts"], W), p + "mlp.correction": (ff["router"]["experts"],)})
                if ff.get("shared"):
                    f = ff["shared"]["ff"]
                    out.update({p + "mlp.shared.gate": (f, W), p + "mlp.shared.up": (f, W), p + "mlp.shared.down": (W, f)})
    out["final.norm"] = (W,)
    return out


def random_weights(cfg, seed):
    """bfloat16-representable float32 weights: matrices ~ N(0, 1 / fan_in), gate and router projections larger (so that gates move and
    the experts' scores spread), norm weights around one, corrections of the order of the scores' differences."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shp in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        if len(shp) == 1 and leaf != "mlp.correction":
            a = 1.0 + 0.2 * rng.standard_normal(shp)
        elif leaf == "embed":
            a = rng.standard_normal(shp) / (cfg.get("embedding") or {}).get("scale", 1.0)
        elif leaf == "mlp.correction":
            a = 0.3 * rng.standard_normal(shp) / shp[0]
        elif leaf in ("mix.g", "mlp.router"):
            a = 3.0 * rng.standard_normal(shp) / np.sqrt(shp[-1])
        else:
            a = rng.standard_normal(shp) / np.sqrt(shp[-1])
        out[name] = bf16_round(a)
    return out


def to_f64(w):
    return {k: np.asarray(v, np.float64) for k, v in w.items()}
