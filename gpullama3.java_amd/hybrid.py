"""Host side of the layer-list family (GL3_ARCH_LAYERLIST: the Noditar, Vonulix, Kosusun and Kugadra designs) over the C-ABI: model folders (config.json + model.safetensors), the step
function with sequence slots, greedy / sampled generation.  The compute path is csrc/gl3_hybrid.hip; nothing here computes.

    plan = HybridPlan.from_dir("model-folder", dtype="bfloat16", ctx=4096, max_batch=512, n_seqs=2)
    seq = plan.acquire()
    logits = plan.step(seq, tokens, start_pos=0, want=[len(tokens) - 1])      # [1, vocab]
    plan.release(seq)
    ids = plan.generate(prompt, 32)                                           # the loop of tools/gl3_run.cpp for model folders
"""
from __future__ import annotations

import ctypes as C
import json
import os
import struct

import numpy as np

from . import hip


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (round to nearest even)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def save_model_dir(path: str, config: dict, tensors: dict, dtype: str = "BF16"):
    """Write config.json and model.safetensors (8-byte little-endian header length, JSON header, data).  tensors: {name: float array}
    in file order; dtype "BF16" stores bfloat16 (values are rounded), "F32" float32.  uint16 arrays are taken as bfloat16 bits."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f, indent=1)
    header, blobs, off = {}, [], 0
    for name, a in tensors.items():
        if a.dtype == np.uint16:
            raw, dt = np.ascontiguousarray(a).tobytes(), "BF16"
        elif dtype == "BF16":
            raw, dt = to_bf16_bits(a).tobytes(), "BF16"
        else:
            raw, dt = np.ascontiguousarray(a, np.float32).tobytes(), "F32"
        header[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    h = json.dumps(header).encode()
    h += b" " * (-len(h) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)


class HybridPlan:
    def __init__(self, ctx_ptr):
        self._ctx = ctx_ptr
        d = hip.ModelDesc()
        hip.check(hip.lib().gl3_get_model_desc(self._ctx, C.byref(d)), self._ctx)
        self.vocab, self.dim, self.n_layers, self.ctx, self.max_batch, self.n_seqs, self.streams = (
            d.vocab, d.dim, d.n_layers, d.ctx, d.max_batch, d.n_seqs, d.streams)
        self.f32 = bool(d.flags & hip.FLAG_F32_COMPUTE)

    @classmethod
    def from_dir(cls, path: str, dtype: str = "bfloat16", ctx: int = 4096, max_batch: int = 512, n_seqs: int = 1, device: int = 0,
                 layer_taps: bool = False) -> "HybridPlan":
        assert dtype in ("bfloat16", "float32")
        L = hip.lib()
        if not L.gl3_is_model_dir(path.encode()):
            raise hip.Gl3Error(hip.E_ARG, "%s is not a model folder (no config.json)" % path)
        opts = hip.ModelDesc()
        opts.struct_size = C.sizeof(hip.ModelDesc)
        opts.ctx, opts.max_batch, opts.n_seqs, opts.device = ctx, max_batch, n_seqs, device
        opts.flags = (hip.FLAG_F32_COMPUTE if dtype == "float32" else 0) | (hip.FLAG_LAYER_TAPS if layer_taps else 0)
        ptr = C.c_void_p()
        hip.check(L.gl3_load_model_dir(path.encode(), C.byref(opts), C.byref(ptr)))
        return cls(ptr)

    # ---- sequence slots and the step ----------------------------------------------------------------------------------------------
    def acquire(self) -> int:
        s = C.c_int32()
        hip.check(hip.lib().gl3_seq_acquire(self._ctx, C.byref(s)), self._ctx)
        return s.value

    def release(self, seq: int):
        hip.check(hip.lib().gl3_seq_release(self._ctx, seq), self._ctx)

    def step(self, seq: int, tokens, start_pos: int, want=()) -> np.ndarray:
        """Run the next tokens of slot `seq`; returns the logits of the wanted rows, [len(want), vocab]."""
        t = np.ascontiguousarray(tokens, np.int32)
        w = np.ascontiguousarray(want, np.int32)
        out = np.empty((w.size, self.vocab), np.float32)
        hip.check(hip.lib().gl3_forward_step(self._ctx, seq, _p(t), t.size, start_pos, _p(w) if w.size else None, w.size,
                                             _p(out) if w.size else None), self._ctx)
        return out

    def layer_rows(self, layer: int, n: int) -> np.ndarray:
        out = np.empty((n, self.dim), np.float32)
        hip.check(hip.lib().gl3_get_layer_rows(self._ctx, layer, _p(out), n), self._ctx)
        return out

    # ---- the single-sequence interface the other families have --------------------------------------------------------------------
    def prefill(self, tokens, start_pos: int = 0):
        t = np.ascontiguousarray(tokens, np.int32)
        hip.check(hip.lib().gl3_forward_prefill(self._ctx, _p(t), t.size, start_pos), self._ctx)

    def forward_decode(self, token: int, position: int) -> np.ndarray:
        out = np.empty(self.vocab, np.float32)
        hip.check(hip.lib().gl3_forward_decode(self._ctx, token, position, _p(out), None), self._ctx)
        return out

    def forward_decode_argmax(self, token: int, position: int) -> int:
        a = C.c_int32()
        hip.check(hip.lib().gl3_forward_decode(self._ctx, token, position, None, C.byref(a)), self._ctx)
        return a.value

    def forward_decode_batch(self, tokens, seq_ids, positions):
        """One token for each of several slots (the slots run one after the other) -> (logits [n, vocab], greedy ids [n])."""
        t, s, p = (np.ascontiguousarray(a, np.int32) for a in (tokens, seq_ids, positions))
        logits, ids = np.empty((t.size, self.vocab), np.float32), np.empty(t.size, np.int32)
        hip.check(hip.lib().gl3_forward_decode_batch(self._ctx, _p(t), _p(s), _p(p), t.size, _p(logits), _p(ids)), self._ctx)
        return logits, ids

    def forward_decode_sample(self, token: int, position: int, temperature: float, topp: float, coin: float) -> int:
        a = C.c_int32()
        hip.check(hip.lib().gl3_forward_decode_sample(self._ctx, token, position, temperature, topp, coin, C.byref(a)), self._ctx)
        return a.value

    def generate(self, prompt, n_new: int, temperature: float = 0.0, topp: float = 0.95, rng=None) -> list:
        """Prompt token k at position k (all but the last through the batched prefill), then n_new tokens: greedy for
        temperature 0, else sampled with one coin rng.random() per token."""
        prompt = list(prompt)
        if len(prompt) > 1:
            self.prefill(prompt[:-1], 0)
        cur, out = prompt[-1], []
        for pos in range(len(prompt) - 1, len(prompt) - 1 + n_new):
            if temperature == 0.0:
                cur = self.forward_decode_argmax(cur, pos)
            else:
                cur = self.forward_decode_sample(cur, pos, temperature, topp, float(np.float32(rng.random()) % 1.0))
            out.append(cur)
        return out

    def close(self):
        if getattr(self, "_ctx", None):
            hip.lib().gl3_destroy(self._ctx)
            self._ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def profile_gemm(rows: int, k: int, m: int, f32: bool = False, glu: bool = False, ksplit: bool = False, iters: int = 20, device: int = 0) -> float:
    """Mean microseconds of one launch of the family's GEMM (m > 8) or matvec (m <= 8) on a rows x k matrix; ksplit: the launch may
    leave K-split partial sums, as the output / down projections do."""
    us = C.c_double()
    hip.check(hip.lib().gl3_profile_hybrid_gemm(device, int(f32), rows, k, m, 1 if glu else 2 if ksplit else 0, iters, C.byref(us)))
    return us.value


# ---- random models of the Noditar design (bench.py, examples) -----------------------------------------------------------------------
def noditar_tensor_shapes(config: dict) -> dict:
    """{tensor name: shape} of a Noditar configuration, in file order."""
    W, S = config["width"], config.get("streams", 1)
    out = {"embed": (config["vocab"], W)}
    for i, layer in enumerate(config["layers"]):
        p, m, ff = "l%d." % i, layer["mixer"], layer["mlp"]
        out[p + "norm1"] = (W,)
        if ff:
            out[p + "norm2"] = (W,)
        od = m["heads"] * m["vdim"]
        if layer["type"] == "attention":
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (m["kv_heads"] * m["dim"], W), p + "mix.v": (m["kv_heads"] * m["vdim"], W),
                        p + "mix.g": (od, W), p + "mix.o": (W, od)})
        elif layer["type"] == "latent_attention":
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.dkv": (m["kv_rank"], W), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (od, m["kv_rank"]), p + "mix.g": (od, W), p + "mix.o": (W, od)})
        else:
            gn = m["groups"] * m["state"]
            out.update({p + "mix.in": (2 * od + 2 * gn + m["heads"], W), p + "mix.conv": (od + 2 * gn, m["conv"]), p + "mix.conv.b": (od + 2 * gn,),
                        p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],), p + "mix.D": (m["heads"],), p + "mix.norm": (od,), p + "mix.o": (W, od)})
        if ff:
            out.update({p + "mlp.gate": (ff["ff"], W), p + "mlp.up": (ff["ff"], W), p + "mlp.down": (W, ff["ff"])})
        for q in ((1, 2) if ff else (1,)):
            out.update({p + "hc%d.in" % q: (S,), p + "hc%d.out" % q: (S,), p + "hc%d.mix" % q: (S, S)})
    out["final.norm"] = (W,)
    out["head"] = (config["vocab"], W)
    return out


def vonulix_tensor_shapes(config: dict) -> dict:
    """{tensor name: shape} of a Vonulix configuration, in file order."""
    W, V, L = config["width"], config["vocab"], len(config["layers"])
    d = (config.get("token_side") or {}).get("dim", 0)
    out = {"embed": (V, W)}
    if d:
        out["side.embed"] = (V, L * d)
    for i, layer in enumerate(config["layers"]):
        p, m, ff = "l%d." % i, layer["mixer"], layer.get("mlp")
        od = m["heads"] * m["vdim"]
        out.update({p + "norm1": (W,), p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (m["kv_heads"] * m["dim"], W),
                    p + "mix.v": (m["kv_heads"] * m["vdim"], W), p + "mix.g": (m["heads"], W), p + "mix.o": (W, od)})
        if ff:
            out[p + "norm2"] = (W,)
            f = ff["expert"]["ff"]
            for e in range(ff["router"]["experts"]):
                out.update({p + "mlp.e%d.gate" % e: (f, W), p + "mlp.e%d.up" % e: (f, W), p + "mlp.e%d.down" % e: (W, f)})
            out[p + "mlp.router"] = (ff["router"]["experts"], W)
            if ff.get("shared"):
                f = ff["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (f, W), p + "mlp.shared.up": (f, W), p + "mlp.shared.down": (W, f), p + "mlp.shared.sg": (1, W)})
        out[p + "dwa"] = (i + 2,)
        if d:
            out.update({p + "side.gate": (d, W), p + "side.proj": (W, d), p + "side.norm": (W,)})
    out["final.norm"] = (W,)
    out["head"] = (V, W)
    return out


def kosusun_tensor_shapes(config: dict) -> dict:
    """{tensor name: shape} of a Kosusun configuration, in file order."""
    W, V = config["width"], config["vocab"]
    out = {"embed": (V, W)}
    for i, layer in enumerate(config["layers"]):
        p, m, ff = "l%d." % i, layer["mixer"], layer.get("mlp")
        out[p + "norm1"] = (W,)
        if layer["type"] == "parallel":
            a, r, q = m["left"], m["right"], p + "mix.left."
            nq, nk, nv = a["heads"] * a["dim"], a["kv_heads"] * a["dim"], a["kv_heads"] * a["vdim"]
            out.update({q + "q": (nq, W), q + "q.b": (nq,), q + "k": (nk, W), q + "k.b": (nk,), q + "v": (nv, W), q + "v.b": (nv,), q + "q.norm": (nq,),
                        q + "k.norm": (nk,), q + "sink": (a["heads"],), q + "o": (W, a["heads"] * a["vdim"])})
            q = p + "mix.right."
            out.update({q + "q": (r["heads"] * r["dim"], W), q + "k": (r["heads"] * r["dim"], W), q + "v": (r["heads"] * r["vdim"], W),
                        q + "g": (r["heads"] * r["vdim"], W), q + "o": (W, r["heads"] * r["vdim"])})
        else:
            q, od = p + "mix.", m["heads"] * m["vdim"]
            out.update({q + "q": (m["heads"] * m["dim"], W), q + "k": (m["heads"] * m["dim"], W), q + "v": (od, W), q + "g": (od, W), q + "o": (W, od),
                        q + "norm": (od,), q + "i": (m["heads"], W), q + "i.b": (m["heads"],), q + "f": (m["heads"], W), q + "f.b": (m["heads"],)})
        if ff:
            out.update({p + "mlp.gate": (ff["ff"], W), p + "mlp.up": (ff["ff"], W), p + "mlp.down": (W, ff["ff"])})
    out["final.norm"] = (W,)
    out["head"] = (V, W)
    return out


def kugadra_tensor_shapes(config: dict) -> dict:
    """{tensor name: shape} of a Kugadra configuration, in file order (the head is the embedding table)."""
    W, V = config["width"], config["vocab"]
    out = {"embed": (V, W)}
    for i, layer in enumerate(config["layers"]):
        p, m, ff = "l%d." % i, layer["mixer"], layer.get("mlp")
        od = m["heads"] * m["vdim"]
        out.update({p + "norm1": (W,), p + "norm1b": (W,)})
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


def random_model_dir(path: str, config: dict, seed: int = 0):
    """A model folder with random weights for timing: matrices are random bfloat16 bit patterns of magnitude 2^-9 .. 2^-6 / sqrt-free (cheap to
    make at billions of elements), vectors and tables are benign constants with noise."""
    rng = np.random.default_rng(seed)
    S = config.get("streams", 1)
    t = {}
    vonulix, kosusun, kugadra = (config["architecture"] == a for a in ("Vonulix", "Kosusun", "Kugadra"))
    shapes = (vonulix_tensor_shapes(config) if vonulix else kosusun_tensor_shapes(config) if kosusun else kugadra_tensor_shapes(config) if kugadra
              else noditar_tensor_shapes(config))
    for name, shp in shapes.items():
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        if kosusun and leaf.endswith((".b", ".sink")):
            t[name] = np.full(shp, 3.0 if leaf.endswith("f.b") else 0.0, np.float32)          # forget gates near one, no other offsets
        elif vonulix and leaf in ("norm1", "norm2", "final.norm"):
            t[name] = np.zeros(shp, np.float32)                  # the file holds weight - 1
        elif leaf == "mlp.correction":
            t[name] = np.zeros(shp, np.float32)
        elif leaf == "dwa":
            t[name] = np.concatenate([np.full(shp[0] - 1, 0.1 / max(1, shp[0] - 1)), [0.9]]).astype(np.float32)
        elif leaf == "mlp.router":
            t[name] = (rng.standard_normal(shp) * 4.0 / np.sqrt(shp[1])).astype(np.float32)       # spread choices over the experts
        elif len(shp) == 2 and shp[0] * shp[1] >= 4096 and not leaf.startswith("hc"):
            bits = rng.integers(0, 1 << 9, shp, dtype=np.uint16) + np.uint16(0x3B00)
            bits |= (rng.integers(0, 2, shp, dtype=np.uint16) << np.uint16(15))
            t[name] = bits
        elif leaf.endswith(".mix") and leaf.startswith("hc"):
            t[name] = (np.eye(S) + 0.05 * rng.standard_normal(shp)).astype(np.float32)
        elif leaf.endswith(".in") and leaf.startswith("hc"):
            t[name] = np.full(shp, 1.0 / S, np.float32)
        elif leaf in ("mix.A_log", "mix.dt_bias"):
            t[name] = rng.uniform(-1.0, 0.0, shp).astype(np.float32)
        elif leaf == "mix.conv":
            t[name] = (0.3 * rng.standard_normal(shp)).astype(np.float32)
        elif leaf == "mix.conv.b":
            t[name] = np.zeros(shp, np.float32)
        else:
            t[name] = np.ones(shp, np.float32)
    save_model_dir(path, config, t)
