"""A plain, slow statement of the Zigipel design in numpy (float64): one function per mechanism, written from the design's equations and
sharing nothing with the product path.  The GPU tests compare the framework against it.

Notation: T tokens, E = width, H query heads, G key/value heads, Dk per-head query/key size, Dv per-head value size, R latent size, Dr rotated
size.  Weights are [out, in] and applied as W @ x.  A model is (cfg, W): cfg is the parsed config.json, W maps tensor names to float64 arrays
(integer tables stay integers).  Every sequence starts at position 0."""
import math

import numpy as np


# ---------------------------------------------------------------------------------------------------------------- small pieces
def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """row of the bigram table for every token of ONE sequence: a hash of (previous, current); the first token takes the extra last row."""
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + int(t) * mul_cur) % buckets)
    return np.asarray(rows, dtype=np.int64)


def embed(cfg, W, tokens):
    x = W["embed"][np.asarray(tokens)]
    bg = cfg.get("embedding", {}).get("bigram")
    if bg:
        x = x + W["bigram"][bigram_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"])]
    return x


def token_shift(h, mu):
    """h [T, E] of one sequence from its start: h_t + (h_{t-1} - h_t) * mu, with h_{-1} = 0 (the previous h as it was BEFORE the replacement)."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]], axis=0)
    return h + (prev - h) * mu


def sink_softmax(scores, ok, sink):
    """weights over the visible keys with one more term exp(sink) in the denominator (no key, no value)."""
    s = np.where(ok, scores, -np.inf)
    m = np.maximum(s.max(axis=-1, keepdims=True), sink)
    e = np.where(ok, np.exp(s - m), 0.0)
    return e / (np.exp(sink - m) + e.sum(axis=-1, keepdims=True))


def window_visible(T, size, keep_first=0):
    """[T, T] bool: i sees j when j <= i and (i - j < size or j < keep_first)."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


# ---------------------------------------------------------------------------------------------------------------- rotary with YaRN
def yarn_frequencies(dims, base, scaling):
    """per pair i < dims / 2: base^(-2 i / dims), blended with its 1 / factor between the two correction dims; and the magnitude factor."""
    f = np.asarray([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def corr(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(corr(scaling["fast"])), 0)
    hi = min(math.ceil(corr(scaling["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, pos, freq, mag):
    """x [T, heads, D] with D = 2 len(freq): entry i is paired with entry i + D / 2."""
    half = len(freq)
    ang = np.asarray(pos, dtype=np.float64)[:, None] * freq[None, :]
    c, s = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return np.concatenate([u * c - v * s, v * c + u * s, x[..., 2 * half:]], axis=-1)


# ---------------------------------------------------------------------------------------------------------------- mixers
def attention_mixer(h, W, p, mx, eps):
    """grouped-query attention without rotation over one sequence from its start: unit-rms values, a logarithmic distance penalty, a sliding
    window that also keeps the first tokens, a learned sink, a sigmoid gate per head."""
    T = h.shape[0]
    H, G, Dk, Dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = (h @ W[p + "mix.q"].T).reshape(T, H, Dk)
    k = (h @ W[p + "mix.k"].T).reshape(T, G, Dk)
    v = rms_unit((h @ W[p + "mix.v"].T).reshape(T, G, Dv), eps)
    ok = window_visible(T, mx["mask"]["size"], mx["mask"].get("keep_first", 0))
    dist = np.maximum(np.arange(T)[:, None] - np.arange(T)[None, :], 0).astype(np.float64)
    gate = sigmoid(h @ W[p + "mix.g"].T)  # [T, H]
    out = np.zeros((T, H, Dv))
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * mx["scale"] - W[p + "mix.r1"][hh] * np.log(1.0 + W[p + "mix.r2"][hh] * dist)
        out[:, hh] = (sink_softmax(s, ok, W[p + "mix.sink"][hh]) @ v[:, g]) * gate[:, hh:hh + 1]
    return out.reshape(T, H * Dv) @ W[p + "mix.o"].T


def latent_mixer(h, W, p, mx, eps):
    """attention whose keys and values are expanded from a small normed latent, plus one rotated key part shared by the heads."""
    T = h.shape[0]
    H, Dk, Dr, Dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    q = (h @ W[p + "mix.q"].T).reshape(T, H, Dk + Dr)
    ckr = h @ W[p + "mix.dkv"].T
    c = rms_norm(ckr[:, :R], W[p + "mix.dkv.norm"], eps)
    rot = mx["rot"]
    freq, mag = yarn_frequencies(Dr, rot["base"], rot.get("scaling"))
    pos = np.arange(T)
    kr = rotate_half(ckr[:, None, R:], pos, freq, mag)[:, 0]   # [T, Dr]
    qr = rotate_half(q[:, :, Dk:], pos, freq, mag)             # [T, H, Dr]
    kn = (c @ W[p + "mix.uk"].T).reshape(T, H, Dk)
    v = (c @ W[p + "mix.uv"].T).reshape(T, H, Dv)
    ok = window_visible(T, mx["mask"]["size"])
    out = np.zeros((T, H, Dv))
    for hh in range(H):
        s = (q[:, hh, :Dk] @ kn[:, hh].T + qr[:, hh] @ kr.T) * mx["scale"]
        out[:, hh] = sink_softmax(s, ok, W[p + "mix.sink"][hh]) @ v[:, hh]
    return out.reshape(T, H * Dv) @ W[p + "mix.o"].T


def feed_forward(h, W, p):
    g = h @ W[p + "mlp.gate"].T + W[p + "mlp.gate.b"]
    u = h @ W[p + "mlp.up"].T + W[p + "mlp.up.b"]
    return (gelu_tanh(g) * u) @ W[p + "mlp.down"].T + W[p + "mlp.down.b"]


def layer(x, cfg, W, il):
    """x <- x + (mixer(shift(h)) + ff(h)), h = norm(x): both sublayers read the same normed input; only the mixer's copy is shifted."""
    L, p, eps = cfg["layers"][il], "l%d." % il, cfg["norm"]["eps"]
    h = rms_norm(x, W[p + "norm1"], eps)
    hm = token_shift(h, W[p + "shift"])
    mix = (attention_mixer if L["type"] == "attention" else latent_mixer)(hm, W, p, L["mixer"], eps)
    if L.get("mlp"):
        mix = mix + feed_forward(h, W, p)
    return x + mix


def layer_runs(cfg):
    """the order in which layers run: [(layer, pass or None, first of its pass)] — layers start .. stop - 1 repeat `times` times in a row."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None, False) for i in range(lp["stop"], n)]


def forward(cfg, W, tokens, residuals=None):
    """logits [T, vocab] of ONE sequence from its start; `residuals` (a list) receives the stream after every layer run."""
    x0 = embed(cfg, W, tokens)
    x = x0
    for il, t, first in layer_runs(cfg):
        if first:
            x = np.concatenate([x, x0], axis=-1) @ W["loop.in"].T + W["loop.step"][t]
        x = layer(x, cfg, W, il)
        if residuals is not None:
            residuals.append(x)
    return rms_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T * cfg.get("logit_scale", 1.0)


# ---------------------------------------------------------------------------------------------------------------- test models
def bf16_round(a):
    """nearest bfloat16 (ties to even) of float values, as float64."""
    u = np.asarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def tensor_shapes(cfg):
    E, V = cfg["width"], cfg["vocab"]
    sh = {"embed": (V, E), "final.norm": (E,), "head": (V, E)}
    bg = cfg.get("embedding", {}).get("bigram")
    if bg:
        sh["bigram"] = (bg["buckets"] + 1, E)
    if cfg.get("loop"):
        sh["loop.in"] = (E, 2 * E)
        sh["loop.step"] = (cfg["loop"]["times"], E)
    for il, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % il, L["mixer"]
        sh[p + "norm1"] = (E,)
        sh[p + "shift"] = (E,)
        H, Dk, Dv = mx["heads"], mx["dim"], mx["vdim"]
        if L["type"] == "attention":
            G = mx.get("kv_heads", H)
            sh.update({p + "mix.q": (H * Dk, E), p + "mix.k": (G * Dk, E), p + "mix.v": (G * Dv, E), p + "mix.r1": (H,), p + "mix.r2": (H,), p + "mix.sink": (H,),
                       p + "mix.g": (H, E), p + "mix.o": (E, H * Dv)})
        else:
            R, Dr = mx["kv_rank"], mx["rot_dim"]
            sh.update({p + "mix.q": (H * (Dk + Dr), E), p + "mix.dkv": (R + Dr, E), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * Dk, R), p + "mix.uv": (H * Dv, R),
                       p + "mix.sink": (H,), p + "mix.o": (E, H * Dv)})
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            sh.update({p + "mlp.gate": (F, E), p + "mlp.gate.b": (F,), p + "mlp.up": (F, E), p + "mlp.up.b": (F,), p + "mlp.down": (E, F), p + "mlp.down.b": (E,)})
    return sh


def random_weights(cfg, seed):
    """weights that are exact bfloat16 values: matrices N(0, 1 / in), norm weights around 1, shifts in [0, 1], sinks and penalties of order 1."""
    rng = np.random.default_rng(seed)
    W = {}
    for name, s in tensor_shapes(cfg).items():
        if name.endswith("norm1") or name.endswith("norm") or name == "final.norm":
            a = 1.0 + 0.2 * rng.standard_normal(s)
        elif name.endswith("shift"):
            a = rng.uniform(0.0, 1.0, s)
        elif name.endswith("sink"):
            a = rng.standard_normal(s)
        elif name.endswith("r1"):
            a = rng.uniform(0.2, 1.5, s)
        elif name.endswith("r2"):
            a = rng.uniform(0.05, 2.0, s)
        elif name in ("embed", "bigram", "loop.step"):
            a = rng.standard_normal(s) * (0.3 if name == "loop.step" else 1.0)
        elif name.endswith(".b"):
            a = 0.3 * rng.standard_normal(s)
        else:
            a = rng.standard_normal(s) * (1.5 / math.sqrt(s[-1]))
        W[name] = bf16_round(a)
    return W


def attention_layer(heads, kv_heads, dim, vdim, size, keep_first, scale, ff):
    mx = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, mask=dict(size=size, keep_first=keep_first))
    return dict(type="attention", mixer=mx, mlp=dict(kind="dense", ff=ff) if ff else None)


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, size, scale, ff, base=10000.0, scaling=None):
    rot = dict(base=base, dims=rot_dim)
    if scaling:
        rot["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    mx = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale, mask=dict(size=size), rot=rot)
    return dict(type="latent_attention", mixer=mx, mlp=dict(kind="dense", ff=ff) if ff else None)


def make_config(width, vocab, layers, loop, bigram=(61, 5, 3), eps=1e-5, logit_scale=1.0):
    cfg = dict(architecture="Zigipel", width=width, vocab=vocab, layers=layers, norm=dict(eps=eps), logit_scale=logit_scale,
               embedding=dict(bigram=dict(buckets=bigram[0], mul_prev=bigram[1], mul_cur=bigram[2])))
    if loop:
        cfg["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return cfg


def save_model(cfg, W, folder):
    """config.json + model.safetensors (bf16 matrices) in `folder`."""
    import json
    import os
    import struct

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, a in W.items():
        raw = (np.asarray(a, dtype=np.float32).view(np.uint32) >> 16).astype("<u2").tobytes()
        header[name] = {"dtype": "BF16", "shape": list(np.shape(a)), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
