"""A plain, slow statement of the Nigozen design in numpy (float64 unless told otherwise): one function per mechanism, written from the
design's equations and sharing nothing with the product path.  The GPU tests compare the framework against it.

Notation: T tokens, E = width, H query heads on G key/value heads, Dk = per-head query/key size, Dv = per-head value size.
Weights are [out, in] and applied as W @ x.  A model is (cfg, W): cfg is the parsed config.json, W maps tensor names to arrays."""
import math

import numpy as np


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w over the last axis, var = mean of squared deviations; no bias."""
    mu = x.mean(axis=-1, keepdims=True)
    d = x - mu
    var = (d * d).mean(axis=-1, keepdims=True)
    return d / np.sqrt(var + eps) * w


def rotate_pairs(x, pos, dims, base):
    """x [T, heads, D]; the first `dims` entries of every head are rotated as neighbouring pairs (2i, 2i+1) by the angle
    pos * base^(-2i/dims); the rest pass through."""
    out = x.copy()
    for i in range(dims // 2):
        ang = np.asarray(pos, dtype=np.float64) * (float(base) ** (-2.0 * i / dims))
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


def visible(pos_q, pos_k, chunk):
    """[Tq, Tk] bool: key j is seen by query i when it is not later and, with a chunk size, lies in the same chunk counted from position 0."""
    pq, pk = np.asarray(pos_q)[:, None], np.asarray(pos_k)[None, :]
    ok = pk <= pq
    if chunk:
        ok &= (pq // chunk) == (pk // chunk)
    return ok


def sink_softmax(scores, ok):
    """p_j = exp(s_j) / (1 + sum_k exp(s_k)) over the visible keys: a sink of score 0 that carries no value."""
    m = np.maximum(np.where(ok, scores, -np.inf).max(axis=-1, keepdims=True), 0.0)
    e = np.where(ok, np.exp(scores - m), 0.0)
    return e / (np.exp(-m) + e.sum(axis=-1, keepdims=True))


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def attention_qkv(h, W, p, mx, pos):
    """projections + rotary of one layer for the tokens in h [T, E]: q [T, H, Dk], k [T, G, Dk], v [T, G, Dv] (v before mixing)."""
    T = h.shape[0]
    H, G, Dk, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ W[p + "mix.q"].T).reshape(T, H, Dk)
    k = (h @ W[p + "mix.k"].T).reshape(T, G, Dk)
    v = (h @ W[p + "mix.v"].T).reshape(T, G, Dv)
    rot = mx.get("rot")
    if rot and rot.get("dims", 0) > 0:
        q = rotate_pairs(q, pos, rot["dims"], rot["base"])
        k = rotate_pairs(k, pos, rot["dims"], rot["base"])
    return q, k, v


def mix_values(v, v_first, lam):
    return (1.0 - lam) * v + lam * v_first


def attend(q, k, v, pos_q, pos_k, scale, chunk):
    """q [Tq, H, Dk] over keys k [Tk, G, Dk], values v [Tk, G, Dv] -> [Tq, H * Dv]; query head h reads kv head h // (H / G)."""
    Tq, H, _ = q.shape
    G = k.shape[1]
    ok = visible(pos_q, pos_k, chunk)
    out = np.zeros((Tq, H, v.shape[2]), dtype=q.dtype)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh, :] @ k[:, g, :].T) * scale
        out[:, hh, :] = sink_softmax(s, ok) @ v[:, g, :]
    return out.reshape(Tq, -1)


def dense_ffn(h, W, p):
    return gelu_erf(h @ W[p + "mlp.up"].T) @ W[p + "mlp.down"].T


def route(h, Wr, top):
    """router logits -> (chosen experts [T, top], weights [T, top]): the `top` largest logits, soft-max over those alone."""
    z = h @ Wr.T
    idx = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zs = np.take_along_axis(z, idx, axis=-1)
    e = np.exp(zs - zs.max(axis=-1, keepdims=True))
    return idx, e / e.sum(axis=-1, keepdims=True)


def moe_ffn(h, W, p, ml):
    idx, w = route(h, W[p + "mlp.router"], ml["router"]["top"])
    out = np.zeros((h.shape[0], W[p + "mlp.e0.down"].shape[0]), dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            a = np.maximum(W[p + "mlp.e%d.up" % e] @ h[t], 0.0) ** 2
            out[t] += w[t, j] * (W[p + "mlp.e%d.down" % e] @ a)
    return out


def router_margin(h, Wr, top):
    """per token: gap between the last chosen and the first rejected router logit, in units of the logits' spread (inf when every expert is chosen)"""
    z = np.sort(h @ Wr.T, axis=-1)[:, ::-1]
    if top >= z.shape[1]:
        return np.full(h.shape[0], np.inf)
    return (z[:, top - 1] - z[:, top]) / (z.std(axis=-1) + 1e-30)


def forward(cfg, W, tokens, dtype=np.float64, return_layers=False, margins=None):
    """Whole-sequence forward of one request from position 0: logits [T, vocab] (and the residual stream after every layer).
    margins: a list that receives, per mixture-of-experts layer, every token's router_margin."""
    W = {k: np.asarray(v, dtype=dtype) for k, v in W.items()}
    T = len(tokens)
    pos = np.arange(T)
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    v_first = None
    layers = []
    for il, L in enumerate(cfg["layers"]):
        p = "l%d." % il
        mx = L["mixer"]
        assert L["type"] == "attention"
        h = layer_norm(x, W[p + "norm1"], eps)
        q, k, v = attention_qkv(h, W, p, mx, pos)
        if mx.get("v_mix"):
            if v_first is None:
                v_first = v
            else:
                v = mix_values(v.reshape(T, -1), v_first.reshape(T, -1), float(W[p + "mix.vmix"])).reshape(v.shape)  # per token, over all its value entries
        chunk = (mx.get("mask") or {}).get("size", 0)
        a = attend(q, k, v, pos, pos, mx["scale"], chunk)
        a = a * sigmoid(h @ W[p + "mix.g"].T)
        x = x + layer_norm(a @ W[p + "mix.o"].T, W[p + "norm1b"], eps)
        ml = L.get("mlp")
        if ml:
            h2 = layer_norm(x, W[p + "norm2"], eps)
            f = dense_ffn(h2, W, p) if ml["kind"] == "dense" else moe_ffn(h2, W, p, ml)
            if margins is not None and ml["kind"] == "moe":
                margins.append(router_margin(h2, W[p + "mlp.router"], ml["router"]["top"]))
            x = x + layer_norm(f, W[p + "norm2b"], eps)
        layers.append(x.copy())
    logits = layer_norm(x, W["final.norm"], eps) @ W["embed"].T
    return (logits, np.stack(layers)) if return_layers else logits


# ----------------------------------------------------------------------------------------------- making small models
def make_config(width, vocab, layers, eps=1e-5, embed_scale=1.0):
    """layers: list of dicts(heads, kv_heads, dim, vdim, rot_dims, rot_base, scale, chunk, v_mix, mlp) with mlp one of
    None, ("dense", ff), ("moe", ff, experts, top)."""
    out = []
    for L in layers:
        mixer = {"heads": L["heads"], "kv_heads": L["kv_heads"], "dim": L["dim"], "vdim": L["vdim"], "mask": {"size": L["chunk"]},
                 "rot": {"base": L.get("rot_base", 10000.0), "dims": L["rot_dims"]}, "scale": L["scale"], "v_mix": bool(L.get("v_mix", False))}
        m = L.get("mlp")
        if m is None:
            mlp = None
        elif m[0] == "dense":
            mlp = {"kind": "dense", "ff": m[1]}
        else:
            mlp = {"kind": "moe", "expert": {"ff": m[1]}, "router": {"experts": m[2], "top": m[3]}}
        out.append({"type": "attention", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Nigozen", "embedding": {"scale": embed_scale}, "layers": out, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def bf16_round(a):
    """float32 values rounded to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.view(np.float32).reshape(np.shape(a))


def random_weights(cfg, seed, gain=1.0):
    """Random weights that are exact in bfloat16 (so that the file and the reference hold the same numbers)."""
    rng = np.random.default_rng(seed)
    E, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(o, i, g=1.0):
        return bf16_round(rng.standard_normal((o, i)).astype(np.float32) * (g * gain / math.sqrt(i)))

    def vec(n):
        return bf16_round((1.0 + 0.2 * rng.standard_normal(n)).astype(np.float32))

    W["embed"] = bf16_round(rng.standard_normal((V, E)).astype(np.float32))
    for il, L in enumerate(cfg["layers"]):
        p = "l%d." % il
        mx = L["mixer"]
        for n in ("norm1", "norm1b"):
            W[p + n] = vec(E)
        W[p + "mix.q"] = mat(mx["heads"] * mx["dim"], E, 1.5)
        W[p + "mix.k"] = mat(mx["kv_heads"] * mx["dim"], E, 1.5)
        W[p + "mix.v"] = mat(mx["kv_heads"] * mx["vdim"], E)
        W[p + "mix.g"] = mat(mx["heads"] * mx["vdim"], E)
        W[p + "mix.o"] = mat(E, mx["heads"] * mx["vdim"])
        W[p + "mix.vmix"] = bf16_round(np.float32(rng.uniform(0.2, 0.8)))
        ml = L["mlp"]
        if ml:
            for n in ("norm2", "norm2b"):
                W[p + n] = vec(E)
            if ml["kind"] == "dense":
                W[p + "mlp.up"] = mat(ml["ff"], E)
                W[p + "mlp.down"] = mat(E, ml["ff"])
            else:
                for e in range(ml["router"]["experts"]):
                    W[p + "mlp.e%d.up" % e] = mat(ml["expert"]["ff"], E, 2.0)
                    W[p + "mlp.e%d.down" % e] = mat(E, ml["expert"]["ff"])
                W[p + "mlp.router"] = mat(ml["router"]["experts"], E, 3.0)
    W["final.norm"] = vec(E)
    return W


def write_model(folder, cfg, W):
    """config.json + model.safetensors (bfloat16) in `folder`."""
    import json
    import os
    import struct

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    head, blobs, at = {}, [], 0
    for name, a in W.items():
        a = np.asarray(a, dtype=np.float32)
        raw = (a.view(np.uint32) >> 16).astype(np.uint16).tobytes()
        head[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(head).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
