"""GPU tests of the Zigipel model class: the engine (llama_lite over the MI355X backend) against the plain numpy reference of
tests/zigipel_ref.py, on small models with their own sizes and random weights.

f32 serving is the sharp instrument: with 32-bit arithmetic end to end ONE key wrongly seen or hidden among a hundred, a window that is
one position off, a lost state row or a forgotten sink moves a logit row by 1e-3 of its spread and more, ten times the gate (1e-4).
bf16 serving is gated at its rounding level.  Where even f32 could hide a fault (a far kept token, a window's edge, the sink) a test
shows that the data discriminate: the same rows are far from the reference computed with the neighbouring rule."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import harness as T
import llama_box_amd as L
import zigipel_ref as R
from llama_box_amd.trace import TraceSession

pytestmark = pytest.mark.gpu

F32_GATE, BF16_GATE = 1e-4, 5e-2


def row_err(got, ref):
    """per row: rms of the difference (means removed) over the rms of the reference row (mean removed)"""
    d = got - ref
    d = d - d.mean(axis=-1, keepdims=True)
    r = ref - ref.mean(axis=-1, keepdims=True)
    return np.sqrt((d * d).mean(axis=-1)) / np.sqrt((r * r).mean(axis=-1))


def toks(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def cfg_a():
    # a latent layer in front, two attention layers and a latent one repeated three times, one layer behind; 2, 1 and 3 query heads per kv head; key size != value
    # size; windows 7, 16, 5 and 33 with 0, 3, 9 (more than the window) kept first tokens; a layer without feed-forward; YaRN on two of three latent layers
    return R.make_config(64, 97, [
        R.latent_layer(heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=40, size=7, scale=0.2, ff=72, base=100.0, scaling=(4.0, 32, 8.0, 1.0)),
        R.attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, size=16, keep_first=3, scale=0.25, ff=48),
        R.attention_layer(heads=3, kv_heads=3, dim=24, vdim=8, size=5, keep_first=9, scale=0.2, ff=None),
        R.latent_layer(heads=2, dim=8, rot_dim=16, vdim=40, kv_rank=24, size=33, scale=0.3, ff=40, base=5000.0),
        R.attention_layer(heads=6, kv_heads=2, dim=8, vdim=16, size=11, keep_first=0, scale=0.35, ff=32),
    ], loop=(1, 4, 3), bigram=(61, 5, 3), eps=3e-5, logit_scale=0.8)


def cfg_b():
    # rows that are no multiple of 8 (width 52, cache rows of 36, 22 and 30 values), one head, a range that starts at layer 0 and runs once, logits unscaled,
    # a head size above 128
    return R.make_config(52, 50, [
        R.latent_layer(heads=1, dim=12, rot_dim=2, vdim=20, kv_rank=20, size=9, scale=0.3, ff=20, base=10.0, scaling=(2.0, 8, 4.0, 1.0)),
        R.attention_layer(heads=3, kv_heads=3, dim=12, vdim=12, size=4, keep_first=1, scale=0.3, ff=36),
        R.attention_layer(heads=2, kv_heads=1, dim=136, vdim=20, size=300, keep_first=0, scale=0.05, ff=None),
        R.latent_layer(heads=5, dim=6, rot_dim=0, vdim=10, kv_rank=30, size=3, scale=0.4, ff=12),
    ], loop=(0, 2, 1), bigram=(7, 31, 1), eps=1e-6, logit_scale=1.0)


def cfg_c():
    # the whole model repeats; windows longer than a block of 64 cells; vocabulary not a multiple of anything
    return R.make_config(96, 257, [
        R.latent_layer(heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=48, size=80, scale=0.18, ff=160, base=50000.0, scaling=(3.0, 64, 16.0, 1.0)),
        R.attention_layer(heads=8, kv_heads=2, dim=24, vdim=24, size=70, keep_first=5, scale=0.2, ff=160),
    ], loop=(0, 2, 2), bigram=(251, 13, 5), eps=1e-6, logit_scale=0.6)


CONFIGS = {"a": cfg_a, "b": cfg_b, "c": cfg_c}


class Served:
    def __init__(self, backend, tmp_path, cfg, seed, dtype, max_tokens=512, n_ubatch=64, W=None):
        self.cfg, self.W = cfg, W if W is not None else R.random_weights(cfg, seed)
        R.save_model(cfg, self.W, str(tmp_path))
        self.s = TraceSession(str(tmp_path), "float32" if dtype == "f32" else "bfloat16", max_tokens=max_tokens, n_ubatch=n_ubatch, backend=backend)
        self.gate = F32_GATE if dtype == "f32" else BF16_GATE

    def ref(self, tokens):
        return R.forward(self.cfg, self.W, tokens)

    def feed(self, rid, tokens, end=False):
        return self.s.step([{"id": rid, "tokens": list(tokens), "want": list(range(len(tokens)))}], [rid] if end else [])

    def free(self):
        self.s.close()


# ------------------------------------------------------------------------------------------------ whole models through the engine
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("which", ["a", "b", "c"])
def test_whole_prompt(backend, tmp_path, plog, which, dtype):
    s = Served(backend, tmp_path, CONFIGS[which](), 11, dtype)
    t = toks(150, s.cfg["vocab"], 5)  # three micro-batches of 64 / 64 / 22 tokens; every position's logits
    e = row_err(s.feed("w", t, end=True), s.ref(t))
    plog(f"zigipel whole prompt cfg {which} {dtype}: max row error {e.max():.3e}")
    assert e.max() <= s.gate, (int(np.argmax(e)), float(e.max()))
    assert backend.stat("attn_f32_nodes") > 0
    s.free()


def single_layer(kind, **kw):
    if kind == "attention":
        d = dict(heads=4, kv_heads=2, dim=16, vdim=12, size=6, keep_first=2, scale=0.25, ff=None)
        d.update(kw)
        layer = R.attention_layer(**d)
    else:
        d = dict(heads=3, dim=8, rot_dim=8, vdim=12, kv_rank=24, size=6, scale=0.3, ff=None, base=100.0, scaling=(4.0, 16, 8.0, 1.0))
        d.update(kw)
        layer = R.latent_layer(**d)
    return layer


@pytest.mark.parametrize("case", ["attention", "latent", "latent_no_scaling", "ffn_only_differs", "no_loop"])
def test_one_mechanism_at_a_time(backend, tmp_path, case):
    """single-layer models: one mixer and nothing else (no feed-forward), so that a fault has one place to be"""
    if case == "attention":
        cfg = R.make_config(48, 40, [single_layer("attention")], loop=(0, 1, 1))
    elif case == "latent":
        cfg = R.make_config(48, 40, [single_layer("latent")], loop=(0, 1, 1))
    elif case == "latent_no_scaling":
        cfg = R.make_config(48, 40, [single_layer("latent", scaling=None, rot_dim=4)], loop=(0, 1, 1))
    elif case == "ffn_only_differs":
        cfg = R.make_config(48, 40, [single_layer("attention", ff=56)], loop=(0, 1, 2))
    else:
        cfg = R.make_config(48, 40, [single_layer("attention"), single_layer("latent", ff=24)], loop=None)
    if case == "no_loop":
        cfg.pop("loop", None)
    s = Served(backend, tmp_path, cfg, 21, "f32")
    t = toks(40, 40, 3)
    assert row_err(s.feed("w", t, end=True), s.ref(t)).max() <= F32_GATE
    s.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_against_token_by_token(backend, tmp_path, dtype):
    s = Served(backend, tmp_path, cfg_a(), 12, dtype)
    t = toks(45, s.cfg["vocab"], 6)
    # the first tokens of a sequence one at a time: position 0 sees itself and the sink, reads the zero state row and the bigram table's last row
    rows = np.concatenate([s.feed("x", [tok]) for tok in t])
    e = row_err(rows, s.ref(t))
    assert e.max() <= s.gate, (int(np.argmax(e)), float(e.max()))
    s.free()


@pytest.mark.parametrize("which", ["a", "b", "c"])
def test_portions_of_every_size(backend, tmp_path, which):
    s = Served(backend, tmp_path, CONFIGS[which](), 13, "f32")
    t = toks(131, s.cfg["vocab"], 7)
    cuts = [2, 3, 2, 7, 1, 16, 5, 2, 64, 2, 9, 18]  # down to two tokens; cuts fall inside windows of 3 .. 33 positions and inside the kept first tokens
    assert sum(cuts) == len(t)
    at, rows = 0, []
    for n in cuts:
        rows.append(s.feed("x", t[at:at + n]))
        at += n
    e = row_err(np.concatenate(rows), s.ref(t))
    assert e.max() <= s.gate, (int(np.argmax(e)), float(e.max()))
    s.free()


def test_long_decoding_past_every_window(backend, tmp_path):
    s = Served(backend, tmp_path, cfg_c(), 14, "f32", max_tokens=512)
    t = toks(330, s.cfg["vocab"], 8)  # 3 prompt tokens, then single steps: the windows of 80 and 70 pass over decoded tokens, the visible part of the cache grows past 256 cells
    rows = [s.feed("x", t[:3])] + [s.feed("x", [tok]) for tok in t[3:]]
    e = row_err(np.concatenate(rows), s.ref(t))
    assert e.max() <= s.gate, (int(np.argmax(e)), float(e.max()))
    s.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_unequal_requests_in_mixed_batches_with_cells_and_slots_used_again(backend, tmp_path, dtype):
    cfg = cfg_a()
    reqs = {name: toks(n, cfg["vocab"], 20 + i) for i, (name, n) in enumerate([("p", 190), ("q", 33), ("r", 1), ("s", 240), ("t", 57), ("u", 175), ("v", 2)])}
    # 256 + 4 x 64 cells for 698 tokens in total: the cells of ended requests are handed out again, as are the four sequence slots with their state rows
    sv = Served(backend, tmp_path, cfg, 15, dtype, max_tokens=256, n_ubatch=64)
    fed = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    plan = [  # (request, tokens) per step: portions beside single tokens, requests left out of steps, ends in between
        [("p", 40), ("q", 2)], [("p", 1), ("q", 30), ("r", 1)], [("p", 1), ("q", 1), ("s", 64), ("v", 2)], [("p", 148), ("s", 3)], [("s", 173)],
        [("t", 20), ("u", 2)], [("t", 1), ("u", 170)], [("u", 1), ("t", 36)], [("u", 2)],
    ]
    for step in plan:
        entries, ends = [], []
        for name, n in step:
            a = fed[name]
            entries.append({"id": name, "tokens": reqs[name][a:a + n], "want": list(range(n))})
            fed[name] = a + n
            if fed[name] == len(reqs[name]):
                ends.append(name)
        rows = sv.s.step(entries, ends)
        at = 0
        for name, n in step:
            got[name].append(rows[at:at + n])
            at += n
    for k in reqs:
        assert fed[k] == len(reqs[k])
        e = row_err(np.concatenate(got[k]), sv.ref(reqs[k]))
        assert e.max() <= sv.gate, (k, int(np.argmax(e)), float(e.max()))
    sv.free()


def test_a_slot_used_again_starts_from_nothing(backend, tmp_path):
    """a request that takes over the slot (state rows, previous token) and the cells of an ended one gives what it gives alone"""
    s = Served(backend, tmp_path, cfg_a(), 16, "f32", max_tokens=64)
    a, b = toks(50, s.cfg["vocab"], 1), toks(60, s.cfg["vocab"], 2)
    s.feed("a", a, end=True)
    rows = np.concatenate([s.feed("b", b[:1]), s.feed("b", b[1:7]), s.feed("b", b[7:], end=True)])
    assert row_err(rows, s.ref(b)).max() <= F32_GATE
    s.free()


def test_greedy_generation_through_the_engine(backend, tmp_path, H):
    s = Served(backend, tmp_path, cfg_a(), 17, "f32")
    prompt = toks(9, s.cfg["vocab"], 9)
    s.s.step([{"id": "g", "tokens": prompt, "want": [len(prompt) - 1]}], [])
    seq = list(prompt)
    for _ in range(24):
        tok = H.llm_sample_greedy(s.s.ctx, -1)  # the engine's own sampler on the engine's own logits
        ref_row = s.ref(seq)[-1]
        top2 = np.sort(ref_row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(ref_row).max():
            assert tok == int(np.argmax(ref_row))
        else:
            tok = int(np.argmax(ref_row))
        seq.append(tok)
        s.s.step([{"id": "g", "tokens": [tok], "want": [0]}], [])
    s.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_fused_steps_equal_the_unfused_nodes(backend, tmp_path, dtype):
    """token shift, state rows, gated activation with biases, bias + sublayer sum + residual, head gates, latent cache rows and query rows as single launches: bit for bit
    what the graph's own nodes give, for a prompt portion and for single tokens"""
    cfg = cfg_a()
    t = toks(90, cfg["vocab"], 41)
    rows = {}
    launches = {}
    for fusion in (1, 0):
        backend.set_option("fusion", fusion)
        s = Served(backend, tmp_path / str(fusion), cfg, 18, dtype)
        before = backend.stat("kernel_launches")
        rows[fusion] = np.concatenate([s.feed("x", t[:70])] + [s.feed("x", [tok]) for tok in t[70:]])
        launches[fusion] = backend.stat("kernel_launches") - before
        s.free()
    backend.set_option("fusion", 1)
    assert np.array_equal(rows[0], rows[1])
    assert launches[1] < 0.7 * launches[0]


# ------------------------------------------------------------------------------------------------ edges: the data must show a rule that is one off
def _variant(cfg, il, **mask):
    c = copy.deepcopy(cfg)
    c["layers"][il]["mixer"]["mask"].update(mask)
    return c


@pytest.mark.parametrize("kind", ["attention", "latent"])
@pytest.mark.parametrize("how", ["prompt", "decoded"])
def test_window_edges_and_kept_first_tokens_show(backend, tmp_path, kind, how):
    """one layer, a window of 12 (attention: 3 kept first tokens).  The engine's rows match the reference with exactly this rule and are far from the reference with a
    window one longer or shorter, with one kept token more or fewer, without the sink, and without the distance penalty — in a prompt and token by token."""
    layer = single_layer(kind, size=12, keep_first=3) if kind == "attention" else single_layer(kind, size=12)
    cfg = R.make_config(48, 40, [layer], loop=(0, 1, 1))
    W = R.random_weights(cfg, 31)
    for name in W:  # sharper scores: one key stands out in most rows, so a key that comes or goes at an edge is seen
        if name.endswith("mix.q"):
            W[name] = R.bf16_round(W[name] * 3.0)
    s = Served(backend, tmp_path, cfg, 0, "f32", W=W)
    t = toks(60, 40, 4)
    rows = s.feed("w", t, end=True) if how == "prompt" else np.concatenate([s.feed("w", t[:5])] + [s.feed("w", [x]) for x in t[5:]])
    assert row_err(rows, R.forward(cfg, W, t)).max() <= F32_GATE
    tail = slice(20, 60)  # positions whose window has left the start behind
    others = [_variant(cfg, 0, size=13), _variant(cfg, 0, size=11)]
    if kind == "attention":
        others += [_variant(cfg, 0, keep_first=4), _variant(cfg, 0, keep_first=2)]
    for other in others:
        assert row_err(rows[tail], R.forward(other, W, t)[tail]).max() > 20 * F32_GATE
    W2 = dict(W)
    W2["l0.mix.sink"] = W["l0.mix.sink"] - 30.0  # a sink that weighs nothing
    assert row_err(rows, R.forward(cfg, W2, t)).max() > 20 * F32_GATE
    if kind == "attention":
        W3 = dict(W)
        W3["l0.mix.r1"] = W["l0.mix.r1"] * 0.0
        assert row_err(rows[tail], R.forward(cfg, W3, t)[tail]).max() > 20 * F32_GATE
    s.free()


def test_far_kept_tokens_in_bf16(backend, tmp_path):
    """bf16 serving, 400 tokens, a window of 8 and 2 kept first tokens: with queries scaled up the kept tokens far back carry real weight — dropping them (keep_first 0)
    moves the rows far beyond bf16's rounding"""
    cfg = R.make_config(64, 40, [R.attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, size=8, keep_first=2, scale=0.25, ff=None)], loop=(0, 1, 1))
    W = R.random_weights(cfg, 33)
    W["l0.mix.r1"] = W["l0.mix.r1"] * 0.05  # a mild penalty, so that distance 400 does not silence the kept tokens
    s = Served(backend, tmp_path, cfg, 0, "bf16", W=W)
    t = toks(400, 40, 5)
    rows = np.concatenate([s.feed("w", t[:330])] + [s.feed("w", [x]) for x in t[330:]])
    assert row_err(rows, R.forward(cfg, W, t)).max() <= BF16_GATE
    assert row_err(rows[300:], R.forward(_variant(cfg, 0, keep_first=0), W, t)[300:]).max() > 4 * BF16_GATE
    s.free()


# ------------------------------------------------------------------------------------------------ mechanisms alone, through the C-ABI
def run(backend, build):
    g = T.G(backend)
    outs = build(g)
    res = g.compute(outs if isinstance(outs, (list, tuple)) else [outs])
    g.free()
    return res


def bf16_bits(a):
    return (np.ascontiguousarray(R.bf16_round(a).astype(np.float32)).view(np.uint32) >> 16).astype(np.uint16)


@pytest.mark.parametrize("kv_type", [L.F32, L.BF16])
@pytest.mark.parametrize("n_q,n_kv,heads,kv_heads,dk,dv,size,keep", [
    (1, 700, 4, 2, 64, 40, 90, 5),       # one decoded token over 700 cells: the window's blocks and the first block
    (3, 300, 6, 1, 80, 64, 50, 0),       # a shared key/value head (a latent row's shape)
    (70, 333, 4, 1, 64, 40, 50, 3),      # a prompt portion (tile / matrix-core form), window edges inside the portion
    (128, 640, 2, 2, 128, 128, 0, 0),    # no window at all: plain causal with distances
    (33, 100, 3, 3, 40, 72, 9, 12),
    (2, 90, 2, 1, 576, 512, 30, 0),      # head sizes of a large latent
    (40, 300, 4, 1, 576, 512, 100, 0),   # ... in a prompt portion: 160 (token, head) pairs on the wide matrix-core form over a bf16 cache
    (45, 150, 3, 1, 160, 136, 40, 2),    # a shared head just beyond 128 entries, value rows that are no multiple of 32
    (9, 777, 16, 1, 320, 256, 500, 0),
])
def test_attention_with_distance_penalty_and_learned_sinks(backend, H, kv_type, n_q, n_kv, heads, kv_heads, dk, dv, size, keep):
    rng = np.random.default_rng(n_q * 1000 + n_kv)
    q = rng.standard_normal((n_q, heads, dk)).astype(np.float32)
    k = rng.standard_normal((n_kv, kv_heads, dk)).astype(np.float32)
    v = rng.standard_normal((n_kv, kv_heads, dv)).astype(np.float32)
    sink = rng.standard_normal(heads).astype(np.float32)
    r1 = rng.uniform(0.2, 1.5, heads).astype(np.float32)
    r2 = rng.uniform(0.05, 2.0, heads).astype(np.float32)
    q_pos = np.arange(n_kv - n_q, n_kv)
    dist = q_pos[:, None] - np.arange(n_kv)[None, :]
    ok = (dist >= 0) & (((dist < size) if size else True) | (np.arange(n_kv)[None, :] < keep))
    mask = np.full((64 * ((n_q + 63) // 64), n_kv), -np.inf, np.float32)
    mask[:n_q][ok] = dist[ok]
    scale = 1.0 / np.sqrt(dk)
    if kv_type == L.BF16:
        k, v = R.bf16_round(k).astype(np.float32), R.bf16_round(v).astype(np.float32)
        wide = kv_heads == 1 and n_q * heads >= 128 and (dk > 128 or dv > 128) and dk <= 640 and dv <= 512
        if dk % 8 == 0 and dv % 8 == 0 and ((n_q >= 32 and dk <= 128 and dv <= 128) or wide):
            q = R.bf16_round(q).astype(np.float32)  # prompt portions over a bf16 cache run on the matrix cores: the queries are rounded to bf16 like every mat-mul operand

    def build(g):
        tq = g.new(L.F32, [dk, heads, n_q], q)
        tk = g.new(kv_type, [dk * kv_heads, n_kv], bf16_bits(k) if kv_type == L.BF16 else k)
        tv = g.new(kv_type, [dv * kv_heads, n_kv], bf16_bits(v) if kv_type == L.BF16 else v)
        esz = 2 if kv_type == L.BF16 else 4
        kk = H.ggml_view_3d(g.ctx, tk, dk, n_kv, kv_heads, dk * kv_heads * esz, dk * esz, 0)
        vv = H.ggml_view_3d(g.ctx, tv, dv, n_kv, kv_heads, dv * kv_heads * esz, dv * esz, 0)
        r = H.ggml_flash_attn_ext(g.ctx, H.ggml_permute(g.ctx, tq, 0, 2, 1, 3), kk, vv, g.new(L.F32, [n_kv, mask.shape[0]], mask), scale, 0.0, 0.0)
        H.ggml_flash_attn_ext_set_prec(r, 10)
        H.ggml_flash_attn_ext_add_sinks(r, g.new(L.F32, [heads], sink))
        H.ggml_flash_attn_ext_add_log_distance(r, g.new(L.F32, [heads, 2], np.stack([r1, r2])))
        return r

    got = run(backend, build)[0].reshape(n_q, heads, dv)
    ref = np.zeros((n_q, heads, dv))
    for h in range(heads):
        g_ = h // (heads // kv_heads)
        s = (q[:, h].astype(np.float64) @ k[:, g_].astype(np.float64).T) * scale - r1[h] * np.log(1.0 + r2[h] * np.maximum(dist, 0))
        ref[:, h] = R.sink_softmax(s, ok, float(sink[h])) @ v[:, g_].astype(np.float64)
    assert np.abs(got - ref).max() <= (2e-5 if kv_type == L.F32 else 2e-3) * max(1.0, np.abs(ref).max())


def test_concat_along_every_dimension(backend, H):
    rng = np.random.default_rng(5)
    a = rng.standard_normal((3, 4, 5, 6)).astype(np.float32)  # numpy order: [ne3, ne2, ne1, ne0]
    for dim, shape in ((0, (3, 4, 5, 2)), (1, (3, 4, 7, 6)), (2, (3, 1, 5, 6)), (3, (2, 4, 5, 6))):
        b = rng.standard_normal(shape).astype(np.float32)

        def build(g):
            ta = g.new(L.F32, list(a.shape[::-1]), a)
            tb = g.new(L.F32, list(shape[::-1]), b)
            return H.ggml_concat(g.ctx, ta, tb, dim)

        got = run(backend, build)[0]
        assert np.array_equal(got, np.concatenate([a, b], axis=3 - dim))

    # sources seen through strides: the leading part of every row of one tensor joined with a permuted view of another
    x = rng.standard_normal((1, 6, 4, 10)).astype(np.float32)
    y = rng.standard_normal((1, 4, 6, 3)).astype(np.float32)

    def build2(g):
        tx = g.new(L.F32, [10, 4, 6], x)
        ty = g.new(L.F32, [3, 6, 4], y)
        vx = H.ggml_view_3d(g.ctx, tx, 7, 4, 6, 10 * 4, 40 * 4, 0)
        return H.ggml_concat(g.ctx, vx, H.ggml_permute(g.ctx, ty, 0, 2, 1, 3), 0)

    got = run(backend, build2)[0]
    assert np.array_equal(got[0], np.concatenate([x[0, :, :, :7], y[0].transpose(1, 0, 2)], axis=-1))


def test_rotation_over_a_frequency_table(backend, H):
    """rotate-half pairs, every pair's angle = position x its table entry, cos and sin times a magnitude; the source is a strided part of wider rows"""
    rng = np.random.default_rng(6)
    n_tok, heads, wide, dr = 9, 3, 20, 8
    x = rng.standard_normal((n_tok, heads, wide)).astype(np.float32)
    pos = np.array([0, 1, 2, 3, 500, 501, 4000, 77, 5], np.int32)
    freq, mag = R.yarn_frequencies(dr, 10000.0, dict(factor=4.0, original=64, fast=8.0, slow=1.0))

    def build(g):
        tx = g.new(L.F32, [wide, heads, n_tok], x)
        part = H.ggml_view_3d(g.ctx, tx, dr, heads, n_tok, wide * 4, wide * heads * 4, (wide - dr) * 4)
        r = H.ggml_rope_ext(g.ctx, part, g.new(L.I32, [n_tok], pos), g.new(L.F32, [dr // 2], freq.astype(np.float32)), dr, 2, 0, 10000.0, 1.0, 0.0, float(mag), 32.0, 1.0)
        H.ggml_rope_set_freq_table(r)
        return r

    got = run(backend, build)[0].reshape(n_tok, heads, dr)
    ref = R.rotate_half(x[:, :, wide - dr:].astype(np.float64), pos, freq.astype(np.float32).astype(np.float64), mag)
    assert np.abs(got - ref).max() <= 1e-3  # (an f32 angle at position 4000 is 2e-4 rad from the f64 one)
    assert np.abs(got[:4] - ref[:4]).max() <= 2e-6


# ------------------------------------------------------------------------------------------------ the program, and random configurations
def test_trace_run_command_line(tmp_path):
    """bin/trace_run as a program: steps on standard input, one 'done <step>' line each, <step>.f32 only where logits were asked for"""
    cfg = cfg_b()
    W = R.random_weights(cfg, 31)
    model_dir, out_dir = str(tmp_path / "model"), str(tmp_path / "out")
    R.save_model(cfg, W, model_dir)
    t = toks(21, cfg["vocab"], 32)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": t[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": t[9:20], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": t[20:], "want": [0]}, {"id": "y", "tokens": t[:2], "want": [1]}], "end": ["x", "y"]}]
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    p = subprocess.run([sys.executable, exe, "--model", model_dir, "--dtype", "float32", "--out", out_dir, "--max-tokens", "128"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert sorted(os.listdir(out_dir)) == ["0.f32", "2.f32"]
    ref = R.forward(cfg, W, t)
    r0 = np.fromfile(os.path.join(out_dir, "0.f32"), dtype="<f4").reshape(2, -1)
    r2 = np.fromfile(os.path.join(out_dir, "2.f32"), dtype="<f4").reshape(2, -1)
    assert row_err(r0, ref[[0, 8]]).max() <= F32_GATE
    assert row_err(r2, np.stack([ref[20], ref[1]])).max() <= F32_GATE  # request y repeats x's first tokens in its own slot


def random_config(seed):
    """a configuration drawn at random: widths with and without whole groups of 8 values, 1 - 5 layers of either mixer in any order, any repeated range, windows
    from 1 position up, kept first tokens, with and without feed-forward / YaRN"""
    rng = np.random.default_rng(1000 + seed)
    width = int(rng.choice([32, 48, 64, 72, 96, 100, 128, 36]))
    vocab = int(rng.integers(40, 300))
    layers = []
    for _ in range(int(rng.integers(1, 6))):
        ff = None if rng.integers(0, 4) == 0 else int(rng.choice([16, 40, 64, 100]))
        size = int(rng.choice([1, 2, 5, 16, 33, 64, 100, 257]))
        if rng.integers(0, 2):
            G = int(rng.choice([1, 2, 3, 4]))
            Hh = G * int(rng.choice([1, 1, 2, 3]))
            dk = int(rng.choice([8, 12, 16, 24, 32, 40, 64, 96, 20]))
            layers.append(R.attention_layer(heads=Hh, kv_heads=G, dim=dk, vdim=int(rng.choice([4, 8, 12, 16, 24, 48, 64])), size=size,
                                            keep_first=int(rng.choice([0, 0, 1, 4, 7])), scale=float(rng.choice([dk ** -0.5, 0.1, 0.25])), ff=ff))
        else:
            dr = int(rng.choice([0, 2, 4, 8, 16, 32]))
            scaling = None if (dr == 0 or rng.integers(0, 3) == 0) else (float(rng.choice([2.0, 4.0, 40.0])), int(rng.choice([8, 64, 512])), float(rng.choice([32.0, 8.0])), float(rng.choice([1.0, 2.0])))
            dk = int(rng.choice([4, 8, 16, 32, 20]))
            layers.append(R.latent_layer(heads=int(rng.integers(1, 9)), dim=dk, rot_dim=dr, vdim=int(rng.choice([4, 8, 12, 24, 48])), kv_rank=int(rng.choice([8, 16, 20, 48, 64, 100])),
                                         size=size, scale=float(rng.choice([(dk + dr) ** -0.5, 0.1, 0.25])), ff=ff, base=float(rng.choice([100.0, 10000.0, 1e6])), scaling=scaling))
    n = len(layers)
    start = int(rng.integers(0, n))
    stop = int(rng.integers(start + 1, n + 1))
    cfg = R.make_config(width, vocab, layers, loop=(start, stop, int(rng.integers(1, 4))), bigram=(int(rng.choice([1, 13, 401])), int(rng.integers(0, 40)), int(rng.integers(1, 40))),
                        eps=float(rng.choice([1e-6, 1e-5, 1e-3])), logit_scale=float(rng.choice([0.5, 1.0, 3.0])))
    return cfg, rng


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(backend, tmp_path, seed):
    """f32 serving of a random configuration: a whole prompt, then the same prompt in random portions beside a second request, its last tokens one by one"""
    cfg, rng = random_config(seed)
    W = R.random_weights(cfg, seed)
    R.save_model(cfg, W, str(tmp_path))
    n, n2 = int(rng.integers(60, 250)), int(rng.integers(5, 70))
    t, t2 = rng.integers(0, cfg["vocab"], n).tolist(), rng.integers(0, cfg["vocab"], n2).tolist()
    ref, ref2 = R.forward(cfg, W, t), R.forward(cfg, W, t2)
    s = TraceSession(str(tmp_path), "float32", max_tokens=512, n_ubatch=128, backend=backend)
    rows = s.step([{"id": "w", "tokens": t, "want": list(range(n))}], ["w"])
    assert row_err(rows, ref).max() <= F32_GATE
    got, got2, at, at2 = [], [], 0, 0
    while at < n - 10:
        c = min(int(rng.integers(1, 70)), n - 10 - at)
        ent = [{"id": "a", "tokens": t[at:at + c], "want": list(range(c))}]
        c2 = min(int(rng.integers(1, 20)), n2 - at2)
        if c2 > 0:
            ent.append({"id": "b", "tokens": t2[at2:at2 + c2], "want": list(range(c2))})
        r = s.step(ent, [])
        got.append(r[:c])
        if c2 > 0:
            got2.append(r[c:c + c2])
        at, at2 = at + c, at2 + max(c2, 0)
    while at < n:
        got.append(s.step([{"id": "a", "tokens": [t[at]], "want": [0]}], []))
        at += 1
    s.step([], ["a", "b"])
    assert row_err(np.concatenate(got), ref).max() <= F32_GATE
    if got2:
        assert row_err(np.concatenate(got2), ref2[:at2]).max() <= F32_GATE
    s.close()


@pytest.mark.parametrize("seed", range(4))
def test_random_configurations_bf16(backend, tmp_path, seed):
    cfg, rng = random_config(100 + seed)
    W = R.random_weights(cfg, seed)
    R.save_model(cfg, W, str(tmp_path))
    t = rng.integers(0, cfg["vocab"], 150).tolist()
    s = TraceSession(str(tmp_path), "bfloat16", max_tokens=512, n_ubatch=128, backend=backend)
    rows = np.concatenate([s.step([{"id": "w", "tokens": t[:100], "want": list(range(100))}], [])] + [s.step([{"id": "w", "tokens": [x], "want": [0]}], []) for x in t[100:]])
    assert row_err(rows, R.forward(cfg, W, t)).max() <= BF16_GATE
    s.close()
