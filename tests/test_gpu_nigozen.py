"""GPU tests of the Nigozen model class: the engine (llama_lite over the MI355X backend) against the plain numpy reference of
tests/nigozen_ref.py, on small models with their own sizes and random weights.

f32 serving is the sharp instrument: with 32-bit arithmetic end to end, ONE key wrongly seen or hidden among a few hundred moves a
logit row by ~1e-3 of its spread and more, ten times the gate (1e-4: the reference is float64, and an f32 rotation angle at position
150 is already 1e-5 rad from it).  bf16 serving is gated at its rounding level, on models whose routers keep EVERY expert: a 1 % error
upstream flips a near-tie between two router logits, another expert is another function, and the flipped token's keys and values
then reach the tokens behind it — which experts are chosen is settled by the f32 runs and by the bf16 expert block on its own.  Where
bf16's level would hide a fault (a far key, a sink, a chunk's edge) the inputs are made so that one score dominates."""
import ctypes as C
import json

import numpy as np
import pytest

import harness as T
import llama_box_amd as L
import nigozen_ref as R
from llama_box_amd.trace import TraceSession
from model_util import Context, Model

pytestmark = pytest.mark.gpu

F32_GATE, BF16_GATE = 1e-4, 5e-2


def row_err(got, ref):
    """per row: rms of the difference (means removed) over the rms of the reference row (mean removed)"""
    d = got - ref
    d = d - d.mean(axis=-1, keepdims=True)
    r = ref - ref.mean(axis=-1, keepdims=True)
    return np.sqrt((d * d).mean(axis=-1)) / np.sqrt((r * r).mean(axis=-1))


def check_rows(got, cfg, W, tokens, dtype):
    e = row_err(got, R.forward(cfg, W, tokens))
    gate = F32_GATE if dtype == "f32" else BF16_GATE
    assert e.max() <= gate, (int(np.argmax(e)), float(e.max()))
    return float(e.max())


def cfg_a(dtype="f32"):
    # chunk sizes 7, none and 16; 2 query heads per kv head, 3, and 2; key size != value size; one layer without a feed-forward; value mixing on
    # three of the four layers (the first of them is layer 0); a router that keeps one expert; rotary on a part, on all and on none of a head
    return R.make_config(64, 97, [
        dict(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=8, rot_base=100.0, scale=0.31, chunk=7, v_mix=True, mlp=("dense", 72)),
        dict(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=16, rot_base=5000.0, scale=0.2, chunk=0, v_mix=False, mlp=None),
        dict(heads=6, kv_heads=2, dim=8, vdim=24, rot_dims=4, rot_base=100.0, scale=0.45, chunk=16, v_mix=True, mlp=("moe", 24, 5, 2) if dtype == "f32" else ("moe", 24, 3, 3)),
        dict(heads=2, kv_heads=1, dim=40, vdim=48, rot_dims=0, scale=0.17, chunk=7, v_mix=True, mlp=("moe", 16, 3, 1) if dtype == "f32" else ("moe", 16, 1, 1)),
    ], eps=3e-5, embed_scale=1.7)


def cfg_b(dtype="f32"):
    # rows that are no multiple of 8 or 32 (width 52, cache rows of 36 and 20 values), head sizes above 128, value mixing that starts at layer 1, every expert used
    return R.make_config(52, 50, [
        dict(heads=3, kv_heads=3, dim=12, vdim=12, rot_dims=12, rot_base=10.0, scale=0.3, chunk=3, v_mix=False, mlp=("moe", 12, 2, 2)),
        dict(heads=2, kv_heads=1, dim=136, vdim=20, rot_dims=2, rot_base=50.0, scale=0.05, chunk=0, v_mix=True, mlp=("dense", 20)),
        dict(heads=1, kv_heads=1, dim=12, vdim=20, rot_dims=6, rot_base=50.0, scale=0.5, chunk=11, v_mix=True, mlp=("dense", 36)),
    ], eps=1e-6, embed_scale=0.25)


def cfg_c(dtype="f32"):
    # a single layer that does not rotate (no reader of the positions in the whole graph), rows of 36 values, an odd vocabulary
    return R.make_config(36, 257, [dict(heads=2, kv_heads=2, dim=8, vdim=32, rot_dims=0, scale=0.25, chunk=33, v_mix=True, mlp=("moe", 16, 5, 2) if dtype == "f32" else ("moe", 16, 2, 2))],
                         eps=1e-5, embed_scale=0.5)


CONFIGS = {"a": cfg_a, "b": cfg_b, "c": cfg_c}


class Served:
    def __init__(self, backend, tmp_path, cfg, seed, dtype, n_ctx=512, n_ubatch=64):
        self.cfg, self.W = cfg, R.random_weights(cfg, seed)
        R.write_model(str(tmp_path), cfg, self.W)
        self.model = Model(folder=str(tmp_path), buft=backend.buft, wtype=L.F32 if dtype == "f32" else L.BF16)
        self.ctx = Context(self.model, backend=backend, n_ctx=n_ctx, n_ubatch=n_ubatch, flash_attn=1)
        self.gate = F32_GATE if dtype == "f32" else BF16_GATE

    def ref(self, tokens):
        return R.forward(self.cfg, self.W, tokens)

    def free(self):
        self.ctx.free()
        self.model.free()


def toks(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("which", ["a", "b", "c"])
def test_whole_prompt(backend, tmp_path, plog, which, dtype):
    s = Served(backend, tmp_path, CONFIGS[which](dtype), 11, dtype)
    t = toks(150, s.cfg["vocab"], 5)  # three micro-batches of 64 / 64 / 22 tokens; every position's logits
    rc, lg = s.ctx.decode(t, range(len(t)))
    assert rc == 0
    e = check_rows(lg, s.cfg, s.W, t, dtype)
    plog(f"nigozen whole prompt cfg {which} {dtype}: max row error {e:.3e}")
    assert backend.stat("attn_f32_nodes") > 0
    s.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_prefill_against_token_by_token(backend, tmp_path, dtype):
    s = Served(backend, tmp_path, cfg_a(dtype), 12, dtype)
    t = toks(40, s.cfg["vocab"], 6)
    rows = []
    for p, tok in enumerate(t):  # the first tokens of a sequence one at a time: position 0 sees only itself and the sink
        rc, lg = s.ctx.decode([tok], [p])
        assert rc == 0
        rows.append(lg[0])
    check_rows(np.stack(rows), s.cfg, s.W, t, dtype)
    s.free()


@pytest.mark.parametrize("which", ["a", "b", "c"])
def test_portions_of_every_size(backend, tmp_path, which):
    s = Served(backend, tmp_path, CONFIGS[which](), 13, "f32")
    t = toks(131, s.cfg["vocab"], 7)
    ref = s.ref(t)
    cuts = [2, 3, 2, 7, 1, 16, 5, 2, 64, 2, 9, 18]  # down to two tokens; cuts fall inside chunks of 3, 7, 11 and 16 positions
    assert sum(cuts) == len(t)
    at, rows = 0, []
    for n in cuts:
        rc, lg = s.ctx.decode(t[at:at + n], range(at, at + n))
        assert rc == 0
        rows.append(lg)
        at += n
    assert row_err(np.concatenate(rows), ref).max() <= s.gate
    s.free()


def test_long_decoding_over_chunk_edges_and_cache_growth(backend, tmp_path):
    s = Served(backend, tmp_path, cfg_a(), 14, "f32", n_ctx=512)
    t = toks(300, s.cfg["vocab"], 8)  # 3 prompt tokens, then 297 single steps: the visible part of the cache grows past 256 cells, chunks of 7 and 16 roll over
    ref = s.ref(t)
    rc, lg = s.ctx.decode(t[:3], range(3))
    assert rc == 0
    rows = [lg]
    for p in range(3, len(t)):
        rc, lg = s.ctx.decode([t[p]], [p])
        assert rc == 0
        rows.append(lg)
    assert row_err(np.concatenate(rows), ref).max() <= s.gate
    s.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_unequal_requests_in_mixed_batches_with_cells_and_slots_used_again(backend, tmp_path, dtype):
    cfg = cfg_a(dtype)
    W = R.random_weights(cfg, 15)
    R.write_model(str(tmp_path), cfg, W)
    reqs = {name: toks(n, cfg["vocab"], 20 + i) for i, (name, n) in enumerate([("p", 190), ("q", 33), ("r", 1), ("s", 240), ("t", 57), ("u", 175)])}
    # 256 + 4 x 64 cells for 696 tokens in total: the cells of ended requests are handed out again, as are the four sequence slots
    sess = TraceSession(str(tmp_path), "float32" if dtype == "f32" else "bfloat16", max_tokens=256, n_ubatch=64, backend=backend)
    fed = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    plan = [  # (request, tokens) per step: portions beside single tokens, requests left out of steps, ends in between
        [("p", 40), ("q", 2)], [("p", 1), ("q", 30), ("r", 1)], [("p", 1), ("q", 1), ("s", 64)], [("p", 148), ("s", 3)], [("s", 173)],
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
        rows = sess.step(entries, ends)
        at = 0
        for name, n in step:
            got[name].append(rows[at:at + n])
            at += n
    for k in reqs:
        assert fed[k] == len(reqs[k])
        check_rows(np.concatenate(got[k]), cfg, W, reqs[k], dtype)
    sess.close()


def test_greedy_generation_through_the_engine(backend, tmp_path, H):
    s = Served(backend, tmp_path, cfg_a(), 16, "f32")
    prompt = toks(9, s.cfg["vocab"], 9)
    rc, _ = s.ctx.decode(prompt, range(len(prompt)), want=[0] * (len(prompt) - 1) + [1])
    assert rc == 0
    seq = list(prompt)
    for _ in range(24):
        tok = H.llm_sample_greedy(s.ctx.c, -1)  # the engine's own sampler on the engine's own logits
        ref_row = s.ref(seq)[-1]
        top2 = np.sort(ref_row)[-2:]
        if top2[1] - top2[0] > 1e-3 * np.abs(ref_row).max():
            assert tok == int(np.argmax(ref_row))
        else:
            tok = int(np.argmax(ref_row))
        seq.append(tok)
        rc, _ = s.ctx.decode([tok], [len(seq) - 1])
        assert rc == 0
    s.free()


# ------------------------------------------------------------------------------------------------ mechanisms alone, through the C-ABI
def run(backend, build):
    g = T.G(backend)
    outs = build(g)
    res = g.compute(outs if isinstance(outs, (list, tuple)) else [outs])
    g.free()
    return res


def bf16_bits(a):
    return (np.ascontiguousarray(R.bf16_round(a)).view(np.uint32) >> 16).astype(np.uint16)


def attention_case(backend, H, kv_type, n_q, n_kv, heads, kv_heads, dk, dv, chunk, sink, q, k, v, q_pos):
    """FLASH_ATTN_EXT over a cache of n_kv cells holding positions 0 .. n_kv - 1 of one sequence; queries at q_pos."""
    ok = R.visible(q_pos, np.arange(n_kv), chunk)
    mask = np.full((64 * ((n_q + 63) // 64), n_kv), -np.inf, np.float32)
    mask[:n_q][ok] = 0.0
    if kv_type == L.BF16:
        k, v = R.bf16_round(k), R.bf16_round(v)
        if n_q >= 32 and dk % 8 == 0 and dv % 8 == 0 and dk <= 128 and dv <= 128:
            q = R.bf16_round(q)  # prompt portions over a bf16 cache run on the matrix cores: the queries are rounded to bf16 like every mat-mul operand

    def build(g):
        tq = g.new(L.F32, [dk, heads, n_q], q)
        tk = g.new(kv_type, [dk * kv_heads, n_kv], bf16_bits(k) if kv_type == L.BF16 else k)
        tv = g.new(kv_type, [dv * kv_heads, n_kv], bf16_bits(v) if kv_type == L.BF16 else v)
        esz = 2 if kv_type == L.BF16 else 4
        kk = H.ggml_view_3d(g.ctx, tk, dk, n_kv, kv_heads, dk * kv_heads * esz, dk * esz, 0)
        vv = H.ggml_view_3d(g.ctx, tv, dv, n_kv, kv_heads, dv * kv_heads * esz, dv * esz, 0)
        r = H.ggml_flash_attn_ext(g.ctx, H.ggml_permute(g.ctx, tq, 0, 2, 1, 3), kk, vv, g.new(L.F32, [n_kv, mask.shape[0]], mask), 0.25, 0.0, 0.0)  # an F32 mask: the 32-bit kernel
        H.ggml_flash_attn_ext_set_prec(r, 10)
        if sink:
            H.ggml_flash_attn_ext_add_sinks(r, g.new(L.F32, [heads], np.zeros(heads, np.float32)))
        return r

    got = run(backend, build)[0].reshape(n_q, heads * dv)
    if sink:
        ref = R.attend(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), q_pos, np.arange(n_kv), 0.25, chunk)
    else:  # the same soft-max without the extra term
        ref = np.zeros((n_q, heads, dv))
        for h in range(heads):
            s = (q[:, h].astype(np.float64) @ k[:, h // (heads // kv_heads)].astype(np.float64).T) * 0.25
            s = np.where(ok, s, -np.inf)
            p = np.exp(s - s.max(axis=-1, keepdims=True))
            ref[:, h] = (p / p.sum(axis=-1, keepdims=True)) @ v[:, h // (heads // kv_heads)]
        ref = ref.reshape(n_q, -1)
    return got, ref


@pytest.mark.parametrize("kv_type", [L.F32, L.BF16])
@pytest.mark.parametrize("n_q,n_kv,heads,kv_heads,dk,dv,chunk,sink", [
    (1, 700, 4, 2, 64, 40, 0, True),      # one decoded token over 700 cells
    (1, 300, 6, 2, 24, 136, 64, True),    # value rows wider than 128
    (5, 200, 2, 2, 16, 16, 7, False),     # a few tokens, tiny chunks, the plain soft-max
    (70, 333, 4, 1, 64, 40, 50, True),    # a prompt portion (the tile form), chunk edges inside the portion
    (128, 640, 2, 2, 128, 128, 0, True),  # head size 128 both ways
    (33, 100, 3, 3, 40, 72, 9, False),
])
def test_attention_alone(backend, H, kv_type, n_q, n_kv, heads, kv_heads, dk, dv, chunk, sink):
    rng = np.random.default_rng(n_q * 1000 + n_kv)
    q = rng.standard_normal((n_q, heads, dk)).astype(np.float32)
    k = rng.standard_normal((n_kv, kv_heads, dk)).astype(np.float32)
    v = rng.standard_normal((n_kv, kv_heads, dv)).astype(np.float32)
    q_pos = np.arange(n_kv - n_q, n_kv)
    got, ref = attention_case(backend, H, kv_type, n_q, n_kv, heads, kv_heads, dk, dv, chunk, sink, q, k, v, q_pos)
    assert np.abs(got - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("n_q", [1, 40])
def test_a_far_key_a_chunk_edge_and_the_sink_show(backend, H, n_q):
    """bf16 cache, one key made to dominate: the output is that key's value row when the rule lets the query see it, and not when it lies one position
    outside the chunk; with every score far below zero the sink takes the weight and the output vanishes."""
    rng = np.random.default_rng(3)
    n_kv, heads, dk, dv, chunk = 600, 2, 32, 40, 250
    k = (0.05 * rng.standard_normal((n_kv, 1, dk))).astype(np.float32)
    v = rng.standard_normal((n_kv, 1, dv)).astype(np.float32)
    q = np.zeros((n_q, heads, dk), np.float32)
    q[:, :, 0] = 8.0
    q_pos = np.arange(n_kv - n_q, n_kv)
    first = int(q_pos[-1]) // chunk * chunk  # first position of the last query's chunk: 500
    for star, seen in ((first, True), (first - 1, False)):
        kk = k.copy()
        kk[star, 0, 0] = 16.0  # score 8 * 16 * 0.25 = 32 against ~0 elsewhere
        got, ref = attention_case(backend, H, L.BF16, n_q, n_kv, heads, 1, dk, dv, chunk, True, q, kk, v, q_pos)
        assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()
        hit = np.abs(got[-1, :dv] - R.bf16_round(v)[star, 0]).max()
        assert (hit < 1e-3) == seen
    got, ref = attention_case(backend, H, L.BF16, n_q, n_kv, heads, 1, dk, dv, chunk, True, -q, np.abs(k) + 4.0, v, q_pos)  # every score about -8
    assert np.abs(got).max() < 0.1 and np.abs(got - ref).max() <= 1e-5


def test_layer_norm_with_weight_and_residual(backend, H):
    rng = np.random.default_rng(5)
    for n, rows in ((52, 3), (256, 70), (4096, 2)):
        x = (rng.standard_normal((rows, n)) * 3 + 1.5).astype(np.float32)
        w = rng.standard_normal(n).astype(np.float32)
        r = rng.standard_normal((rows, n)).astype(np.float32)

        def build(g):
            t = H.ggml_mul(g.ctx, H.ggml_norm(g.ctx, g.new(L.F32, [n, rows], x), 1e-5), g.new(L.F32, [n], w))
            return [H.ggml_add(g.ctx, t, g.new(L.F32, [n, rows], r)), H.ggml_norm(g.ctx, g.new(L.F32, [n, rows], x), 1e-5)]

        got = run(backend, build)
        ref = R.layer_norm(x.astype(np.float64), w.astype(np.float64), 1e-5) + r
        assert np.abs(got[0].reshape(rows, n) - ref).max() <= 1e-5
        assert np.abs(got[1].reshape(rows, n) - R.layer_norm(x.astype(np.float64), 1.0, 1e-5)).max() <= 1e-5


def test_rotary_on_the_leading_pairs(backend, H):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((9, 3, 20)).astype(np.float32)
    pos = np.array([0, 1, 2, 3, 50, 51, 1000, 1001, 4095], np.int32)

    def build(g):
        return H.ggml_rope_ext(g.ctx, g.new(L.F32, [20, 3, 9], x), g.new(L.I32, [9], pos), None, 12, 0, 4096, 1000.0, 1.0, 0.0, 1.0, 32.0, 1.0)

    got = run(backend, build)[0].reshape(9, 3, 20)
    assert np.abs(got - R.rotate_pairs(x.astype(np.float64), pos, 12, 1000.0)).max() <= 2e-4  # (angles up to 4095 rad in f32)
    assert np.array_equal(got[:, :, 12:], x[:, :, 12:])


@pytest.mark.parametrize("wtype", [L.F32, L.BF16])
@pytest.mark.parametrize("K,N,M", [(52, 30, 1), (256, 192, 1), (256, 100, 7), (64, 97, 40), (320, 256, 150), (2048, 64, 3)])
def test_mat_mul_with_bf16_and_f32_matrices(backend, H, wtype, K, N, M):
    rng = np.random.default_rng(K + N + M)
    w = R.bf16_round(rng.standard_normal((N, K)).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float32)

    def build(g):
        return H.ggml_mul_mat(g.ctx, g.new(wtype, [K, N], bf16_bits(w) if wtype == L.BF16 else w), g.new(L.F32, [K, M], x))

    got = run(backend, build)[0].reshape(M, N)
    xr = R.bf16_round(x) if wtype == L.BF16 else x  # the activations are rounded to the matrix's type, the sum is 32-bit
    ref = xr.astype(np.float64) @ w.astype(np.float64).T
    assert np.abs(got - ref).max() <= 3e-5 * np.sqrt(K)


@pytest.mark.parametrize("wtype", [L.F32, L.BF16])
@pytest.mark.parametrize("T_,E,ff,n_exp,top", [(1, 64, 24, 5, 2), (3, 52, 12, 2, 2), (90, 64, 40, 6, 3), (200, 128, 64, 8, 1),
                                               (90, 36, 24, 5, 2),     # rows of 36 values: the up projection runs column by column, the down projection (24) grouped by expert
                                               (70, 64, 12, 3, 3)])    # ... and the other way round
def test_experts_router_and_weighted_sum(backend, H, wtype, T_, E, ff, n_exp, top):
    """the whole mixture-of-experts block as the engine builds it: router logits, the top entries, soft-max over them, squared-ReLU experts, the weighted sum"""
    rng = np.random.default_rng(T_ + E)
    Wn = {"mlp.router": R.bf16_round(rng.standard_normal((n_exp, E)).astype(np.float32))}
    for e in range(n_exp):
        Wn["mlp.e%d.up" % e] = R.bf16_round((rng.standard_normal((ff, E)) / np.sqrt(E)).astype(np.float32))
        Wn["mlp.e%d.down" % e] = R.bf16_round((rng.standard_normal((E, ff)) / np.sqrt(ff)).astype(np.float32))
    h = R.bf16_round(rng.standard_normal((T_, E)).astype(np.float32))
    conv = (lambda a: bf16_bits(a)) if wtype == L.BF16 else (lambda a: a)

    def build(g):
        cur = g.new(L.F32, [E, T_], h)
        ups = g.new(wtype, [E, ff, n_exp], conv(np.stack([Wn["mlp.e%d.up" % e] for e in range(n_exp)])))
        downs = g.new(wtype, [ff, E, n_exp], conv(np.stack([Wn["mlp.e%d.down" % e] for e in range(n_exp)])))
        logits = H.ggml_mul_mat(g.ctx, g.new(L.F32, [E, n_exp], Wn["mlp.router"]), cur)
        sel = H.ggml_top_k(g.ctx, logits, top)
        w = H.ggml_get_rows(g.ctx, H.ggml_reshape_3d(g.ctx, logits, 1, n_exp, T_), sel)
        w = H.ggml_soft_max(g.ctx, H.ggml_reshape_2d(g.ctx, w, top, T_))
        up = H.ggml_mul_mat_id(g.ctx, ups, H.ggml_reshape_3d(g.ctx, cur, E, 1, T_), sel)
        act = H.ggml_sqr(g.ctx, H.ggml_unary(g.ctx, up, 6))  # GGML_UNARY_OP_RELU
        down = H.ggml_mul(g.ctx, H.ggml_mul_mat_id(g.ctx, downs, act, sel), H.ggml_reshape_3d(g.ctx, w, 1, top, T_))
        return [down, H.ggml_cont(g.ctx, sel)]

    down, sel = run(backend, build)
    got = down.reshape(T_, top, E).sum(axis=1)
    idx, _ = R.route(h.astype(np.float64), Wn["mlp.router"].astype(np.float64), top)
    assert np.array_equal(sel.reshape(T_, top), idx)
    ref = R.moe_ffn(h.astype(np.float64), {k: a.astype(np.float64) for k, a in Wn.items()}, "", {"router": {"top": top}})
    tol = 2e-5 if wtype == L.F32 else 2e-2  # (bf16: the expert's hidden activations are rounded to bf16 on their way into the down projection)
    assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max())


def test_erf_gelu_and_squared_relu(backend, H):
    x = np.linspace(-6, 6, 1001).astype(np.float32)

    def build(g):
        t = g.new(L.F32, [1001], x)
        return [H.ggml_unary(g.ctx, t, 14), H.ggml_sqr(g.ctx, H.ggml_unary(g.ctx, t, 6))]  # GELU_ERF; RELU then SQR

    ge, rs = run(backend, build)
    assert np.abs(ge.reshape(-1) - R.gelu_erf(x.astype(np.float64))).max() <= 1e-6
    assert np.abs(rs.reshape(-1) - np.maximum(x.astype(np.float64), 0) ** 2).max() <= 1e-5


def test_trace_run_command_line(tmp_path):
    """bin/trace_run as a program: steps on standard input, one 'done <step>' line each, <step>.f32 only where logits were asked for"""
    import os
    import subprocess
    import sys

    cfg = cfg_b()
    W = R.random_weights(cfg, 31)
    model_dir, out_dir = str(tmp_path / "model"), str(tmp_path / "out")
    R.write_model(model_dir, cfg, W)
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
    """a configuration drawn at random: widths with and without whole groups of 8 values, 1 - 6 layers, every chunk / rotary / feed-forward combination, value rows of one
    total width (what value mixing needs) split over 1 - 8 key/value heads"""
    rng = np.random.default_rng(seed)
    width = int(rng.choice([32, 48, 64, 72, 96, 100, 128, 160, 36]))
    vocab = int(rng.integers(40, 300))
    kvd = int(rng.choice([24, 48, 96, 64, 40]))
    layers = []
    for _ in range(int(rng.integers(1, 7))):
        opts = [(g, kvd // g) for g in (1, 2, 3, 4, 6, 8) if kvd % g == 0 and kvd // g >= 4]
        G, dv = opts[int(rng.integers(len(opts)))]
        H = G * int(rng.choice([1, 1, 2, 3, 4]))
        dk = int(rng.choice([8, 12, 16, 24, 32, 40, 64, 96, 128, 20]))
        rot = min(int(rng.choice([0, 2, 4, dk, 8])), dk) // 2 * 2
        chunk = int(rng.choice([0, 3, 5, 16, 33, 64, 100, 257]))
        kind = int(rng.integers(0, 4))
        if kind == 0:
            mlp = None
        elif kind == 1:
            mlp = ("dense", int(rng.choice([16, 40, 64, 100, 256])))
        else:
            ne = int(rng.integers(1, 9))
            mlp = ("moe", int(rng.choice([8, 16, 24, 64])), ne, int(rng.integers(1, ne + 1)))
        layers.append(dict(heads=H, kv_heads=G, dim=dk, vdim=dv, rot_dims=rot, rot_base=float(rng.choice([100.0, 10000.0, 1e6])), scale=float(rng.choice([dk ** -0.5, 0.1, 0.25])),
                           chunk=chunk, v_mix=bool(rng.integers(0, 2)), mlp=mlp))
    cfg = R.make_config(width, vocab, layers, eps=float(rng.choice([1e-6, 1e-5, 1e-3])), embed_scale=float(rng.choice([0.5, 1.0, 3.0])))
    return cfg, rng


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations(backend, tmp_path, seed):
    """f32 serving of a random configuration: a whole prompt, then the same prompt in random portions beside a second request, its last tokens one by one"""
    cfg, rng = random_config(seed)
    W = R.random_weights(cfg, seed)
    R.write_model(str(tmp_path), cfg, W)
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
