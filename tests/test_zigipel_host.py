"""Host side of the Zigipel model class, without a GPU: the loader (config.json + safetensors: per-head transposed expansion matrices, the
penalty pairs, the table of rotation frequencies), what it refuses, the order of layer runs, and what the scheduler uploads for a mixed
batch — window masks with kept first positions and distances, bigram rows, token-shift sources — checked against the plain reference."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import llama_box_amd as L
import zigipel_ref as R


def small_cfg():
    return R.make_config(40, 53, [
        R.latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, size=5, scale=0.3, ff=24, base=100.0, scaling=(4.0, 16, 8.0, 1.0)),
        R.attention_layer(heads=4, kv_heads=2, dim=8, vdim=12, size=6, keep_first=2, scale=0.25, ff=None),
        R.attention_layer(heads=2, kv_heads=1, dim=16, vdim=8, size=3, keep_first=0, scale=0.2, ff=32),
    ], loop=(1, 3, 3), bigram=(11, 7, 3), eps=1e-5, logit_scale=0.7)


def _get(H, m, name, dtype=np.float32):
    t = H.llm_model_tensor(m, name.encode())
    assert t, name
    raw = np.empty(H.ggml_nbytes(t), np.uint8)
    H.ggml_backend_tensor_get(t, raw.ctypes.data_as(C.c_void_p), 0, raw.nbytes)
    tt = t.contents
    if tt.type == L.BF16:
        a = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    else:
        a = raw.view(dtype)
    return a.reshape([tt.ne[3], tt.ne[2], tt.ne[1], tt.ne[0]])[0]


def test_loader_reads_a_checkpoint_folder(H, tmp_path):
    cfg = small_cfg()
    W = R.random_weights(cfg, 3)
    R.save_model(cfg, W, str(tmp_path))
    for wtype in (L.BF16, L.F32):
        m = H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), wtype)
        assert m
        hp = H.llm_model_hparams(m).contents
        assert (hp.arch, hp.n_layer, hp.n_embd, hp.n_vocab) == (b"zigipel", 3, 40, 53)
        assert np.array_equal(_get(H, m, "blk.0.attn_q.weight")[0], W["l0.mix.q"])
        # W_uk is kept per head with its ROWS along dim 0: [dk, rank, head]
        uk = _get(H, m, "blk.0.attn_k_b_t.weight")  # [head][rank][dk]
        assert uk.shape == (3, 20, 8)
        assert np.array_equal(uk, W["l0.mix.uk"].reshape(3, 8, 20).transpose(0, 2, 1))
        uv = _get(H, m, "blk.0.attn_v_b.weight")    # [head][dv][rank]
        assert np.array_equal(uv, W["l0.mix.uv"].reshape(3, 12, 20))
        r12 = _get(H, m, "blk.1.attn_dist.weight")  # r1 of every head, then r2 of every head
        assert np.array_equal(r12.reshape(2, 4), np.stack([W["l1.mix.r1"], W["l1.mix.r2"]]))
        freq, mag = R.yarn_frequencies(4, 100.0, cfg["layers"][0]["mixer"]["rot"]["scaling"])
        assert np.allclose(_get(H, m, "blk.0.rope_freq.weight").reshape(-1), freq, rtol=1e-6, atol=0)
        assert _get(H, m, "bigram_embd.weight")[0].shape == (12, 40) and _get(H, m, "loop_in.weight")[0].shape == (40, 80)
        assert H.llm_model_tensor(m, b"blk.1.shift.weight").contents.type == L.F32
        assert not H.llm_model_tensor(m, b"blk.1.ffn_up.weight")  # a layer without a feed-forward has none
        H.llm_model_free(m)


@pytest.mark.parametrize("breakage", ["shape", "missing", "heads", "loop", "mixer", "kind"])
def test_loader_refuses_what_it_cannot_serve(H, tmp_path, breakage):
    cfg = small_cfg()
    W = R.random_weights(cfg, 4)
    if breakage == "shape":
        W["l0.mix.uk"] = W["l0.mix.uk"][:, :-4]
    elif breakage == "missing":
        del W["l1.mix.sink"]
    elif breakage == "heads":
        cfg["layers"][1]["mixer"]["kv_heads"] = 3
    elif breakage == "loop":
        cfg["loop"]["stop"] = 7
    elif breakage == "mixer":
        cfg["layers"][2]["type"] = "something_else"
    elif breakage == "kind":
        cfg["layers"][2]["mlp"]["kind"] = "moe"
    R.save_model(cfg, W, str(tmp_path))
    assert not H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), L.BF16)


def test_reference_pieces():
    """The plain reference itself at places where a slip would not show in random data."""
    ok = R.window_visible(8, 3, 2)
    assert ok[7].nonzero()[0].tolist() == [0, 1, 5, 6, 7] and ok[2].nonzero()[0].tolist() == [0, 1, 2] and ok[4].nonzero()[0].tolist() == [0, 1, 2, 3, 4]
    assert R.window_visible(8, 3)[7].nonzero()[0].tolist() == [5, 6, 7]
    p = R.sink_softmax(np.array([[0.0, 0.0, 5.0]]), np.array([[True, True, False]]), 0.0)
    assert np.allclose(p, [[1 / 3, 1 / 3, 0.0]])
    assert R.bigram_rows([4, 9, 9], 11, 7, 3).tolist() == [11, (4 * 7 + 9 * 3) % 11, (9 * 7 + 9 * 3) % 11]
    h = np.arange(6.0).reshape(3, 2)
    assert np.allclose(R.token_shift(h, np.array([1.0, 0.5])), [[0, 0.5], [0, 2], [2, 4]])
    x = R.rotate_half(np.ones((1, 1, 6)), [3], np.array([1.0, 0.1]), 2.0)  # pairs (0, 2) and (1, 3); entries 4, 5 pass
    assert np.allclose(x[0, 0], [2 * (np.cos(3) - np.sin(3)), 2 * (np.cos(0.3) - np.sin(0.3)), 2 * (np.cos(3) + np.sin(3)), 2 * (np.cos(0.3) + np.sin(0.3)), 1, 1])
    f, mag = R.yarn_frequencies(8, 10000.0, dict(factor=4.0, original=64, fast=4.0, slow=1.0))
    plain = np.array([10000.0 ** (-2 * i / 8) for i in range(4)])
    assert np.isclose(f[0], plain[0]) and np.isclose(f[3], plain[3] / 4) and np.isclose(mag, 0.1 * np.log(4.0) + 1)
    assert [r[0] for r in R.layer_runs(small_cfg())] == [0, 1, 2, 1, 2, 1, 2]


def _probe(H, m, n_ctx, steps, n_ubatch=64):
    """llm_decode with a compute callback that records op counts and the named inputs the engine filled (host memory here)."""
    seen = []
    want = (b"KQ_mask", b"inp_bigram_rows", b"shift_src", b"shift_last_rows", b"shift_slots", b"k_idxs")

    def comp(g, _n):
        gg = g.contents
        ops, inputs = {}, {}
        for i in range(gg.n_nodes):
            t = gg.nodes[i].contents
            name = H.ggml_op_name(t.op).decode()
            ops[name] = ops.get(name, 0) + 1
            for s in range(6):
                if t.src[s] and t.src[s].contents.name.startswith(want):
                    mt = t.src[s].contents
                    ct = {L.F32: C.c_float, L.I32: C.c_int32, L.I64: C.c_int64}[mt.type]
                    inputs[mt.name.decode()] = np.ctypeslib.as_array(C.cast(mt.data, C.POINTER(ct)), shape=(mt.ne[1], mt.ne[0])).copy()
        seen.append((ops, inputs))
        return 0

    fn = L.COMPUTE_FN(comp)
    cp = L.ContextParams(n_ctx, n_ubatch, 1, 0, 1, 0, 0, 4)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    assert c
    for toks, pos, seq in steps:
        n = len(toks)
        rc = H.llm_decode(c, n, (C.c_int32 * n)(*toks), (C.c_int32 * n)(*pos), (C.c_int32 * n)(*seq), None)
        assert rc == 0
        if toks == "free":
            pass
    H.llm_context_free(c)
    return seen


def test_scheduler_inputs_of_a_mixed_batch(H):
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 7, H.ggml_backend_cpu_buffer_type(), L.BF16)
    assert m
    # sequence 2: positions 0..9 as one portion; then sequence 0 (0..6) beside three more tokens of sequence 2, interleaved
    s1 = ([5, 6, 7, 8, 9, 10, 11, 12, 13, 14], list(range(10)), [2] * 10)
    toks2 = [20, 21, 30, 22, 23, 31, 24, 25, 26, 32]
    seq2 = [0, 0, 2, 0, 0, 2, 0, 0, 0, 2]
    pos2 = [0, 1, 10, 2, 3, 11, 4, 5, 6, 12]
    seen = _probe(H, m, 256, [s1, (toks2, pos2, seq2)])
    ops, inp = seen[-1]
    assert ops["FLASH_ATTN_EXT"] == 7 and ops["CONCAT"] >= 7 + 3 and ops["SET_ROWS"] == 7 * 2 + 6  # 7 layer runs: token-shift state + caches (one row for latent, two for attention)
    # cells are handed out in order: cell j holds (seq, pos) of the j-th token fed
    cell_seq = np.array(s1[2] + seq2)
    cell_pos = np.array(s1[1] + pos2)
    qs, qp = np.array(seq2), np.array(pos2)
    rules = {(5, 0, False): None, (6, 2, True): None, (3, 0, True): None}
    masks = {k: v for k, v in inp.items() if k.startswith("KQ_mask")}
    assert len(masks) == 3
    for name, arr in masks.items():
        a = arr[: len(qp), : len(cell_pos)]
        assert not np.isfinite(arr[: len(qp), len(cell_pos):]).any()  # empty cells are never visible
        for (size, keep, dist) in rules:
            d = qp[:, None] - cell_pos[None, :]
            vis = (qs[:, None] == cell_seq[None, :]) & (d >= 0) & ((d < size) | (cell_pos[None, :] < keep))
            if np.array_equal(np.isfinite(a), vis) and np.array_equal(a[vis], (d[vis] if dist else 0 * d[vis]).astype(np.float32)):
                rules[(size, keep, dist)] = name
    assert all(rules.values()) and len(set(rules.values())) == 3
    # bigram rows: the hash of (previous, current) with the previous token taken from the batch or from the sequence's last call; row `buckets` at position 0
    prev = {0: None, 2: 14}
    want_rows = []
    for t, s, p in zip(toks2, seq2, pos2):
        want_rows.append(11 if p == 0 else (prev[s] * 7 + t * 3) % 11)
        prev[s] = t
    assert inp["inp_bigram_rows"].reshape(-1).tolist() == want_rows
    # token-shift sources: the row before in the batch, else the sequence's state row (T + slot), else the zero row (T + slots)
    T_, S_ = len(toks2), 4
    assert inp["shift_src"].reshape(-1).tolist() == [T_ + S_, 0, T_ + 2, 1, 3, 2, 4, 6, 7, 5]
    assert inp["shift_last_rows"].reshape(-1).tolist() == [8, 9] and inp["shift_slots"].reshape(-1).tolist() == [0, 2]
    H.llm_model_free(m)


def test_micro_batches_carry_the_state(H):
    """a prompt cut into micro-batches by the engine: the first token of the second micro-batch reads its sequence's state row and hashes with the last token before"""
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 9, H.ggml_backend_cpu_buffer_type(), L.F32)
    toks = list(range(1, 12))
    seen = _probe(H, m, 256, [(toks, list(range(11)), [1] * 11)], n_ubatch=8)
    assert len(seen) == 2
    second = seen[1][1]
    assert second["shift_src"].reshape(-1).tolist() == [3 + 1, 0, 1] and second["inp_bigram_rows"].reshape(-1)[0] == (8 * 7 + 9 * 3) % 11
    assert second["shift_slots"].reshape(-1).tolist() == [1]
    H.llm_model_free(m)


def test_sequence_ids_beyond_the_state_rows_are_refused(H):
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 9, H.ggml_backend_cpu_buffer_type(), L.F32)
    fn = L.COMPUTE_FN(lambda g, n: 0)
    cp = L.ContextParams(256, 64, 1, 0, 1, 0, 0, 2)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    one = (C.c_int32 * 1)
    assert H.llm_decode(c, 1, one(3), one(0), one(1), None) == 0
    assert H.llm_decode(c, 1, one(3), one(0), one(2), None) == -1
    H.llm_context_free(c)
    H.llm_model_free(m)
