"""Host side of the Nigozen model class, without a GPU: the checkpoint-folder loader (config.json + safetensors), what it refuses, the graph
the engine builds for it, and the attention masks it uploads — checked against the plain reference's visibility rule."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import llama_box_amd as L
import nigozen_ref as R


def small_cfg():
    return R.make_config(48, 61, [
        dict(heads=4, kv_heads=2, dim=8, vdim=12, rot_dims=4, scale=0.3, chunk=5, v_mix=True, mlp=("dense", 40)),
        dict(heads=2, kv_heads=2, dim=16, vdim=12, rot_dims=16, scale=0.2, chunk=0, v_mix=False, mlp=None),
        dict(heads=6, kv_heads=1, dim=8, vdim=24, rot_dims=0, scale=0.4, chunk=9, v_mix=True, mlp=("moe", 16, 5, 2)),
    ], eps=1e-5, embed_scale=0.7)


def test_loader_reads_a_checkpoint_folder(H, tmp_path):
    cfg = small_cfg()
    W = R.random_weights(cfg, 3)
    R.write_model(str(tmp_path), cfg, W)
    for wtype, esz in ((L.BF16, 2), (L.F32, 4)):
        m = H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), wtype)
        assert m
        hp = H.llm_model_hparams(m).contents
        assert (hp.arch, hp.n_layer, hp.n_embd, hp.n_vocab) == (b"nigozen", 3, 48, 61)
        t = H.llm_model_tensor(m, b"blk.0.attn_q.weight").contents
        assert (t.type, t.ne[0], t.ne[1]) == (wtype, 48, 32)
        raw = np.empty(48 * 32 * esz, np.uint8)
        H.ggml_backend_tensor_get(H.llm_model_tensor(m, b"blk.0.attn_q.weight"), raw.ctypes.data_as(C.c_void_p), 0, raw.nbytes)
        got = raw.view(np.float32) if wtype == L.F32 else (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
        assert np.array_equal(got.reshape(32, 48), W["l0.mix.q"])
        # the experts of a layer are stacked: [in, ff, expert]; routers and norm weights stay f32
        e = H.llm_model_tensor(m, b"blk.2.ffn_up_exps.weight").contents
        assert (e.ne[0], e.ne[1], e.ne[2]) == (48, 16, 5)
        assert H.llm_model_tensor(m, b"blk.2.ffn_gate_inp.weight").contents.type == L.F32
        assert H.llm_model_tensor(m, b"blk.1.attn_post_norm.weight").contents.type == L.F32
        assert not H.llm_model_tensor(m, b"blk.1.ffn_up.weight")  # a layer without a feed-forward has none
        H.llm_model_free(m)


@pytest.mark.parametrize("breakage", ["arch", "shape", "missing", "heads", "top", "json"])
def test_loader_refuses_what_it_cannot_serve(H, tmp_path, breakage):
    cfg = small_cfg()
    W = R.random_weights(cfg, 4)
    if breakage == "arch":
        cfg["architecture"] = "SomethingElse"
    elif breakage == "shape":
        W["l0.mix.k"] = W["l0.mix.k"][:, :-8]
    elif breakage == "missing":
        del W["l2.mlp.e3.down"]
    elif breakage == "heads":
        cfg["layers"][0]["mixer"]["kv_heads"] = 3
    elif breakage == "top":
        cfg["layers"][2]["mlp"]["router"]["top"] = 9
    R.write_model(str(tmp_path), cfg, W)
    if breakage == "json":
        with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
            f.write("{\"architecture\": \"Nigozen\", ")
    assert not H.llm_model_load_dir(str(tmp_path).encode(), H.ggml_backend_cpu_buffer_type(), L.BF16)


def _graph_probe(H, m, n_ctx, steps):
    """Runs llm_decode with a compute callback that records the op counts and the masks the engine filled (host memory here)."""
    seen = []

    def comp(g, _n):
        gg = g.contents
        ops, masks = {}, {}
        for i in range(gg.n_nodes):
            t = gg.nodes[i].contents
            name = H.ggml_op_name(t.op).decode()
            ops[name] = ops.get(name, 0) + 1
            for s in range(4):
                if t.src[s] and t.src[s].contents.name.startswith(b"KQ_mask"):
                    mt = t.src[s].contents
                    arr = np.ctypeslib.as_array(C.cast(mt.data, C.POINTER(C.c_float)), shape=(mt.ne[1], mt.ne[0])).copy()
                    masks[mt.name.decode()] = arr
        seen.append((ops, masks))
        return 0

    fn = L.COMPUTE_FN(comp)
    cp = L.ContextParams(n_ctx, 64, 1, 0, 1, 0, 0)
    c = H.llm_context_new(m, None, fn, C.byref(cp))
    assert c
    for toks, pos, seq in steps:
        n = len(toks)
        rc = H.llm_decode(c, n, (C.c_int32 * n)(*toks), (C.c_int32 * n)(*pos), (C.c_int32 * n)(*seq), None)
        assert rc == 0
    H.llm_context_free(c)
    return seen


def test_graph_and_masks_of_a_mixed_batch(H):
    cfg = small_cfg()
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 7, H.ggml_backend_cpu_buffer_type(), L.BF16)
    assert m
    # sequence 0: positions 0..11 as one portion, then sequence 1 (0..6) beside three more tokens of sequence 0
    steps = [([1] * 12, list(range(12)), [0] * 12),
             ([2] * 7 + [3] * 3, list(range(7)) + [12, 13, 14], [1] * 7 + [0] * 3)]
    seen = _graph_probe(H, m, 256, steps)
    ops, masks = seen[-1]
    assert ops["FLASH_ATTN_EXT"] == 3 and ops["NORM"] == 3 * 2 + 2 * 2 + 1 and ops["MUL_MAT_ID"] == 2 and ops["ARGSORT"] == 1
    assert len(masks) == 3  # chunk sizes 5, 0 and 9: one mask each
    # cells are handed out in order: cell j holds (seq, pos) of the j-th token fed
    cell_seq = np.array([0] * 12 + [1] * 7 + [0] * 3)
    cell_pos = np.array(list(range(12)) + list(range(7)) + [12, 13, 14])
    q_seq, q_pos = np.array(steps[1][2]), np.array(steps[1][1])
    by_chunk = {}
    for name, arr in masks.items():
        vis = np.isfinite(arr[: len(q_pos), : len(cell_pos)])
        assert not np.isfinite(arr[: len(q_pos), len(cell_pos):]).any()  # empty cells are never visible
        for chunk in (5, 0, 9):
            want = R.visible(q_pos, cell_pos, chunk) & (q_seq[:, None] == cell_seq[None, :])
            if np.array_equal(vis, want):
                by_chunk[chunk] = name
    assert sorted(by_chunk) == [0, 5, 9]
    H.llm_model_free(m)


def test_reference_attention_edges():
    """The plain reference itself: the sink takes weight, a chunk's edge lies where the rule floor(i / size) == floor(j / size) puts it."""
    ok = R.visible([4, 5, 9, 10], np.arange(12), 5)
    assert ok[0].nonzero()[0].tolist() == [0, 1, 2, 3, 4] and ok[1].nonzero()[0].tolist() == [5]
    assert ok[2].nonzero()[0].tolist() == [5, 6, 7, 8, 9] and ok[3].nonzero()[0].tolist() == [10]
    p = R.sink_softmax(np.array([[0.0, 0.0, 0.0]]), np.array([[True, True, False]]))
    assert np.allclose(p, [[1 / 3, 1 / 3, 0.0]])
    x = R.rotate_pairs(np.ones((1, 1, 6)), [3], 4, 100.0)
    assert np.allclose(x[0, 0, 4:], 1.0) and np.allclose(x[0, 0, 0], np.cos(3) - np.sin(3)) and np.allclose(x[0, 0, 3], np.cos(0.3) + np.sin(0.3))


def test_a_model_without_rotary_layers_has_no_position_input(H):
    """no layer rotates -> nothing reads the positions: the engine must not upload into an input the graph allocator never placed"""
    cfg = R.make_config(36, 57, [dict(heads=2, kv_heads=2, dim=8, vdim=32, rot_dims=0, scale=0.25, chunk=33, v_mix=True, mlp=("moe", 16, 5, 2))])
    m = H.llm_model_synth_config(json.dumps(cfg).encode(), 1, H.ggml_backend_cpu_buffer_type(), L.BF16)
    assert m
    seen = _graph_probe(H, m, 256, [([1, 2, 3, 4, 5], [0, 1, 2, 3, 4], [0] * 5), ([6], [5], [0])])
    assert len(seen) == 2 and "ROPE" not in seen[0][0]
    H.llm_model_free(m)
