"""Replays a trace of token ids through a model: requests arrive in portions, several per step, and the logits at chosen places come back.

Nothing here computes: a step is ONE llm_decode batch of the engine (llama_lite: unified cache of cells, micro-batching, graph per
micro-batch on the MI355X backend).  A request takes one of the engine's sequence slots at its first portion and gives the slot and
its cache cells back when it ends, so cells and slots are used again by later requests.

    session = TraceSession(model_dir, dtype="bfloat16", max_tokens=2048)
    rows = session.step([{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], end=[])   # -> float32 array [wanted, vocab]
"""
import ctypes as C
import json
import os
import sys

import numpy as np

import llama_box_amd as L

N_SLOTS = 4  # sequence slots of a session (live requests)


class TraceSession:
    def __init__(self, model_dir, dtype="bfloat16", max_tokens=4096, n_ubatch=512, backend=None):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError("dtype is bfloat16 or float32")
        self.H = L.host()
        self.backend = backend if backend is not None else L.Backend(0)  # raises without a gfx950 device: there is no CPU path
        self._own_backend = backend is None
        wtype = L.BF16 if dtype == "bfloat16" else L.F32
        self.model = self.H.llm_model_load_dir(os.fsencode(model_dir), self.backend.buft, wtype)
        if not self.model:
            raise RuntimeError("model could not be loaded from %s" % model_dir)
        self.n_vocab = self.H.llm_model_hparams(self.model).contents.n_vocab
        # every live request may hold a last, partly filled group of 64 cells beyond what it asked for
        n_ctx = int(max_tokens) + 64 * N_SLOTS
        cp = L.ContextParams(n_ctx, n_ubatch, 1, 0, 1, 0, 0, N_SLOTS)
        self.ctx = self.H.llm_context_new(self.model, self.backend.backend, L.COMPUTE_FN(), C.byref(cp))
        if not self.ctx:
            raise RuntimeError("context creation failed")
        self.slot_of = {}   # request id -> sequence slot
        self.n_past = {}    # request id -> tokens already in the cache
        self.free_slots = list(range(N_SLOTS))

    def step(self, entries, end=()):
        tokens, pos, seq, want = [], [], [], []
        for e in entries:
            rid = e["id"]
            if rid not in self.slot_of:
                if not self.free_slots:
                    raise RuntimeError("more than %d live requests" % N_SLOTS)
                self.slot_of[rid] = self.free_slots.pop(0)
                self.n_past[rid] = 0
            toks = e["tokens"]
            flags = [0] * len(toks)
            for w in e.get("want", ()):
                flags[w] = 1
            base = self.n_past[rid]
            tokens += toks
            pos += range(base, base + len(toks))
            seq += [self.slot_of[rid]] * len(toks)
            want += flags
            self.n_past[rid] = base + len(toks)
        rows = np.zeros((0, self.n_vocab), dtype=np.float32)
        if tokens:
            n = len(tokens)
            rc = self.H.llm_decode(self.ctx, n, (C.c_int32 * n)(*tokens), (C.c_int32 * n)(*pos), (C.c_int32 * n)(*seq), (C.c_int8 * n)(*want))
            if rc != 0:
                raise RuntimeError("llm_decode failed with code %d" % rc)
            no = self.H.llm_n_outputs(self.ctx)
            if no:
                rows = np.ctypeslib.as_array(self.H.llm_get_logits(self.ctx), shape=(no, self.n_vocab)).astype(np.float32, copy=True)
        for rid in end:
            if rid in self.slot_of:
                slot = self.slot_of.pop(rid)
                self.H.llm_kv_seq_rm(self.ctx, slot, -1, -1)  # its cells are free again
                self.free_slots.append(slot)
                del self.n_past[rid]
        return rows

    def close(self):
        if self.ctx:
            self.H.llm_context_free(self.ctx)
            self.ctx = None
        if self.model:
            self.H.llm_model_free(self.model)
            self.model = None
        if self._own_backend and self.backend:
            self.backend.close()
            self.backend = None


def main(argv=None):
    import argparse

    ap = argparse.ArgumentParser(prog="trace_run", description="feed token ids through a model step by step and write the logits asked for")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, default=4096, help="cache cells for the live requests together")
    a = ap.parse_args(argv)
    if not (os.path.exists(L.BACKEND_SO) and os.path.exists(L.HOST_SO)):
        L.build()  # a fresh checkout: the first call compiles the two libraries
    os.makedirs(a.out, exist_ok=True)
    s = TraceSession(a.model, a.dtype, a.max_tokens)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        rows = s.step(st.get("entries", []), st.get("end", []))
        if rows.shape[0]:
            rows.astype("<f4").tofile(os.path.join(a.out, "%d.f32" % st["step"]))
        sys.stdout.write("done %d\n" % st["step"])
        sys.stdout.flush()
    s.close()
    return 0
