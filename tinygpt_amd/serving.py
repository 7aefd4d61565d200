"""Slot scheduler for layered models: requests come and go, the engine steps a ragged batch.

`SlotEngine` owns one `Model` built from a model directory.  A request is admitted to a free sequence slot by its first step, may
sit out steps, and gives its slot and its pages of the latent pool back when it ends; slots and pages are used again by later
requests.  `step()` is the engine step every caller shares (the trace replay of bin/trace_run, `generate()` below, tools that
drive continuous batching): portions of prompts ride beside single decoded tokens in one pass.

The reference's engine rebuilds a fixed batch per call (src/engine/GPTEngine.cpp:154-174) and lists continuous batching as a
TODO (README.md:33-34); this is that scheduler for the families whose step takes ragged batches.
"""
from __future__ import annotations

import json
import os

import numpy as np

from .desc import load_desc, StackDesc
from .ffi import GREEDY, Model, SamplerCfg, TgxError


class SlotEngine:
    def __init__(self, model_dir: str = None, dtype: str = "bf16", max_seqs: int = 4, max_tokens: int = 0, max_ctx: int = 0, device: int = 0,
                 desc: StackDesc = None, tensors=None, backend=None):
        """model_dir: config.json + model.safetensors (or desc + tensors: an in-memory checkpoint).  max_tokens: tokens of the shared cache
        pool, rounded up to whole pages per live request by the caller; max_ctx: longest sequence of a slot (default: the pool)."""
        if desc is None:
            desc = load_desc(model_dir, dtype, max_seqs, max_ctx=max_ctx or max(max_tokens, 64), budget_tokens=max_tokens)
        if not isinstance(desc, StackDesc):
            raise ValueError("SlotEngine serves layered models; the flat families step through Model.forward_row / Model.decode")
        self.desc = desc
        self.model = Model(desc, backend, device)
        if tensors is not None:
            self.model.load_state(tensors, strict=True)
        else:
            self.model.load_dir(model_dir, strict=False)
        self.model.finalize()
        self.slot_of = {}                                # request id -> slot
        self.free = list(range(desc.max_seqs - 1, -1, -1))

    # -- lifecycle -----------------------------------------------------------------------------------------------------------
    def admit(self, rid) -> int:
        if rid not in self.slot_of:
            if not self.free:
                raise RuntimeError(f"no free sequence slot for request {rid!r} ({self.desc.max_seqs} slots)")
            self.slot_of[rid] = self.free.pop()
        return self.slot_of[rid]

    def release(self, rid):
        slot = self.slot_of.pop(rid, None)
        if slot is not None:
            self.model.reset_row(slot)
            self.free.append(slot)

    def length(self, rid) -> int:
        return self.model.past_length_row(self.slot_of[rid]) if rid in self.slot_of else 0

    @property
    def free_tokens(self) -> int:
        return self.model.get_option("kv.free_tokens")

    # -- the engine step -----------------------------------------------------------------------------------------------------
    def step(self, entries, end=()):
        """entries: [(request id, token ids, wanted places among these tokens)]; returns the wanted logits in entry / place order,
        [n][vocab].  `end` lists the requests that are finished after this step."""
        batch, want, base = [], [], 0
        for rid, tokens, places in entries:
            slot = self.admit(rid)
            if len(tokens) == 0:                         # an entry that brings nothing this step only keeps (or takes) its slot
                continue
            batch.append((slot, tokens))
            want += [base + int(p) for p in places]
            base += len(tokens)
        out = self.model.step_ragged(batch, want) if batch else np.empty((0, self.desc.vocab), np.float32)
        for rid in end:
            self.release(rid)
        return out

    # -- generation through the same step + the library's sampler -------------------------------------------------------------
    def generate(self, prompts, max_new_tokens: int, cfg: SamplerCfg = GREEDY, seed: int = 0, portion: int = 0):
        """continuous batching over `prompts` (lists of ids): at most max_seqs live; a prompt enters in portions of `portion` tokens
        (0: whole) while the others decode one token per step.  Returns the new ids of every prompt."""
        m, todo = self.model, list(enumerate(prompts))
        out = [[] for _ in prompts]
        live = {}                                        # index -> tokens of the prompt not yet fed
        while todo or live:
            while todo and self.free:
                i, p = todo.pop(0)
                self.admit(("gen", i))
                live[i] = list(p)
            entries, sampled = [], []
            for i, rest in live.items():
                if rest:                                 # next portion of the prompt; its last token's logits when it completes the prompt
                    n = len(rest) if portion <= 0 else min(portion, len(rest))
                    entries.append((("gen", i), rest[:n], [n - 1] if n == len(rest) else []))
                    live[i] = rest[n:]
                else:
                    entries.append((("gen", i), [out[i][-1]], [0]))
                if entries[-1][2]:
                    sampled.append(i)
            self.step(entries)
            done = []
            for i in sampled:
                out[i].append(m.sample_row(self.slot_of[("gen", i)], cfg, seed))
                if len(out[i]) >= max_new_tokens:
                    done.append(i)
            for i in done:
                self.release(("gen", i))
                del live[i]
        return out

    def close(self):
        self.model.close()


def replay_trace(engine: SlotEngine, lines, out_dir: str, emit=print):
    """One JSON object a line: {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}.  Writes <out_dir>/<n>.f32 (the wanted
    logits, little-endian fp32 [wanted][vocab]) for steps that want something and reports 'done <n>' after every step."""
    for line in lines:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in st.get("entries", [])]
        logits = engine.step(entries, st.get("end", []))
        if len(logits):
            tmp = os.path.join(out_dir, f".{st['step']}.part")
            logits.astype("<f4").tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{st['step']}.f32"))
        emit(f"done {st['step']}")
