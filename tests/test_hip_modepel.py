"""The Modepel design on the GPU against the plain oracle of tests/modepel_oracle.py: every mechanism on a configuration of its own, prompts against
token-by-token decoding, portions down to two tokens, mixed batches, slots and pages that are used again, contexts around page borders, sharp far keys,
long decoding through the recurrent state, and greedy generation through the slot scheduler, tgx_forward / tgx_sample / tgx_decode, the C++ engine, the
command line and bin/trace_run.  Models are config dictionaries of the checkpoint format, so the configuration reader is on the path of every test.
fp32 storage is the sharp comparison (nothing is rounded: 1e-4 of the largest logit); bf16 storage rounds the cached keys and values (3e-2)."""
import copy
import json
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

import modepel_oracle as mo
from tinygpt_amd.desc import stack_desc_from_config
from tinygpt_amd.ffi import GREEDY, Model, TgxError
from tinygpt_amd.serving import SlotEngine

pytestmark = pytest.mark.gpu
TOL = {"fp32": 1e-4, "bf16": 3e-2}


# ---- configurations ---------------------------------------------------------------------------------------------------------------
def attn(mlp=None, **kw):
    m = dict(heads=4, kv_heads=2, dim=8, vdim=6, rot={"dims": 4, "base": 100.0}, scale=0.6, v_mix=True)
    m.update(kw)
    return {"type": "attention", "mixer": m, "mlp": mlp}


def rec(mlp=None, **kw):
    m = dict(heads=2, dim=6, vdim=8, gate_cap=15.0)
    m.update(kw)
    return {"type": "mlstm", "mixer": m, "mlp": mlp}


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=4, identity=2, top=2, scale=1.5, count=2, keep=1, ff=12, shared=10):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}},
            "shared": {"ff": shared} if shared else None}


def config(layers=None, width=24, vocab=67, eps=1e-5):
    return {"architecture": "Modepel", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "layers": copy.deepcopy(layers) if layers is not None else [rec(dense()), attn(moe()), attn(moe(top=3, count=3, keep=2)), rec(moe(shared=0))]}


def engine(cfg, dtype="fp32", seed=0, overrides=None, **kw):
    w = mo.random_tensors(cfg, seed, overrides)
    kw = dict(dict(max_seqs=4, max_ctx=1024, budget_tokens=2048), **kw)
    eng = SlotEngine(desc=stack_desc_from_config(cfg, dtype, **kw), tensors={k: np.asarray(v, np.float32) for k, v in w.items()})
    return eng, w


def tokens(cfg, n, seed=0):
    return np.random.default_rng(100 + seed).integers(0, cfg["vocab"], n).tolist()


def want_of(cfg, w, toks):
    return mo.forward(cfg, w, toks)[0]


def check(got, want, dtype, what=""):
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < TOL[dtype], f"{what}: {err:.3e}"


def run_whole(eng, rid, toks):
    return eng.step([(rid, toks, list(range(len(toks))))], [rid])


# ---- every mechanism on a configuration of its own --------------------------------------------------------------------------------------
MECH = {
    "attention_alone": [attn(v_mix=False)],
    "one_key_head_per_query_head": [attn(kv_heads=4, v_mix=False)],
    "one_key_head_for_all": [attn(heads=6, kv_heads=1, v_mix=False)],
    "all_dimensions_rotated": [attn(rot={"dims": 8, "base": 10000.0}, v_mix=False)],
    "two_dimensions_rotated": [attn(rot={"dims": 2, "base": 7.0}, v_mix=False)],
    "wide_heads": [attn(heads=2, kv_heads=1, dim=80, vdim=72, rot={"dims": 32, "base": 500.0}, scale=0.2, v_mix=False)],      # more than one channel per lane
    "value_mixing_over_three_layers": [attn(), attn(), attn(v_mix=False), attn()],
    "value_mixing_starts_late": [attn(v_mix=False), rec(), attn(), attn()],
    "sharp_scores": [attn(scale=3.0), attn(scale=3.0)],
    "mlstm_alone": [rec()],
    "mlstm_one_head_wide": [rec(heads=1, dim=40, vdim=70)],                  # two column chunks, rows spread over the waves
    "mlstm_large_keys": [rec(heads=2, dim=130, vdim=9)],
    "mlstm_very_large_keys": [rec(heads=1, dim=260, vdim=20)],
    "mlstm_small_cap": [rec(gate_cap=1.5), rec(gate_cap=1.5)],
    "dense_ff": [attn(dense(ff=33), v_mix=False)],
    "experts_top_one": [attn(moe(top=1, count=1, keep=1))],
    "experts_no_identity": [rec(moe(identity=0, count=2, keep=1))],
    "experts_only_identity_kept_possible": [attn(moe(experts=2, identity=4, top=2, count=3, keep=1))],
    "experts_no_groups_no_shared": [attn(moe(count=1, keep=1, shared=0, top=4))],
    "experts_many": [rec(moe(experts=60, identity=12, top=6, count=8, keep=3, ff=8))],
    "experts_all_groups_kept": [attn(moe(count=3, keep=3, top=5))],
    "no_feed_forward_anywhere": [attn(), rec(), attn()],
    "ragged_sizes": [rec(dense(ff=19), heads=3, dim=5, vdim=7), attn(moe(ff=11, shared=9), heads=6, kv_heads=3, dim=6, vdim=5, rot={"dims": 6, "base": 50.0})],
    "deep": [rec(dense()), attn(moe()), attn(moe()), rec(moe())] * 2,
}
WIDTHS = {"ragged_sizes": dict(width=27, vocab=53), "wide_heads": dict(width=40)}


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("name", list(MECH))
def test_mechanism(name, dtype):
    cfg = config(MECH[name], **WIDTHS.get(name, {}))
    eng, w = engine(cfg, dtype, seed=len(name))
    toks = tokens(cfg, 21, seed=len(name))
    check(run_whole(eng, "a", toks), want_of(cfg, w, toks), dtype, name)
    # ... and the same tokens one by one through the cache and the recurrent state
    got = np.concatenate([eng.step([("b", [t], [0])]) for t in toks])
    check(got, want_of(cfg, w, toks), dtype, name + " by steps")
    eng.close()


def test_the_sink_takes_the_weight_when_every_score_is_low():
    """queries and keys made large and opposed: every score is far below the sink's 0, so the mixer's output almost vanishes; a softmax without the
    sink would return an average of the values instead"""
    cfg = config([attn(scale=1.0, v_mix=False, rot={"dims": 2, "base": 100.0})])
    w0 = mo.random_tensors(cfg, 1)
    over = {"l0.mix.q": np.zeros_like(w0["l0.mix.q"]), "l0.mix.k": np.zeros_like(w0["l0.mix.k"]),
            "l0.mix.q.b": np.tile([0, 0, 3.0, 3.0, 3.0, 3.0, 3.0, 3.0], 4), "l0.mix.k.b": np.tile([0, 0, -3.0, -3.0, -3.0, -3.0, -3.0, -3.0], 2)}
    eng, w = engine(cfg, "fp32", 1, over)
    toks = tokens(cfg, 30)
    want = want_of(cfg, w, toks)
    no_mixer = want_of(cfg, {**w, "l0.mix.o": np.zeros_like(w["l0.mix.o"])}, toks)
    assert np.abs(want - no_mixer).max() / np.abs(want).max() < 0.5      # (the norm behind the mixer rescales whatever is left, so the comparison is loose)
    check(run_whole(eng, "a", toks), want, "fp32")
    eng.close()


# ---- prompts, decoding, portions --------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_prompt_then_token_by_token(dtype):
    cfg = config()
    eng, w = engine(cfg, dtype, 1)
    toks = tokens(cfg, 40)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:9], list(range(9)))])]
    for i in range(9, 40):
        got.append(eng.step([("r", [toks[i]], [0])]))
    check(np.concatenate(got), want, dtype)
    eng.release("r")
    got = np.concatenate([eng.step([("s", [toks[i]], [0])]) for i in range(6)])      # the first tokens of a sequence in a slot that held another one
    check(got, want[:6], dtype, "from the first token")
    eng.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("sizes", [[2] * 20, [3, 2, 5, 2, 7, 1, 11, 2, 2], [64, 2, 63, 1], [1, 128, 2, 65], [5, 59, 64, 2]])
def test_portions(sizes, dtype):
    cfg = config()
    eng, w = engine(cfg, dtype, 2)
    toks = tokens(cfg, sum(sizes), seed=len(sizes))
    want = want_of(cfg, w, toks)
    got, at = [], 0
    for n in sizes:
        got.append(eng.step([("r", toks[at:at + n], list(range(n)))]))
        at += n
    check(np.concatenate(got), want, dtype)
    eng.close()


@pytest.mark.parametrize("n", [1, 63, 64, 65, 127, 128, 129, 200])
def test_contexts_around_page_borders(n):
    cfg = config([attn(scale=2.0), rec(moe()), attn(dense())])
    eng, w = engine(cfg, "fp32", 4)
    toks = tokens(cfg, n + 3, seed=n)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:n], [n - 1])])]
    got += [eng.step([("r", [toks[n + i]], [0])]) for i in range(3)]      # decoding across the border
    check(np.concatenate(got), want[n - 1:], "fp32")
    eng.close()


def test_far_keys_carry_weight():
    """sharp scores over a long context: the keys that hold a query's weight lie anywhere, hundreds of tokens back; in a prompt's portion and for decoded tokens"""
    cfg = config([attn(scale=4.0, heads=2, kv_heads=1, dim=8, vdim=8, v_mix=False, rot={"dims": 4, "base": 10000.0})])
    eng, w = engine(cfg, "fp32", 5)
    toks = tokens(cfg, 600)
    want = want_of(cfg, w, toks)
    got = [eng.step([("r", toks[:590], [0, 1, 2, 300, 588, 589])])]
    got += [eng.step([("r", [toks[590 + i]], [0])]) for i in range(10)]
    check(np.concatenate(got), want[[0, 1, 2, 300, 588, 589] + list(range(590, 600))], "fp32")
    eng.close()


def test_one_far_key_stands_out():
    """one early token's key is made to match the later queries: token id 7 has an embedding row that the key projection answers strongly, and it occurs
    once, at position 3; every later query must find it among hundreds of keys (also across page borders and in decoded tokens)"""
    cfg = config([attn(scale=1.0, heads=2, kv_heads=1, dim=8, vdim=8, v_mix=False, rot={"dims": 2, "base": 10000.0})], width=16)
    w0 = mo.random_tensors(cfg, 6)
    emb = w0["embed"].copy()
    emb[:, 0] = 0.0; emb[7] = 0.0; emb[7, 0] = 6.0                  # a token whose stream is one loud coordinate that no other token has
    k = w0["l0.mix.k"].copy(); k[:, 0] = 0.0; k[5, 0] = 8.0         # ... that the key projection turns into a large un-rotated key coordinate
    qb = w0["l0.mix.q.b"].copy(); qb[5] = 4.0; qb[13] = 4.0         # ... which every query of both heads asks for
    eng, w = engine(cfg, "fp32", 6, {"embed": emb, "l0.mix.k": k, "l0.mix.q.b": qb})
    toks = [t if t != 7 else 8 for t in tokens(cfg, 400)]
    toks[3] = 7
    want = want_of(cfg, w, toks)
    without = list(toks); without[3] = 9
    assert np.abs(want_of(cfg, w, without)[390:] - want[390:]).max() / np.abs(want).max() > 0.05      # the far key decides these logits
    got = [eng.step([("r", toks[:200], [2, 3, 4, 199])]), eng.step([("r", toks[200:390], [0, 189])])]
    got += [eng.step([("r", [toks[390 + i]], [0])]) for i in range(10)]
    check(np.concatenate(got), want[[2, 3, 4, 199, 200, 389] + list(range(390, 400))], "fp32")
    eng.close()


def test_split_keys_form_equals_the_direct_form():
    cfg = config([attn(scale=2.0), attn(moe())])
    eng, w = engine(cfg, "fp32", 6)
    toks = tokens(cfg, 700)
    want = want_of(cfg, w, toks)
    eng.step([("r", toks[:690], [])])
    eng.model.set_option("attn.split_min", 64)            # steps of few tokens now divide the keys between workgroups
    got = np.concatenate([eng.step([("r", [toks[690 + i]], [0])]) for i in range(10)])
    check(got, want[690:], "fp32")
    eng.close()


def test_long_memory_through_the_recurrent_state():
    """forget gates held near one: the matrix memory still carries the first tokens after hundreds of steps, through portions and single tokens"""
    cfg = config([rec(dense()), rec()])
    w0 = mo.random_tensors(cfg, 7)
    eng, w = engine(cfg, "fp32", 7, {"l0.mix.f.b": np.full(2, 9.0), "l1.mix.f.b": np.full(2, 9.0)})
    toks = tokens(cfg, 330)
    want = want_of(cfg, w, toks)
    other = want_of(cfg, w, [toks[0] + 1] + toks[1:])
    assert np.abs(other[-1] - want[-1]).max() / np.abs(want).max() > 1e-3      # the first token still matters at the end
    got = [eng.step([("r", toks[:5], [4])]), eng.step([("r", toks[5:130], [0, 124])]), eng.step([("r", toks[130:300], [169])])]
    got += [eng.step([("r", [toks[300 + i]], [0])]) for i in range(30)]
    check(np.concatenate(got), want[[4, 5, 129, 299] + list(range(300, 330))], "fp32")
    eng.close()


# ---- batches, slots, pages ----------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_unequal_requests_in_one_batch(dtype):
    cfg = config()
    eng, w = engine(cfg, dtype, 7)
    seqs = {"a": tokens(cfg, 70, 1), "b": tokens(cfg, 9, 2), "c": tokens(cfg, 33, 3), "d": tokens(cfg, 1, 4)}
    want = {k: want_of(cfg, w, v) for k, v in seqs.items()}
    cuts = {"a": [17, 2, 30, 1, 1, 19], "b": [1, 1, 1, 2, 4, 0], "c": [2, 0, 2, 29, 0, 0], "d": [0, 0, 1, 0, 0, 0]}      # 0: the request sits the step out
    got = {k: [] for k in seqs}
    at = {k: 0 for k in seqs}
    for step in range(6):
        entries = []
        for k in seqs:
            n = cuts[k][step]
            if n:
                entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
        out = eng.step(entries)
        o = 0
        for k, tk, _ in entries:
            got[k].append(out[o:o + len(tk)]); o += len(tk); at[k] += len(tk)
    for k in seqs:
        g = np.concatenate(got[k])
        check(g, want[k][:len(g)], dtype, k)
        assert len(g) == min(len(seqs[k]), sum(cuts[k]))
    eng.close()


def test_slots_and_pages_are_used_again():
    cfg = config()
    eng, w = engine(cfg, "fp32", 8, budget_tokens=256, max_ctx=256, max_seqs=2)      # four pages of 64 tokens, two slots
    assert eng.free_tokens == 256
    for rnd in range(5):
        a, b = tokens(cfg, 100 + rnd, 10 + rnd), tokens(cfg, 60 + rnd, 20 + rnd)
        out = eng.step([(("a", rnd), a, [len(a) - 1]), (("b", rnd), b[:-1], [])])
        assert eng.free_tokens == 256 - 128 - 64
        with pytest.raises(RuntimeError):      # both slots are taken
            eng.step([(("c", rnd), [1], [])])
        out2 = eng.step([(("b", rnd), b[-1:], [0])], end=[("a", rnd)])
        check(np.concatenate([out, out2]), np.stack([want_of(cfg, w, a)[-1], want_of(cfg, w, b)[-1]]), "fp32", f"round {rnd}")
        eng.release(("b", rnd))
        assert eng.free_tokens == 256
    eng.step([("big", tokens(cfg, 200), [])])          # the pool refuses what it cannot hold and leaves the slots as they were
    with pytest.raises(TgxError):
        eng.step([("more", tokens(cfg, 100), [])])
    assert eng.length("big") == 200 and eng.length("more") == 0
    eng.close()


def test_a_request_is_the_same_alone_and_beside_others():
    """nothing a token computes reads another entry of the batch; what differs is the summation order of the products (few rows stream the weights,
    many take the matrix-core tiles)"""
    cfg = config()
    eng, w = engine(cfg, "fp32", 9)
    a, b, c = tokens(cfg, 50, 1), tokens(cfg, 20, 2), tokens(cfg, 3, 3)
    alone = np.concatenate([eng.step([("a", a[:31], [30])]), eng.step([("a", a[31:], [18])], ["a"])])
    eng.step([("c", c, [])])
    mixed = np.concatenate([eng.step([("b", b[:7], []), ("a", a[:31], [30])]), eng.step([("a", a[31:], [18]), ("c", [5], []), ("b", b[7:], [])], ["a", "b", "c"])])
    assert np.abs(alone - mixed).max() / np.abs(alone).max() < 1e-5
    eng.close()


# ---- generation ---------------------------------------------------------------------------------------------------------------------------
def oracle_greedy(cfg, w, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(np.argmax(want_of(cfg, w, seq)[-1])))
    return seq[len(prompt):]


def test_greedy_generation_through_the_slot_scheduler():
    cfg = config()
    eng, w = engine(cfg, "fp32", 9, max_seqs=2)
    prompts = [tokens(cfg, 11, 1), tokens(cfg, 5, 2), tokens(cfg, 23, 3)]      # three requests on two slots
    want = [oracle_greedy(cfg, w, p, 6) for p in prompts]
    assert eng.generate(prompts, 6) == want
    assert eng.generate(prompts, 6, portion=4) == want
    eng.close()


def test_long_decoding_through_forward_sample_decode():
    cfg = config([rec(moe()), attn(dense()), attn()])
    w = mo.random_tensors(cfg, 10)
    m = Model(stack_desc_from_config(cfg, "fp32", max_seqs=2, max_ctx=512)).load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True).finalize()
    prompts = np.array([tokens(cfg, 7, 1), tokens(cfg, 7, 2)])
    m.forward(prompts)
    first = m.sample(GREEDY)
    rest = np.concatenate([m.decode(75, GREEDY), m.decode(75, GREEDY)])      # crosses two page borders; positions, state and its buffer parity (an odd count) advance on the device
    for b in range(2):
        got = [int(first[b])] + rest[:, b].tolist()
        seq = prompts[b].tolist() + got
        lg = want_of(cfg, w, seq[:-1])
        top2 = np.sort(lg[6:], -1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 1e-3 * np.abs(lg).max()
        assert (np.argmax(lg[6:], -1)[clear] == np.array(got)[clear]).all()
        assert clear.mean() > 0.9
    assert m.past_length == 7 + 150
    m.close()


# ---- the C++ host engine, the command line, the trace replay ---------------------------------------------------------------------------------
def write_model_dir(path, cfg, w):
    """config.json + model.safetensors (bf16; the oracle's weights are on the bf16 grid)"""
    with open(f"{path}/config.json", "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, a in w.items():
        bits = (np.asarray(a, np.float32).reshape(-1).view(np.uint32) >> 16).astype(np.uint16)
        header[name] = {"dtype": "BF16", "shape": list(np.shape(a)), "data_offsets": [at, at + bits.nbytes]}
        blobs.append(bits.tobytes()); at += bits.nbytes
    hj = json.dumps(header).encode()
    with open(f"{path}/model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def test_host_engine_and_cli_generate_greedy(tmp_path):
    from host_util import HostEngine, host_lib
    from tinygpt_amd import build
    cfg = config([rec(dense()), attn(moe()), attn()])
    w = mo.random_tensors(cfg, 11)
    write_model_dir(str(tmp_path), cfg, w)
    prompts = [tokens(cfg, 9, 1), tokens(cfg, 4, 2), tokens(cfg, 13, 3)]           # unequal lengths: no padding is fed
    want = [oracle_greedy(cfg, w, p, 5) for p in prompts]
    e = HostEngine(host_lib(), model_dir=str(tmp_path), device="mi355x", dtype=0, max_batch=4)
    assert e.prepare(), e.error()
    e.reconfigure(max_new=5)
    ids, new, fin = e.generate_sync(prompts)
    assert new == 5 and [ids[b, -5:].tolist() for b in range(3)] == want
    e.reconfigure(max_new=5)
    ids2, new2, fin2, seen = e.generate_async(prompts[2])
    assert ids2[-5:].tolist() == want[2]
    e.close()
    build.build_host()
    arg = ";".join(",".join(str(x) for x in p) for p in prompts)
    r = subprocess.run([build.HOST_CLI, "--model", str(tmp_path), "--dtype", "fp32", "--max-tokens", "5", "--temperature", "0", "--top-p", "1", "--prompt-ids", arg,
                        "--context", "256"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    outs = [[int(x) for x in line.split(":")[1].split()] for line in r.stdout.splitlines() if line.startswith("Output ids")]
    assert outs == want


def test_trace_replay_script(tmp_path):
    cfg = config([attn(moe()), rec(dense())])
    w = mo.random_tensors(cfg, 12)
    mdir, out = tmp_path / "m", tmp_path / "o"
    mdir.mkdir()
    write_model_dir(str(mdir), cfg, w)
    a, b = tokens(cfg, 30, 1), tokens(cfg, 12, 2)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": b[:11], "want": []}, {"id": "x", "tokens": a[20:22], "want": [1]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": a[22:], "want": [7]}, {"id": "y", "tokens": b[11:], "want": [0]}], "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype, tol in (("float32", "fp32"), ("bfloat16", "bf16")):
        r = subprocess.run([sys.executable, f"{root}/bin/trace_run", "--model", str(mdir), "--dtype", dtype, "--out", str(out), "--max-tokens", "128"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
        wa, wb = want_of(cfg, w, a), want_of(cfg, w, b)
        check(np.fromfile(out / "0.f32", "<f4").reshape(2, -1), wa[[0, 19]], tol)
        check(np.fromfile(out / "1.f32", "<f4").reshape(1, -1), wa[[21]], tol)
        check(np.fromfile(out / "2.f32", "<f4").reshape(2, -1), np.stack([wa[29], wb[11]]), tol)


def test_what_the_library_refuses():
    bad = config([attn(kv_heads=3)])                     # query heads not a multiple of the key heads
    with pytest.raises(TgxError):
        Model(stack_desc_from_config(bad, "fp32"))
    bad = config([attn(), attn(vdim=4)])                 # value mixing between layers of different value size
    with pytest.raises(TgxError):
        Model(stack_desc_from_config(bad, "fp32"))
    bad = config([attn(moe(count=4))])                   # six router outputs do not form four equal groups
    with pytest.raises(TgxError):
        Model(stack_desc_from_config(bad, "fp32"))
    cfg = config([rec()])
    w = mo.random_tensors(cfg, 0)
    m = Model(stack_desc_from_config(cfg, "fp32"))
    del w["l0.mix.f.b"]
    m.load_state({k: np.asarray(v, np.float32) for k, v in w.items()}, strict=True)
    with pytest.raises(TgxError, match="l0.mix.f.b"):
        m.finalize()
    m.close()


# ---- attention on the matrix cores (16-bit storage; key sizes 64 / 128 / 256, value sizes in steps of 32) --------------------------------------
@pytest.mark.parametrize("heads,kv,dim,vdim", [(4, 1, 64, 32), (8, 2, 128, 128), (6, 3, 64, 96), (2, 2, 128, 256), (16, 4, 64, 64), (3, 1, 256, 192)])
def test_matrix_core_attention_equals_the_lane_kernel(heads, kv, dim, vdim):
    """the same bf16 weights and cached rows through both attention kernels: portions whose 32-row tiles cut through tokens, a mixed batch, decoding,
    contexts across page borders, and the split-keys form.  The two differ by summation order and the two-term rounding of q and p only."""
    mixer = dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, rot={"dims": 32, "base": 10000.0}, scale=1.2 * dim ** -0.5)
    cfg = config([attn(**mixer), attn(moe(), **mixer)], width=64)
    w = mo.random_tensors(cfg, heads)
    tens = {k: np.asarray(v, np.float32) for k, v in w.items()}
    mk = lambda: SlotEngine(desc=stack_desc_from_config(cfg, "bf16", max_seqs=4, max_ctx=1024, budget_tokens=2048), tensors=tens)
    fast, slow = mk(), mk()
    slow.model.set_option("attn.mfma", 0)
    a, b, c = tokens(cfg, 200, 1), tokens(cfg, 75, 2), tokens(cfg, 9, 3)
    want = want_of(cfg, w, a)[[0, 1, 69, 130, 131, 199]]
    outs = []
    for eng in (fast, slow):
        o = [eng.step([("a", a[:70], [0, 1, 69]), ("b", b[:3], [2])])]
        o.append(eng.step([("a", a[70:131], [60]), ("c", c, [8]), ("b", b[3:4], [0])]))
        o.append(eng.step([("b", b[4:], [70]), ("a", a[131:132], [0])]))
        o.append(eng.step([("a", a[132:199], [])]))
        eng.model.set_option("attn.split_min", 64)
        o.append(eng.step([("a", a[199:], [0]), ("b", [5], [0])]))
        outs.append(np.concatenate(o))
    assert np.abs(outs[0] - outs[1]).max() / np.abs(outs[1]).max() < 3e-4
    check(outs[0][[0, 1, 2, 4, 8, 9]], want, "bf16")               # a's positions 0, 1, 69, 130, 131, 199 in the order the steps returned them
    check(outs[0][[6, 7]], want_of(cfg, w, b)[[3, 74]], "bf16")
    fast.close(); slow.close()


@pytest.mark.parametrize("dim,vdim", [(6, 8), (24, 70), (128, 40), (250, 33)])
def test_both_column_splits_of_the_matrix_memory_scan(dim, vdim):
    """the scan gives a wave sixteen columns, or eight when the step leaves most of the chip idle: the same steps through both (and against the oracle)"""
    cfg = config([rec(dense(), heads=2, dim=dim, vdim=vdim), rec(heads=3, dim=dim, vdim=vdim)], width=32)
    w = mo.random_tensors(cfg, dim)
    tens = {k: np.asarray(v, np.float32) for k, v in w.items()}
    a, b = tokens(cfg, 90, 1), tokens(cfg, 37, 2)
    outs = []
    for narrow in (0, 1):
        eng = SlotEngine(desc=stack_desc_from_config(cfg, "fp32", max_seqs=4, max_ctx=256, budget_tokens=512), tensors=tens)
        eng.model.set_option("mlstm.narrow", narrow)
        o = [eng.step([("a", a[:50], [0, 31, 32, 49]), ("b", b[:1], [0])])]
        o.append(eng.step([("a", a[50:52], [1]), ("b", b[1:36], [34])]))
        o.append(eng.step([("a", a[52:], [37]), ("b", b[36:], [0])]))
        outs.append(np.concatenate(o))
        eng.close()
    wa, wb = want_of(cfg, w, a), want_of(cfg, w, b)
    want = np.stack([wa[0], wa[31], wa[32], wa[49], wb[0], wa[51], wb[35], wa[89], wb[36]])
    check(outs[0], want, "fp32", "sixteen columns")
    check(outs[1], want, "fp32", "eight columns")
