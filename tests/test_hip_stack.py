"""The layered (Zakusun) model on the GPU against the plain oracle of tests/stack_oracle.py: every mechanism on configurations of its own, prompts
against token-by-token decoding, portions, mixed batches, slots and pages that are used again, contexts around page borders, long decoding, and
greedy generation through the slot scheduler and through tgx_forward / tgx_sample / tgx_decode.  fp32 storage is the sharp comparison (nothing is
rounded: 1e-4 of the largest logit); bf16 storage rounds the cached latents (3e-2)."""
import numpy as np
import pytest

import stack_oracle as so
from tinygpt_amd.desc import LayerDesc, StackDesc
from tinygpt_amd.ffi import GREEDY, Model, TgxError
from tinygpt_amd.serving import SlotEngine

pytestmark = pytest.mark.gpu
TOL = {"fp32": 1e-4, "bf16": 3e-2}


def moe_layer(**kw):
    base = dict(heads=3, dim=8, vdim=4, kv_rank=16, scale=0.4, mlp="moe", experts=5, top=2, ff=24, limit=1.5)
    base.update(kw)
    return LayerDesc(**base)


def plain_layer(**kw):
    base = dict(heads=2, dim=8, vdim=8, kv_rank=8, scale=0.35, mlp=None)
    base.update(kw)
    return LayerDesc(**base)


def small_desc(dtype="fp32", layers=None, **kw):
    base = dict(width=32, vocab=97, canon_taps=4, norm_groups=2, norm_eps=1e-6, logit_scale=0.5, max_seqs=4, max_ctx=1024, budget_tokens=2048,
                compute_dtype=dtype, layers=layers or [moe_layer(), plain_layer(), moe_layer(heads=2, dim=16, kv_rank=24, experts=4, top=3)])
    base.update(kw)
    return StackDesc(**base)


def engine(desc, seed=0, **kw):
    t = so.random_tensors(desc, seed, **kw)
    return SlotEngine(desc=desc, tensors={k: v.astype(np.float32) for k, v in t.items()}), t


def tokens(desc, n, seed=0):
    return np.random.default_rng(100 + seed).integers(0, desc.vocab, n).tolist()


def check(got, want, dtype, what=""):
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < TOL[dtype], f"{what}: {err:.3e}"


def run_whole(eng, rid, toks):
    return eng.step([(rid, toks, list(range(len(toks))))], [rid])


# ---- every mechanism on a configuration of its own -----------------------------------------------------------------------------
MECH = {
    "one_group_one_tap": dict(norm_groups=1, canon_taps=1, layers=[plain_layer()]),
    "four_groups": dict(norm_groups=4, layers=[plain_layer()]),
    "two_taps": dict(canon_taps=2, layers=[plain_layer()]),
    "five_taps": dict(canon_taps=5, layers=[plain_layer(), plain_layer()]),
    "one_head": dict(layers=[plain_layer(heads=1, dim=16, vdim=12, kv_rank=24)]),
    "wide_latent": dict(layers=[plain_layer(heads=4, dim=8, vdim=8, kv_rank=160)]),          # several latent channels per lane
    "very_wide_latent": dict(layers=[plain_layer(heads=2, dim=8, vdim=8, kv_rank=1100)]),
    "sharp_scores": dict(layers=[plain_layer(scale=3.0), plain_layer(scale=3.0)]),            # peaked softmax: single keys carry the output
    "top_one": dict(layers=[moe_layer(top=1)]),
    "top_all": dict(layers=[moe_layer(experts=4, top=4)]),
    "many_experts": dict(layers=[moe_layer(experts=70, top=6, ff=8)]),
    "tight_clamp": dict(layers=[moe_layer(limit=0.25)]),
    "ragged_sizes": dict(width=36, vocab=101, norm_groups=3, layers=[moe_layer(heads=3, dim=6, vdim=5, kv_rank=10, ff=18), plain_layer(heads=5, dim=4, vdim=3, kv_rank=7)]),
    "odd_width": dict(width=27, vocab=53, norm_groups=3, canon_taps=3, layers=[moe_layer(heads=3, dim=5, vdim=7, kv_rank=9, ff=11, experts=3, top=2), plain_layer(heads=2, dim=3, vdim=5, kv_rank=6)]),
    "no_feed_forward_anywhere": dict(layers=[plain_layer(), plain_layer(), plain_layer()]),
    "deep": dict(layers=[moe_layer(), plain_layer()] * 4),
    "logit_scale": dict(logit_scale=3.0, layers=[plain_layer()]),
}


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("name", list(MECH))
def test_mechanism(name, dtype):
    d = small_desc(dtype, **MECH[name])
    eng, t = engine(d, seed=len(name))
    toks = tokens(d, 19, seed=len(name))
    check(run_whole(eng, "a", toks), so.forward(d, t, toks), dtype, name)
    eng.close()


def test_sink_and_gate_matter():
    """the comparison above would not see a mechanism whose weights were negligible: the sink and the gate change these logits by far more than the tolerance"""
    d = small_desc("fp32", layers=[plain_layer()])
    t = so.random_tensors(d, 3)
    toks = tokens(d, 12)
    base = so.forward(d, t, toks)
    no_sink = dict(t); no_sink["l0.mix.sink"] = np.full_like(t["l0.mix.sink"], -60.0)
    no_gate = dict(t); no_gate["l0.mix.g"] = np.zeros_like(t["l0.mix.g"])
    for other in (no_sink, no_gate):
        assert np.abs(so.forward(d, other, toks) - base).max() / np.abs(base).max() > 50 * TOL["fp32"]


# ---- prompts, decoding, portions -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_prompt_then_token_by_token(dtype):
    d = small_desc(dtype)
    eng, t = engine(d, 1)
    toks = tokens(d, 40)
    want = so.forward(d, t, toks)
    got = [eng.step([("r", toks[:9], list(range(9)))])]
    for i in range(9, 40):
        got.append(eng.step([("r", [toks[i]], [0])]))
    check(np.concatenate(got), want, dtype)
    # the first tokens of a sequence, one by one from an empty slot (shorter than the convolution)
    eng.release("r")
    got = np.concatenate([eng.step([("s", [toks[i]], [0])]) for i in range(6)])
    check(got, want[:6], dtype, "from the first token")
    eng.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("sizes", [[2] * 20, [3, 2, 5, 2, 7, 1, 11, 2, 2], [64, 2, 63, 1], [1, 128, 2, 65], [5, 59, 64, 2]])
def test_portions(sizes, dtype):
    d = small_desc(dtype)
    eng, t = engine(d, 2)
    toks = tokens(d, sum(sizes), seed=len(sizes))
    want = so.forward(d, t, toks)
    got, at = [], 0
    for n in sizes:
        got.append(eng.step([("r", toks[at:at + n], list(range(n)))]))
        at += n
    check(np.concatenate(got), want, dtype)
    eng.close()


@pytest.mark.parametrize("n", [1, 63, 64, 65, 127, 128, 129, 200])
def test_contexts_around_page_borders(n):
    d = small_desc("fp32", layers=[plain_layer(scale=2.0), moe_layer()])
    eng, t = engine(d, 4)
    toks = tokens(d, n + 3, seed=n)
    want = so.forward(d, t, toks)
    got = [eng.step([("r", toks[:n], [n - 1])])]
    got += [eng.step([("r", [toks[n + i]], [0])]) for i in range(3)]      # decoding across the border
    check(np.concatenate(got), want[n - 1:], "fp32")
    eng.close()


def test_far_keys_carry_weight():
    """sharp scores over a long context: the keys that hold a query's weight lie anywhere, hundreds of tokens back; prompt portion and decoded tokens"""
    d = small_desc("fp32", layers=[plain_layer(scale=4.0, heads=2, dim=8, vdim=8, kv_rank=12)], budget_tokens=1024)
    eng, t = engine(d, 5, sink_scale=0.5)
    toks = tokens(d, 600)
    want = so.forward(d, t, toks)
    got = [eng.step([("r", toks[:590], [0, 1, 2, 300, 588, 589])])]
    got += [eng.step([("r", [toks[590 + i]], [0])]) for i in range(10)]
    check(np.concatenate(got), want[[0, 1, 2, 300, 588, 589] + list(range(590, 600))], "fp32")
    eng.close()


def test_split_keys_form_equals_the_direct_form():
    d = small_desc("fp32", layers=[plain_layer(scale=2.0), moe_layer()], budget_tokens=1024)
    eng, t = engine(d, 6)
    toks = tokens(d, 700)
    want = so.forward(d, t, toks)
    eng.step([("r", toks[:690], [])])
    eng.model.set_option("attn.split_min", 64)            # steps of few tokens now divide the keys between workgroups
    got = np.concatenate([eng.step([("r", [toks[690 + i]], [0])]) for i in range(10)])
    check(got, want[690:], "fp32")
    eng.close()


# ---- batches, slots, pages --------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_unequal_requests_in_one_batch(dtype):
    d = small_desc(dtype)
    eng, t = engine(d, 7)
    seqs = {"a": tokens(d, 70, 1), "b": tokens(d, 9, 2), "c": tokens(d, 33, 3), "d": tokens(d, 1, 4)}
    want = {k: so.forward(d, t, v) for k, v in seqs.items()}
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
    d = small_desc("fp32", budget_tokens=256, max_ctx=256, max_seqs=2)      # four pages of 64 tokens, two slots
    eng, t = engine(d, 8)
    assert eng.free_tokens == 256
    for rnd in range(5):
        a, b = tokens(d, 100 + rnd, 10 + rnd), tokens(d, 60 + rnd, 20 + rnd)
        out = eng.step([(("a", rnd), a, [len(a) - 1]), (("b", rnd), b[:-1], [])])
        assert eng.free_tokens == 256 - 128 - 64
        with pytest.raises(RuntimeError):      # both slots are taken
            eng.step([(("c", rnd), [1], [])])
        out2 = eng.step([(("b", rnd), b[-1:], [0])], end=[("a", rnd)])
        check(np.concatenate([out, out2]), np.stack([so.forward(d, t, a)[-1], so.forward(d, t, b)[-1]]), "fp32", f"round {rnd}")
        eng.release(("b", rnd))
        assert eng.free_tokens == 256
    # the pool refuses what it cannot hold and leaves the slots as they were
    eng.step([("big", tokens(d, 200), [])])
    with pytest.raises(TgxError):
        eng.step([("more", tokens(d, 100), [])])
    assert eng.length("big") == 200 and eng.length("more") == 0
    eng.close()


# ---- generation -------------------------------------------------------------------------------------------------------------------
def oracle_greedy(d, t, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(np.argmax(so.forward(d, t, seq)[-1])))
    return seq[len(prompt):]


def test_greedy_generation_through_the_slot_scheduler():
    d = small_desc("fp32", max_seqs=2)
    eng, t = engine(d, 9)
    prompts = [tokens(d, 11, 1), tokens(d, 5, 2), tokens(d, 23, 3)]      # three requests on two slots
    want = [oracle_greedy(d, t, p, 6) for p in prompts]
    assert eng.generate(prompts, 6) == want
    assert eng.generate(prompts, 6, portion=4) == want
    eng.close()


def test_long_decoding_through_forward_sample_decode():
    d = small_desc("fp32", layers=[moe_layer(), plain_layer()])
    t = so.random_tensors(d, 10)
    m = Model(d).load_state({k: v.astype(np.float32) for k, v in t.items()}, strict=True).finalize()
    prompts = np.array([tokens(d, 7, 1), tokens(d, 7, 2)])
    m.forward(prompts)
    first = m.sample(GREEDY)
    rest = m.decode(150, GREEDY)                                         # crosses two page borders
    for b in range(2):
        got = [int(first[b])] + rest[:, b].tolist()
        seq = prompts[b].tolist() + got
        lg = so.forward(d, t, seq[:-1])
        # teacher-forced: every produced token is the oracle's argmax given the tokens before it (wherever the oracle's top-2 gap is not a tie)
        top2 = np.sort(lg[6:], -1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 1e-3 * np.abs(lg).max()
        assert (np.argmax(lg[6:], -1)[clear] == np.array(got)[clear]).all()
        assert clear.mean() > 0.9
    assert m.past_length == 7 + 150
    m.close()


# ---- the C++ host engine and the command line ---------------------------------------------------------------------------------------
def write_stack_dir(path, d, t, cfg_extra=None):
    """config.json + model.safetensors (bf16) of a layered model"""
    import json
    import struct
    layers = []
    for l in d.layers:
        e = {"type": l.mixer, "mixer": {"heads": l.heads, "dim": l.dim, "vdim": l.vdim, "kv_rank": l.kv_rank, "scale": l.scale}, "mlp": None}
        if l.mlp:
            e["mlp"] = {"kind": l.mlp, "expert": {"ff": l.ff, "limit": l.limit}, "router": {"experts": l.experts, "top": l.top}}
        layers.append(e)
    cfg = {"architecture": "Zakusun", "width": d.width, "vocab": d.vocab, "logit_scale": d.logit_scale, "norm": {"eps": d.norm_eps, "groups": d.norm_groups},
           "canon": {"taps": d.canon_taps}, "layers": layers}
    with open(f"{path}/config.json", "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, a in t.items():
        bits = (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)      # the oracle's weights are bf16-representable
        header[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [at, at + bits.nbytes]}
        blobs.append(bits.tobytes()); at += bits.nbytes
    hj = json.dumps(header).encode()
    with open(f"{path}/model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def test_host_engine_and_cli_generate_greedy(tmp_path):
    import subprocess
    from host_util import HostEngine, host_lib
    from tinygpt_amd import build
    d = small_desc("fp32", layers=[moe_layer(), plain_layer()])
    t = so.random_tensors(d, 11)
    write_stack_dir(str(tmp_path), d, t)
    prompts = [tokens(d, 9, 1), tokens(d, 4, 2), tokens(d, 13, 3)]           # unequal lengths: no padding is fed
    want = [oracle_greedy(d, t, p, 5) for p in prompts]
    e = HostEngine(host_lib(), model_dir=str(tmp_path), device="mi355x", dtype=0, max_batch=4)
    assert e.prepare(), e.error()
    e.reconfigure(max_new=5)
    ids, new, fin = e.generate_sync(prompts)
    assert new == 5 and [ids[b, -5:].tolist() for b in range(3)] == want
    e.reconfigure(max_new=5)
    ids2, new2, fin2, seen = e.generate_async(prompts[2])                     # streaming: forward + the ticket pipeline
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
    """bin/trace_run: steps in on stdin, logits out as files, 'done <n>' per step; slots are named by the trace's request ids"""
    import json
    import subprocess
    import sys
    d = small_desc("fp32", layers=[plain_layer(), moe_layer()])
    t = so.random_tensors(d, 12)
    mdir, out = tmp_path / "m", tmp_path / "o"
    mdir.mkdir()
    write_stack_dir(str(mdir), d, t)
    a, b = tokens(d, 30, 1), tokens(d, 12, 2)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": b[:11], "want": []}, {"id": "x", "tokens": a[20:22], "want": [1]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": a[22:], "want": [7]}, {"id": "y", "tokens": b[11:], "want": [0]}], "end": ["x", "y"]}]
    root = __import__("os").path.dirname(__import__("os").path.dirname(__import__("os").path.abspath(__file__)))
    r = subprocess.run([sys.executable, f"{root}/bin/trace_run", "--model", str(mdir), "--dtype", "float32", "--out", str(out), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = so.forward(d, t, a), so.forward(d, t, b)
    check(np.fromfile(out / "0.f32", "<f4").reshape(2, -1), wa[[0, 19]], "fp32")
    check(np.fromfile(out / "1.f32", "<f4").reshape(1, -1), wa[[21]], "fp32")
    check(np.fromfile(out / "2.f32", "<f4").reshape(2, -1), np.stack([wa[29], wb[11]]), "fp32")


# ---- latent attention on the matrix cores (16-bit storage, latent widths of 128 .. 512) ---------------------------------------------
@pytest.mark.parametrize("heads,rank", [(3, 128), (16, 256), (5, 384), (32, 128), (40, 512)])
def test_matrix_core_attention_equals_the_lane_kernel(heads, rank):
    """the same bf16 weights and cached latents through both attention kernels: portions whose 32-row tiles cut through tokens, a mixed batch,
    decoding, contexts across page borders, and the split-keys form.  The two differ by summation order and the two-term rounding of q' and p only."""
    d = small_desc("bf16", width=64, budget_tokens=2048, layers=[plain_layer(heads=heads, dim=8, vdim=8, kv_rank=rank, scale=1.5), moe_layer(heads=heads, kv_rank=rank, dim=4)])
    t = so.random_tensors(d, heads)
    tens = {k: v.astype(np.float32) for k, v in t.items()}
    fast, slow = SlotEngine(desc=d, tensors=tens), SlotEngine(desc=d, tensors=tens)
    slow.model.set_option("attn.mfma", 0)
    a, b, c = tokens(d, 200, 1), tokens(d, 75, 2), tokens(d, 9, 3)
    want = so.forward(d, t, a)[[0, 1, 69, 130, 131, 199]]
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
    check(outs[0][[6, 7]], so.forward(d, t, b)[[3, 74]], "bf16")
    fast.close(); slow.close()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_few_row_kernel_equals_the_matrix_core_tiles(dtype):
    """steps of few rows stream the weights through the few-row kernel, larger ones take the matrix-core tiles: the same steps through both"""
    d = small_desc(dtype, layers=[moe_layer(experts=6, top=3), plain_layer(), moe_layer()])
    t = so.random_tensors(d, 21)
    tens = {k: v.astype(np.float32) for k, v in t.items()}
    few, tiles = SlotEngine(desc=d, tensors=tens), SlotEngine(desc=d, tensors=tens)
    tiles.model.set_option("stack.gemv", 0)
    a, b = tokens(d, 40, 1), tokens(d, 17, 2)
    outs = []
    for eng in (few, tiles):
        o = [eng.step([("a", a[:1], [0])])]                                        # one row
        o.append(eng.step([("a", a[1:3], [0, 1]), ("b", b[:1], [0])]))             # three rows, two slots
        o.append(eng.step([("a", a[3:12], list(range(9))), ("b", b[1:8], [6])]))   # sixteen rows
        o.append(eng.step([("a", a[12:], [27]), ("b", b[8:], [8])]))               # beyond: tiles in both engines
        outs.append(np.concatenate(o))
    assert np.abs(outs[0] - outs[1]).max() / np.abs(outs[1]).max() < (1e-5 if dtype == "fp32" else 3e-4)
    check(outs[0][[0, 1, 2] + list(range(4, 13))], so.forward(d, t, a)[:12], dtype)      # (row 3 is b's first token)
    few.close(); tiles.close()
