"""Closed-form checks of the plain Modepel oracle (tests/modepel_oracle.py), so that the GPU comparison rests on something: every mechanism on inputs
whose result can be written down, and a demonstration that each mechanism moves the logits by far more than the comparison's tolerance.  CPU only."""
import copy

import numpy as np

import modepel_oracle as mo


def test_scalar_norm_and_poly_norm():
    x = np.array([[3.0, -4.0, 0.0, 0.0]])
    assert np.allclose(mo.scalar_rms_norm(x, 2.0, 0.0), x / 2.5 * 2.0)
    z = np.array([[1.0, -1.0, 1.0, -1.0]])                # N(z) = z, N(z^2) = 1, N(z^3) = z
    assert np.allclose(mo.poly_norm(z, [0.5, 2.0, 0.25, -1.0], 0.0), 0.75 * z + 2.0 - 1.0)


def test_rotation_pairs_and_angles():
    v = np.arange(1.0, 9.0)
    assert np.allclose(mo.rotate(v, 0, 4, 100.0), v)
    r = mo.rotate(v, 3, 4, 100.0)
    assert np.allclose(r[4:], v[4:])                       # dimensions beyond rot.dims pass unchanged
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5                     # pair (0, 2) turns by 3, pair (1, 3) by 3 / 10
    assert np.allclose([r[0], r[2]], [v[0] * np.cos(a0) - v[2] * np.sin(a0), v[2] * np.cos(a0) + v[0] * np.sin(a0)])
    assert np.allclose([r[1], r[3]], [v[1] * np.cos(a1) - v[3] * np.sin(a1), v[3] * np.cos(a1) + v[1] * np.sin(a1)])


def tiny_attention(W=4):
    m = {"heads": 2, "kv_heads": 1, "dim": 2, "vdim": 3, "rot": {"dims": 2, "base": 10.0}, "scale": 0.5, "v_mix": False}
    rng = np.random.default_rng(0)
    w = {"q": rng.standard_normal((4, W)), "q.b": rng.standard_normal(4), "k": rng.standard_normal((2, W)), "k.b": rng.standard_normal(2),
         "v": rng.standard_normal((3, W)), "v.b": rng.standard_normal(3), "g": rng.standard_normal((6, W)), "o": rng.standard_normal((W, 6))}
    return m, w


def test_attention_first_token_is_a_two_way_softmax_with_the_sink():
    m, w = tiny_attention()
    h = np.array([[0.3, -1.0, 0.7, 0.2]])
    q, k, v = h @ w["q"].T + w["q.b"], h @ w["k"].T + w["k.b"], h @ w["v"].T + w["v.b"]
    gate = mo.sigmoid(h @ w["g"].T)
    heads = []
    for a in range(2):
        s = (q[0, 2 * a:2 * a + 2] @ k[0]) * 0.5
        heads.append(np.exp(s) / (1.0 + np.exp(s)) * v[0])     # position 0 turns nothing; both query heads read the one key head
    want = (np.concatenate(heads) * gate[0]) @ w["o"].T
    assert np.allclose(mo.attention(h, w, m)[0], want)


def test_value_mixing_uses_the_first_layers_values():
    m, w = tiny_attention()
    h = np.random.default_rng(1).standard_normal((5, 4))
    vf = np.random.default_rng(2).standard_normal((5, 3))
    w["vmix"] = 0.25
    mixed = mo.attention(h, w, m, vf)
    w2 = dict(w); w2["v"] = np.zeros_like(w["v"]); w2["v.b"] = np.zeros_like(w["v.b"])
    only_first = mo.attention(h, w2, m, vf)                 # lambda * v_first alone
    w3 = dict(w); w3["vmix"] = 0.0
    only_own = mo.attention(h, w3, m, np.zeros_like(vf))
    assert np.allclose(mixed, 0.75 * only_own + only_first)  # the output is linear in the values


def test_mlstm_first_steps_closed_form():
    m = {"heads": 1, "dim": 2, "vdim": 2, "gate_cap": 15.0}
    W = 3
    rng = np.random.default_rng(3)
    w = {n: rng.standard_normal(s) for n, s in {"q": (2, W), "k": (2, W), "v": (2, W), "g": (2, W), "i": (1, W), "f": (1, W)}.items()}
    w.update({"i.b": np.array([0.3]), "f.b": np.array([2.0]), "norm": np.array([1.5, 0.5]), "o": np.eye(W)[:, :2]})
    h = rng.standard_normal((2, W))
    q, k, v = h @ w["q"].T / np.sqrt(2.0), h @ w["k"].T, h @ w["v"].T
    i = 15.0 * np.tanh((h @ w["i"].T + 0.3) / 15.0)[:, 0]
    f = mo.log_sigmoid(15.0 * np.tanh((h @ w["f"].T + 2.0) / 15.0))[:, 0]
    # token 0: the state was zero and the maximum starts at 0
    m0 = max(f[0] + 0.0, i[0])
    S0, n0 = np.exp(i[0] - m0) * np.outer(k[0], v[0]), np.exp(i[0] - m0) * k[0]
    o0 = S0.T @ q[0] / (max(abs(n0 @ q[0]), np.exp(-m0)) + 1e-6)
    m1 = max(f[1] + m0, i[1])
    S1 = np.exp(f[1] + m0 - m1) * S0 + np.exp(i[1] - m1) * np.outer(k[1], v[1])
    n1 = np.exp(f[1] + m0 - m1) * n0 + np.exp(i[1] - m1) * k[1]
    o1 = S1.T @ q[1] / (max(abs(n1 @ q[1]), np.exp(-m1)) + 1e-6)
    want = np.stack([o / np.sqrt((o * o).mean() + 1e-5) for o in (o0, o1)]) * w["norm"] * mo.sigmoid(h @ w["g"].T)
    got, st = mo.mlstm(h, w, m, 1e-5)
    assert np.allclose(got[:, :2], want)
    # carried state: two tokens at once = one token, then one more
    a, s1 = mo.mlstm(h[:1], w, m, 1e-5)
    b, s2 = mo.mlstm(h[1:], w, m, 1e-5, s1)
    assert np.allclose(np.concatenate([a, b]), got) and np.allclose(s2[0], st[0]) and np.allclose(s2[2], st[2])


def test_router_groups_correction_and_identity():
    r = {"experts": 4, "identity": 2, "top": 2, "scale": 1.5, "groups": {"count": 3, "keep": 1}}
    wr = np.eye(6)
    h = np.array([[0.0, 0.0, 3.0, 2.9, 0.0, 2.95]])        # scores rank 2 > 5 > 3; groups are (0, 1), (2, 3), (4, 5)
    chosen, weights = mo.route(h, wr, np.zeros(6), r)
    assert chosen[0].tolist() == [2, 3]                     # only the best group's members are eligible, although output 5 scores higher than 3
    s = np.exp(h[0]) / np.exp(h[0]).sum()
    assert np.allclose(weights[0], s[[2, 3]] * 1.5)         # not renormalised
    chosen, weights = mo.route(h, wr, np.array([0, 0, -1.0, 0, 0, 0]), r)
    assert chosen[0].tolist() == [5, 4]                     # the correction moves the choice (group 2 now leads) ...
    assert np.allclose(weights[0], s[[5, 4]] * 1.5)         # ... but not the weights
    r2 = dict(r, groups={"count": 3, "keep": 3})
    assert mo.route(h, wr, np.zeros(6), r2)[0][0].tolist() == [2, 5]
    # identity outputs hand the input through
    f = {"kind": "moe", "expert": {"ff": 3}, "router": dict(r, top=1, groups={"count": 1, "keep": 1}), "shared": None}
    w = {"router": wr, "correction": np.zeros(6)}
    for e in range(4):
        w.update({f"e{e}.gate": np.ones((3, 6)), f"e{e}.up": np.ones((3, 6)), f"e{e}.down": np.ones((6, 3))})
    h5 = np.array([[0.0, 0.0, 0.0, 0.0, 0.0, 4.0]])
    s5 = np.exp(4.0) / (np.exp(4.0) + 5.0)
    assert np.allclose(mo.moe_ff(h5, w, f), 1.5 * s5 * h5)


def small_cfg():
    attn = {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "rot": {"dims": 4, "base": 100.0}, "scale": 0.6, "v_mix": True},
            "mlp": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 4, "identity": 2, "top": 2, "scale": 1.5, "groups": {"count": 2, "keep": 1}}, "shared": {"ff": 10}}}
    rec = {"type": "mlstm", "mixer": {"heads": 2, "dim": 6, "vdim": 8, "gate_cap": 15.0}, "mlp": {"kind": "dense", "ff": 20}}
    return {"architecture": "Modepel", "width": 16, "vocab": 41, "norm": {"eps": 1e-5}, "layers": [rec, attn, copy.deepcopy(attn)]}


def test_every_mechanism_moves_the_logits():
    """a comparison against this oracle would not see a mechanism whose contribution were negligible: switching each one off changes these logits by far more
    than 1e-4 of their size"""
    cfg = small_cfg()
    w = mo.random_tensors(cfg, 5)
    ids = np.random.default_rng(6).integers(0, 41, 24)
    base, _ = mo.forward(cfg, w, ids)

    def moved(cfg2=None, **over):
        got, _ = mo.forward(cfg2 or cfg, {**w, **over}, ids)
        return np.abs(got - base).max() / np.abs(base).max()

    assert moved(**{"l2.mix.vmix": np.float32(0.0)}) > 1e-2                                  # value mixing
    assert moved(**{"l1.mix.g": np.zeros_like(w["l1.mix.g"])}) > 1e-2                        # output gate
    assert moved(**{"l1.mlp.correction": np.zeros_like(w["l1.mlp.correction"])}) > 1e-3      # the correction changes choices
    assert moved(**{"l0.mlp.act": np.array([1, 0, 0, 0], np.float32)}) > 1e-2                # PolyNorm's higher powers and offset
    assert moved(**{"l0.mix.f.b": w["l0.mix.f.b"] - 8.0}) > 1e-2                             # the forget gate (memory of earlier tokens)
    assert moved(**{"l1.norm1b": np.float32(1.0)}) > 1e-2                                    # the norm behind a sublayer
    for path, val in (("rot", {"dims": 8, "base": 100.0}), ("scale", 0.3)):
        c2 = copy.deepcopy(cfg); c2["layers"][1]["mixer"][path] = val
        assert moved(c2) > 1e-3, path
    c2 = copy.deepcopy(cfg); c2["layers"][1]["mlp"]["router"]["groups"] = {"count": 1, "keep": 1}
    assert moved(c2) > 1e-3                                                                  # the group limit
    c2 = copy.deepcopy(cfg); c2["layers"][2]["mlp"]["shared"] = None
    assert moved(c2) > 1e-2                                                                  # the shared expert
    # the sink: without it the one-token softmax is exactly 1, with it e^s / (1 + e^s)
    m, wa = tiny_attention()
    h = np.array([[0.3, -1.0, 0.7, 0.2]])
    v = h @ wa["v"].T + wa["v.b"]
    no_sink = (np.concatenate([v[0], v[0]]) * mo.sigmoid(h @ wa["g"].T)[0]) @ wa["o"].T
    assert np.abs(mo.attention(h, wa, m)[0] - no_sink).max() > 1e-2
