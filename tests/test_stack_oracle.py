"""CPU checks of the layered model's test oracle and of its configuration reader (no GPU): the oracle's mechanisms against closed forms, so that the
GPU tests compare the library with something that is itself pinned."""
import numpy as np
import pytest

import stack_oracle as so
from tinygpt_amd.desc import LayerDesc, StackDesc, stack_desc_from_config, is_stack_config


def test_position_vector_interleaves_sin_and_cos():
    v = so.position_vector(3, 8)
    assert np.allclose(v[0], np.sin(3.0)) and np.allclose(v[1], np.cos(3.0))
    assert np.allclose(v[6], np.sin(3.0 * 10000.0 ** (-6 / 8))) and np.allclose(v[7], np.cos(3.0 * 10000.0 ** (-6 / 8)))
    assert np.allclose(so.position_vector(0, 6), [0, 1, 0, 1, 0, 1])


def test_grouped_norm_normalises_each_part_alone():
    x = np.array([[3.0, 4.0, 0.0, 10.0]])
    y = so.grouped_rms_norm(x, np.ones(4), 2, 0.0)
    assert np.allclose(y, [[3 / np.sqrt(12.5), 4 / np.sqrt(12.5), 0.0, 10 / np.sqrt(50.0)]])
    assert np.allclose(so.grouped_rms_norm(x, np.ones(4), 1, 0.0), x / np.sqrt((x * x).mean()))


def test_convolution_is_causal_and_adds_the_input():
    h = np.arange(12.0).reshape(6, 2)
    f = np.array([[1.0, 0.0, 0.0], [0.0, 0.0, 2.0]])      # channel 0 reads two rows back, channel 1 doubles the current row
    y = so.input_convolution(h, f)
    assert np.allclose(y[:, 0], h[:, 0] + np.concatenate([[0, 0], h[:-2, 0]]))
    assert np.allclose(y[:, 1], 3 * h[:, 1])


def test_sink_only_lowers_the_weights():
    rng = np.random.default_rng(0)
    W, H, dim, vd, R = 8, 2, 4, 3, 5
    w = {"q": rng.standard_normal((H * dim, W)), "dkv": rng.standard_normal((R, W)), "dkv.norm": np.ones(R), "uk": rng.standard_normal((H * dim, R)),
         "uv": rng.standard_normal((H * vd, R)), "sink": np.array([-50.0, -50.0]), "g": np.zeros((H * vd, W)), "o": np.eye(W, H * vd)}
    h = rng.standard_normal((1, W))
    # one token, a sink of no weight, a gate of 1/2: the output is half the token's own value vector
    c = h @ w["dkv"].T
    c = c / np.sqrt((c * c).mean() + 1e-6)
    want = 0.5 * (c @ w["uv"].T) @ w["o"].T
    assert np.allclose(so.latent_attention(h, w, H, dim, vd, R, 0.3, 1e-6), want)
    w["sink"] = np.array([50.0, 50.0])      # a heavy sink takes all the weight
    assert np.abs(so.latent_attention(h, w, H, dim, vd, R, 0.3, 1e-6)).max() < 1e-12


def test_router_weights_are_a_softmax_over_the_chosen():
    z = np.array([[0.0, 2.0, 1.0, -1.0]])
    ids, w = so.route(np.ones((1, 1)), z.T, np.zeros(4), 2)
    assert ids.tolist() == [[1, 2]]
    assert np.allclose(w, [[np.e / (np.e + 1), 1 / (np.e + 1)]])


def test_expert_clamps():
    gw, uw, dw = np.array([[10.0]]), np.array([[-10.0]]), np.array([[1.0]])
    y = so.expert(np.array([1.0]), gw, uw, dw, 2.0)      # gate 10 -> 2, up -10 -> -2
    assert np.allclose(y, 2.0 / (1 + np.exp(-3.404)) * (-1.0))


def test_config_reader_takes_every_size_from_the_file():
    cfg = {"architecture": "Zakusun", "canon": {"taps": 3}, "logit_scale": 0.25, "norm": {"eps": 1e-5, "groups": 4}, "vocab": 77, "width": 48,
           "layers": [{"type": "latent_attention", "mixer": {"dim": 12, "heads": 3, "kv_rank": 20, "scale": 0.5, "vdim": 8}, "mlp": None},
                      {"type": "latent_attention", "mixer": {"dim": 6, "heads": 5, "kv_rank": 10, "scale": 0.1, "vdim": 4},
                       "mlp": {"kind": "moe", "expert": {"ff": 24, "limit": 3.0}, "router": {"experts": 6, "top": 2}}}]}
    assert is_stack_config(cfg) and not is_stack_config({"model_type": "llama"})
    d = stack_desc_from_config(cfg, "fp32", max_seqs=3, max_ctx=256, budget_tokens=512)
    assert (d.width, d.vocab, d.canon_taps, d.norm_groups, d.logit_scale, d.norm_eps) == (48, 77, 3, 4, 0.25, 1e-5)
    assert d.layers[0].mlp is None and d.layers[1].mlp == "moe" and (d.layers[1].experts, d.layers[1].top, d.layers[1].ff, d.layers[1].limit) == (6, 2, 24, 3.0)
    shapes = d.tensor_shapes()
    assert "l0.norm2" not in shapes and "l0.canon2" not in shapes and shapes["l1.canon2"] == (48, 3)
    assert shapes["l1.mix.uk"] == (30, 10) and shapes["l1.dwa"] == (3,) and shapes["l1.mlp.e5.down"] == (48, 24)
    sd, layers = d.to_c()
    assert sd.layers == 2 and layers[1].experts == 6 and abs(layers[0].scale - 0.5) < 1e-7
    with pytest.raises(ValueError):
        stack_desc_from_config(dict(cfg, architecture="Other"))


def test_oracle_prefix_property():
    """a causal model: the logits of a prefix do not change when tokens follow"""
    d = StackDesc(width=16, vocab=19, canon_taps=3, norm_groups=2, logit_scale=0.5,
                  layers=[LayerDesc(heads=2, dim=4, vdim=3, kv_rank=6, scale=0.5, mlp="moe", experts=3, top=2, ff=8, limit=1.5)])
    t = so.random_tensors(d, 1)
    toks = [3, 1, 4, 1, 5, 9, 2]
    full = so.forward(d, t, toks)
    assert np.allclose(so.forward(d, t, toks[:4]), full[:4], atol=1e-12)
