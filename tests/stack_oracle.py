"""A plain, slow restatement of the layered (Zakusun) model in numpy float64 — test infrastructure only, one function per mechanism.

Notation: x[t] is the residual stream of token t (t counts from 0 in its sequence), W the width.  Every function takes whole
sequences and loops over tokens and keys where that keeps the equation visible; nothing here is shared with tinygpt_amd/.
"""
import numpy as np


def position_vector(p, width):
    """v[2i] = sin(p / 10000^(2i/width)), v[2i+1] = cos(same angle)"""
    v = np.zeros(width)
    for c in range(width):
        ang = p * 10000.0 ** (-2.0 * (c // 2) / width)
        v[c] = np.cos(ang) if c % 2 else np.sin(ang)
    return v


def grouped_rms_norm(x, weight, groups, eps):
    """x split into `groups` consecutive equal parts; each part / sqrt(mean(part^2) + eps); then * weight"""
    out = np.empty_like(x)
    n = x.shape[-1] // groups
    for g in range(groups):
        part = x[..., g * n:(g + 1) * n]
        out[..., g * n:(g + 1) * n] = part / np.sqrt((part * part).mean(-1, keepdims=True) + eps)
    return out * weight


def input_convolution(h, filt):
    """h[t] + sum_j filt[:, j] * h[t - (taps - 1) + j], rows before the sequence's start are zero.  h: [T][W], filt: [W][taps]"""
    T, taps = h.shape[0], filt.shape[1]
    out = h.copy()
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += filt[:, j] * h[s]
    return out


def latent_attention(h, w, heads, dim, vdim, rank, scale, eps):
    """h: [T][W] (the mixer's input).  w: q, dkv, dkv.norm, uk, uv, sink, g, o.  Causal; softmax denominators also hold exp(sink[head])."""
    T = h.shape[0]
    q = h @ w["q"].T
    c = h @ w["dkv"].T
    c = c / np.sqrt((c * c).mean(-1, keepdims=True) + eps) * w["dkv.norm"]
    k = c @ w["uk"].T
    v = c @ w["uv"].T
    gate = 1.0 / (1.0 + np.exp(-(h @ w["g"].T)))
    mixed = np.zeros((T, heads * vdim))
    for t in range(T):
        for hd in range(heads):
            s = k[:t + 1, hd * dim:(hd + 1) * dim] @ q[t, hd * dim:(hd + 1) * dim] * scale      # scores against keys 0 .. t
            m = max(s.max(), w["sink"][hd])
            e = np.exp(s - m)
            p = e / (e.sum() + np.exp(w["sink"][hd] - m))
            mixed[t, hd * vdim:(hd + 1) * vdim] = p @ v[:t + 1, hd * vdim:(hd + 1) * vdim]
    return (mixed * gate) @ w["o"].T


def route(h, w_router, b_router, top):
    """logits = W h + b; the `top` largest; weights = softmax over those logits alone.  Returns (expert ids, weights) per token."""
    z = h @ w_router.T + b_router
    ids = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zs = np.take_along_axis(z, ids, -1)
    e = np.exp(zs - zs.max(-1, keepdims=True))
    return ids, e / e.sum(-1, keepdims=True)


def expert(h, gate_w, up_w, down_w, limit):
    g = np.minimum(gate_w @ h, limit)
    u = np.clip(up_w @ h, -limit, limit)
    return down_w @ (g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0))


def mixture_of_experts(h, w, n_experts, top, limit):
    ids, pw = route(h, w["router"], w["router.b"], top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += pw[t, j] * expert(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)
    return out


def depth_average(results, weights):
    """sum_j weights[j] * results[j] over the embedding output and every layer result so far"""
    return sum(weights[j] * results[j] for j in range(len(results)))


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(desc, tensors, tokens, streams=None):
    """logits [T][vocab] of one whole sequence.  desc: tinygpt_amd.desc.StackDesc (sizes only); tensors: name -> float64 array."""
    W, T = desc.width, len(tokens)
    x = np.stack([tensors["embed"][tok] + position_vector(p, W) for p, tok in enumerate(tokens)])
    results = [x]
    for i, l in enumerate(desc.layers):
        p = f"l{i}."
        h = input_convolution(grouped_rms_norm(x, tensors[p + "norm1"], desc.norm_groups, desc.norm_eps), tensors[p + "canon1"])
        x = x + latent_attention(h, sub(tensors, p + "mix."), l.heads, l.dim, l.vdim, l.kv_rank, l.scale, desc.norm_eps)
        if l.mlp == "moe":
            h = input_convolution(grouped_rms_norm(x, tensors[p + "norm2"], desc.norm_groups, desc.norm_eps), tensors[p + "canon2"])
            x = x + mixture_of_experts(h, sub(tensors, p + "mlp."), l.experts, l.top, l.limit)
        results.append(x)
        x = depth_average(results, tensors[p + "dwa"])
        if streams is not None:
            streams.append(x.copy())
    xn = grouped_rms_norm(x, tensors["final.norm"], desc.norm_groups, desc.norm_eps)
    return xn @ tensors["embed"].T * desc.logit_scale


def random_tensors(desc, seed, sink_scale=2.0, router_scale=1.0):
    """weights as float64 arrays holding bf16-representable values (so that 16-bit storage rounds nothing); sinks and router logits spread wide
    enough that a missing sink term or a wrong expert shows in the logits"""
    rng = np.random.default_rng(seed)

    def bf16(a):
        b = np.asarray(a, dtype=np.float32).view(np.uint32)
        b = ((b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
        return b.view(np.float32).astype(np.float64)

    out = {}
    for name, shape in desc.tensor_shapes().items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2") or name in ("final.norm",) or name.endswith("dkv.norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "sink":
            a = sink_scale * rng.standard_normal(shape)
        elif leaf == "dwa":
            a = np.full(shape, 1.0 / shape[0]) + 0.2 * rng.standard_normal(shape)
        elif leaf in ("canon1", "canon2"):
            a = 0.4 * rng.standard_normal(shape)
        elif leaf == "b" or leaf == "router":
            a = router_scale * rng.standard_normal(shape) / (1.0 if leaf == "b" else np.sqrt(shape[-1]) / 3.0)
        elif name == "embed":
            a = rng.standard_normal(shape)
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = bf16(a)
    return out
