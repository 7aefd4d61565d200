"""A plain, slow restatement of the Modepel design in numpy float64 — test infrastructure only, one function per mechanism.

A model is (cfg, w): cfg the parsed config.json (width, vocab, norm.eps, layers[type, mixer, mlp]), w a dict of checkpoint name -> array.
x[t] is the residual stream of token t (t counts from 0 in its sequence).  Every function takes a whole sequence and loops over tokens and keys
where that keeps the equation visible; nothing here is shared with tinygpt_amd/.
"""
import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def scalar_rms_norm(x, g, eps):
    """every row divided by sqrt(mean(row^2) + eps), times the single number g"""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * g


def rotate(v, pos, dims, base):
    """the first `dims` coordinates of v in pairs (i, i + dims / 2), turned by the angle pos * base^(-2i / dims); the rest unchanged"""
    out = v.copy()
    half = dims // 2
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = np.cos(ang), np.sin(ang)
        out[i] = v[i] * c - v[i + half] * s
        out[i + half] = v[i + half] * c + v[i] * s
    return out


def attention_values(h, w, m):
    """v = W_v h + b: what a value-mixing layer hands to the later ones (before its own mixing)"""
    return h @ w["v"].T + w["v.b"]


def attention(h, w, m, v_first=None):
    """h: [T][W].  w: q, q.b, k, k.b, v, v.b, vmix, g, o.  m: heads, kv_heads, dim, vdim, rot{dims, base}, scale, v_mix.
    Causal; the softmax denominator holds one more term, exp(0), that carries no value.  v_first: the values of the first value-mixing
    layer for the same tokens (None: this layer mixes nothing)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w["q"].T + w["q.b"]
    k = h @ w["k"].T + w["k.b"]
    v = h @ w["v"].T + w["v.b"]
    if v_first is not None:
        lam = float(w["vmix"])
        v = (1.0 - lam) * v + lam * v_first
    for t in range(T):
        for a in range(H):
            q[t, a * D:(a + 1) * D] = rotate(q[t, a * D:(a + 1) * D], t, m["rot"]["dims"], m["rot"]["base"])
        for a in range(G):
            k[t, a * D:(a + 1) * D] = rotate(k[t, a * D:(a + 1) * D], t, m["rot"]["dims"], m["rot"]["base"])
    mixed = np.zeros((T, H * V))
    for t in range(T):
        for a in range(H):
            kv = a // (H // G)
            s = k[:t + 1, kv * D:(kv + 1) * D] @ q[t, a * D:(a + 1) * D] * m["scale"]
            mx = max(s.max(), 0.0)
            e = np.exp(s - mx)
            p = e / (np.exp(-mx) + e.sum())
            mixed[t, a * V:(a + 1) * V] = p @ v[:t + 1, kv * V:(kv + 1) * V]
    return (mixed * sigmoid(h @ w["g"].T)) @ w["o"].T


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def mlstm(h, w, m, eps, state=None):
    """matrix memory with a running maximum.  h: [T][W].  w: q, k, v, g, o, norm, i, i.b, f, f.b.  m: heads, dim, vdim, gate_cap.
    state: (S [H][D][V], n [H][D], mx [H]) carried in, zeros when None; returns (output, state)."""
    T = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w["q"].T) * D ** -0.5
    k = h @ w["k"].T
    v = h @ w["v"].T
    ig = cap * np.tanh((h @ w["i"].T + w["i.b"]) / cap)
    fg = log_sigmoid(cap * np.tanh((h @ w["f"].T + w["f.b"]) / cap))
    if state is None:
        state = (np.zeros((H, D, V)), np.zeros((H, D)), np.zeros(H))
    S, n, mx = (a.copy() for a in state)
    out = np.zeros((T, H * V))
    for t in range(T):
        for a in range(H):
            qt, kt, vt = q[t, a * D:(a + 1) * D], k[t, a * D:(a + 1) * D], v[t, a * V:(a + 1) * V]
            m_new = max(fg[t, a] + mx[a], ig[t, a])
            keep, take = np.exp(fg[t, a] + mx[a] - m_new), np.exp(ig[t, a] - m_new)
            S[a] = keep * S[a] + take * np.outer(kt, vt)
            n[a] = keep * n[a] + take * kt
            mx[a] = m_new
            o = S[a].T @ qt / (max(abs(n[a] @ qt), np.exp(-m_new)) + 1e-6)
            out[t, a * V:(a + 1) * V] = o / np.sqrt((o * o).mean() + eps)
    return (out * w["norm"] * sigmoid(h @ w["g"].T)) @ w["o"].T, (S, n, mx)


def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with N(u) = u / sqrt(mean(u^2) + eps) over a token's values"""
    N = lambda u: u / np.sqrt((u * u).mean(-1, keepdims=True) + eps)
    return coef[0] * N(z) + coef[1] * N(z * z) + coef[2] * N(z * z * z) + coef[3]


def dense_ff(h, w, eps):
    return poly_norm(h @ w["up"].T, w["act"], eps) @ w["down"].T


def gated_expert(h, gate, up, down):
    z = h @ gate.T
    return (z * sigmoid(z) * (h @ up.T)) @ down.T


def route(h, w_router, correction, r):
    """-> (chosen [T][top], weights [T][top]).  r: experts, identity, top, scale, groups{count, keep}.  Scores are a softmax over all router outputs;
    the choice is made on scores + correction inside the best groups, the weights are the plain scores times r.scale."""
    z = h @ w_router.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    T, n = s.shape
    per = n // r["groups"]["count"]
    chosen = np.zeros((T, r["top"]), int)
    weights = np.zeros((T, r["top"]))
    for t in range(T):
        c = s[t] + correction
        best = [c[g * per:(g + 1) * per].max() for g in range(r["groups"]["count"])]
        kept = sorted(range(len(best)), key=lambda g: (-best[g], g))[:r["groups"]["keep"]]
        allowed = [e for e in range(n) if e // per in kept]
        pick = sorted(allowed, key=lambda e: (-c[e], e))[:r["top"]]
        chosen[t] = pick
        weights[t] = s[t, pick] * r["scale"]
    return chosen, weights


def moe_ff(h, w, f):
    """w: router, correction, e<j>.gate|up|down, shared.gate|up|down|sg.  Router outputs experts .. experts + identity - 1 hand the input through."""
    r = f["router"]
    chosen, weights = route(h, w["router"], w["correction"], r)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t], weights[t]):
            if e >= r["experts"]:
                out[t] += wt * h[t]
            else:
                out[t] += wt * gated_expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if f.get("shared"):
        out += sigmoid(h @ w["shared.sg"].T) * gated_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


def sub(w, prefix):
    return {k[len(prefix):]: np.asarray(v, np.float64) for k, v in w.items() if k.startswith(prefix)}


def forward(cfg, w, ids, states=None, residuals=None):
    """logits [T][vocab] of one whole sequence.  states: per-layer recurrent state carried in (None: a new sequence; only the recurrent
    layers can continue this way).  residuals: a list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = np.asarray(w["embed"], np.float64)[np.asarray(ids)]
    v_first = None
    new_states = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        g = lambda name: float(np.asarray(w[p + name], np.float64))
        h = scalar_rms_norm(x, g("norm1"), eps)
        mw = sub(w, p + "mix.")
        if L["type"] == "attention":
            mixes = bool(L["mixer"].get("v_mix"))
            y = attention(h, mw, L["mixer"], v_first if mixes else None)
            if mixes and v_first is None:
                v_first = attention_values(h, mw, L["mixer"])
            new_states.append(None)
        elif L["type"] == "mlstm":
            y, st = mlstm(h, mw, L["mixer"], eps, states[i] if states else None)
            new_states.append(st)
        else:
            raise ValueError(L["type"])
        x = x + scalar_rms_norm(y, g("norm1b"), eps)
        f = L.get("mlp")
        if f is not None:
            h = scalar_rms_norm(x, g("norm2"), eps)
            fw = sub(w, p + "mlp.")
            y = dense_ff(h, fw, eps) if f["kind"] == "dense" else moe_ff(h, fw, f)
            x = x + scalar_rms_norm(y, g("norm2b"), eps)
        if residuals is not None:
            residuals.append(x.copy())
    x = scalar_rms_norm(x, float(np.asarray(w["final.norm"], np.float64)), eps)
    return x @ np.asarray(w["head"], np.float64).T, new_states


def tensor_shapes(cfg):
    """checkpoint name -> shape"""
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"])}
    for i, L in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.", L["mixer"], L.get("mlp")
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if f is not None else ()):
            out[p + n] = ()
        if L["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, W), p + "mix.q.b": (H * D,), p + "mix.k": (G * D, W), p + "mix.k.b": (G * D,), p + "mix.v": (G * V, W),
                        p + "mix.v.b": (G * V,), p + "mix.g": (H * V, W), p + "mix.o": (W, H * V)})
            if m.get("v_mix"):
                out[p + "mix.vmix"] = ()
        else:
            H, D, V = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (H * D, W), p + "mix.v": (H * V, W), p + "mix.g": (H * V, W), p + "mix.o": (W, H * V),
                        p + "mix.norm": (H * V,), p + "mix.i": (H, W), p + "mix.i.b": (H,), p + "mix.f": (H, W), p + "mix.f.b": (H,)})
        if f is None:
            continue
        if f["kind"] == "dense":
            out.update({p + "mlp.up": (f["ff"], W), p + "mlp.down": (W, f["ff"]), p + "mlp.act": (4,)})
        else:
            r = f["router"]
            for e in range(r["experts"]):
                out.update({p + f"mlp.e{e}.gate": (f["expert"]["ff"], W), p + f"mlp.e{e}.up": (f["expert"]["ff"], W), p + f"mlp.e{e}.down": (W, f["expert"]["ff"])})
            out.update({p + "mlp.router": (r["experts"] + r["identity"], W), p + "mlp.correction": (r["experts"] + r["identity"],)})
            if f.get("shared"):
                sf = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf), p + "mlp.shared.sg": (1, W)})
    out["final.norm"] = ()
    out["head"] = (cfg["vocab"], W)
    return out


def bf16_round(a):
    """round-to-nearest-even onto the bfloat16 grid, so that every storage dtype of the library holds the same numbers"""
    u = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def random_tensors(cfg, seed=0, overrides=None):
    """weights on the bfloat16 grid, scaled so that every mechanism matters: projections ~ 1 / sqrt(inputs), norm numbers near 1, gate biases spread"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if len(shape) == 2:
            v = rng.standard_normal(shape) / np.sqrt(shape[1])
            if name.endswith("mlp.router"):
                v *= 4.0
            if name in ("embed",):
                v = rng.standard_normal(shape)
        elif leaf in ("norm1", "norm2", "final"):
            v = rng.uniform(0.7, 1.3, shape)
        elif name == "final.norm":
            v = rng.uniform(0.7, 1.3, shape)
        elif leaf in ("norm1b", "norm2b"):
            v = rng.uniform(0.3, 0.8, shape)
        elif leaf == "vmix":
            v = rng.uniform(0.2, 0.6, shape)
        elif leaf == "act":
            v = rng.uniform(-1.0, 1.0, shape)
        elif leaf == "correction":
            v = rng.uniform(-0.2, 0.2, shape)
        elif name.endswith("mix.norm"):
            v = rng.uniform(0.5, 1.5, shape)
        elif name.endswith("f.b"):
            v = rng.uniform(1.0, 4.0, shape)
        elif name.endswith("i.b"):
            v = rng.uniform(-2.0, 1.0, shape)
        else:
            v = rng.standard_normal(shape) * 0.3
        out[name] = bf16_round(v)
    for k, v in (overrides or {}).items():
        out[k] = bf16_round(v)
    return out
