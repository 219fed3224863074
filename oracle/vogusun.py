"""Plain, slow float64 restatement of the Vogusun design, one function per mechanism, token by token where the mechanism is
sequential.  Test infrastructure only: numpy, no kernels, no code shared with the product path.

Notation: h [n, width] the rows of ONE sequence in order (row p is position p); weights as the checkpoint stores them
([out, in]); w maps the names below '<layer>.mix.' / '<layer>.mlp.' to arrays."""
import math

import numpy as np


def f64(a):
    return np.asarray(a, np.float64)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dyt_norm(x, alpha, w, b):
    """the norm without statistics: a squashed copy of the row, scaled and shifted per channel"""
    return np.tanh(float(alpha) * f64(x)) * f64(w) + f64(b)


def unit_rms(x, w, eps):
    x = f64(x)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * f64(w)


# -- rotary positions -----------------------------------------------------------------------------------------------------
def rotary_frequencies(rot):
    """-> (frequency per pair [dims / 2], magnitude of cos and sin)"""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])
    turn = lambda t: dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo, hi = max(math.floor(turn(float(sc["fast"]))), 0), min(math.ceil(turn(float(sc["slow"]))), dims - 1)
    out = np.empty_like(f)
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x, pos, rot, layout):
    """x [heads, dim] of the token at position pos; layout 'pairs': (2i, 2i+1), 'halves': (i, i + dims/2).  The angle is the
    32-bit product of position and frequency."""
    dims = int(rot["dims"])
    f, mag = rotary_frequencies(rot)
    ang = (np.float32(pos) * f.astype(np.float32)).astype(np.float64)
    c, s = np.cos(ang) * mag, np.sin(ang) * mag
    out = f64(x).copy()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if layout == "pairs" else (i, i + dims // 2)
        u, v = f64(x)[:, a], f64(x)[:, b]
        out[:, a], out[:, b] = u * c[i] - v * s[i], v * c[i] + u * s[i]
    return out


# -- attention ------------------------------------------------------------------------------------------------------------
def causal_attention_rows(q, k, v, scale, sink_one=False, softcap=None):
    """q [n, H, D], k [n, G, D], v [n, G, V] -> [n, H, V]; head h reads key/value head h // (H / G)"""
    n, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((n, H, v.shape[2]))
    for i in range(n):
        for h in range(H):
            g = h // (H // G)
            s = (k[:i + 1, g] @ q[i, h]) * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            mx = max(float(s.max()), 0.0) if sink_one else float(s.max())
            e = np.exp(s - mx)
            den = e.sum() + (math.exp(-mx) if sink_one else 0.0)
            out[i, h] = (e[:, None] * v[:i + 1, g]).sum(0) / den
    return out


def attention(h, w, m, eps, kind, v_first=None):
    """kind 'attention': query/key norm, paired rotation, a sink of score 0, sigmoid gate per head.
    kind 'attention_2': biases, half-split rotation (scaled frequencies), capped scores.  m: the layer's mixer config.
    v_first: the values [n, G, V] of the first value-mixing layer (None: this layer is it, or does not mix) -> (out, values)"""
    n = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    h = f64(h)
    q, k, v = h @ f64(w["q"]).T, h @ f64(w["k"]).T, h @ f64(w["v"]).T
    if kind == "attention_2":
        q, k, v = q + f64(w["q.b"]), k + f64(w["k.b"]), v + f64(w["v.b"])
    q, k, v = q.reshape(n, H, D), k.reshape(n, G, D), v.reshape(n, G, V)
    if kind == "attention":
        q, k = unit_rms(q, w["q.norm"], eps), unit_rms(k, w["k.norm"], eps)
    layout = "pairs" if kind == "attention" else "halves"
    q = np.stack([rotate(q[p], p, m["rot"], layout) for p in range(n)])
    k = np.stack([rotate(k[p], p, m["rot"], layout) for p in range(n)])
    if m.get("v_mix") and v_first is not None:
        lam = float(np.asarray(w["vmix"], np.float64))
        v = (1.0 - lam) * v + lam * v_first
    o = causal_attention_rows(q, k, v, float(m["scale"]), sink_one=kind == "attention", softcap=m.get("softcap"))
    if kind == "attention":
        o = o * sigmoid(h @ f64(w["g"]).T)[:, :, None]
    return o.reshape(n, H * V) @ f64(w["o"]).T, v


# -- gated linear attention ---------------------------------------------------------------------------------------------------
def gla_recurrence(q, k, v, alpha):
    """q, k, alpha [n, H, D], v [n, H, V]; per head S <- diag(alpha_t) S + k_t v_t^T from S = 0, o_t = S^T q_t -> [n, H, V]"""
    n, H, D = q.shape
    V = v.shape[2]
    S = np.zeros((H, D, V))
    out = np.zeros((n, H, V))
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = np.einsum("hdv,hd->hv", S, q[t])
    return out


def gla(h, w, m, eps):
    n = h.shape[0]
    H, D, V, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    h = f64(h)
    q = (h @ f64(w["q"]).T * D ** -0.5).reshape(n, H, D)
    k = (h @ f64(w["k"]).T).reshape(n, H, D)
    v = (h @ f64(w["v"]).T).reshape(n, H, V)
    z = (h @ f64(w["a1"]).T) @ f64(w["a2"]).T + f64(w["a2.b"])
    alpha = (sigmoid(z) ** (1.0 / tau)).reshape(n, H, D)
    o = unit_rms(gla_recurrence(q, k, v, alpha), w["norm"], eps).reshape(n, H * V)
    g = h @ f64(w["g"]).T
    return (o * (g * sigmoid(g))) @ f64(w["o"]).T


# -- feed-forward -----------------------------------------------------------------------------------------------------------
def dense_ff(h, w):
    h = f64(h)
    return (gelu_tanh(h @ f64(w["gate"]).T) * (h @ f64(w["up"]).T)) @ f64(w["down"]).T


def expert_ff(h, gate, up, down, limit):
    g = np.minimum(h @ f64(gate).T, limit)
    u = np.clip(h @ f64(up).T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ f64(down).T


def moe_ff(h, w, experts, top, limit, chosen=None):
    """every token: the `top` experts of largest router logit, weighted by the softmax over those logits alone"""
    h = f64(h)
    z = h @ f64(w["router"]).T + f64(w["router.b"])
    out = np.zeros((h.shape[0], f64(w["e0.down"]).shape[0]))
    for t in range(h.shape[0]):
        idx = np.argsort(-z[t], kind="stable")[:top]
        p = np.exp(z[t, idx] - z[t, idx].max())
        p /= p.sum()
        if chosen is not None:
            chosen.append(idx.tolist())
        for e, pe in zip(idx, p):
            out[t] += pe * expert_ff(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)[0]
    return out


# -- the model --------------------------------------------------------------------------------------------------------------
def _sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def vogusun_forward(config, tensors, tokens, layer_streams=None):
    """tensors: name -> numpy array.  -> logits [n, vocab] (float64); layer_streams collects the stream after every layer"""
    eps = float(config["norm"]["eps"])
    x = f64(tensors["embed"])[list(tokens)]
    v_first = None
    for i, lc in enumerate(config["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        h = dyt_norm(x, tensors[p + "norm1.alpha"], tensors[p + "norm1"], tensors[p + "norm1.b"])
        wm = _sub(tensors, p + "mix.")
        if lc["type"] in ("attention", "attention_2"):
            mo, v = attention(h, wm, m, eps, lc["type"], v_first if m.get("v_mix") else None)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif lc["type"] == "gla":
            mo = gla(h, wm, m, eps)
        else:
            raise ValueError(lc["type"])
        ff = lc.get("mlp")
        if ff is not None:
            wf = _sub(tensors, p + "mlp.")
            if ff["kind"] == "dense":
                mo = mo + dense_ff(h, wf)
            else:
                mo = mo + moe_ff(h, wf, int(ff["router"]["experts"]), int(ff["router"]["top"]), float(ff["expert"]["limit"]))
        x = x + mo
        if layer_streams is not None:
            layer_streams.append(x)
    xn = dyt_norm(x, tensors["final.norm.alpha"], tensors["final.norm"], tensors["final.norm.b"])
    return xn @ f64(tensors["head"]).T


def bf16_values(a):
    """float32 array whose values are exactly representable in bfloat16 (round to nearest even)"""
    u = np.asarray(a, np.float32).view(np.uint32)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


def random_vogusun(rng, width=72, vocab=97, layers=("attention+dense", "gla+moe", "attention_2+dense", "attention+moe"), heads=6, kv_heads=2,
                   dim=24, vdim=16, rot_dims=None, base=10000.0, base2=50000.0, scale=None, softcap=20.0, scaling=True, v_mix=True,
                   gla_heads=3, gla_dim=20, gla_vdim=24, gla_rank=8, tau=8.0, ff=88, experts=5, top=2, expert_ff_size=24, limit=1.5,
                   eps=1e-5):
    """A small random model -> (config, tensors as float32 arrays of bf16 values).  Layer specs: '<mixer>[+dense|+moe]' with
    mixer attention / attention_2 / gla; '!mix' after an attention spec switches its value mixing off."""
    bf = bf16_values
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else 1.0 / math.sqrt(s[-1]), s))
    cfg = {"architecture": "Vogusun", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": []}
    t = {"embed": r(vocab, width, sd=1.0), "head": r(vocab, width)}

    def norm(name):
        t[name], t[name + ".b"] = bf(1 + 0.1 * rng.normal(size=width)), bf(0.1 * rng.normal(size=width))
        t[name + ".alpha"] = bf(np.float32(rng.uniform(0.4, 1.2)))
    norm("final.norm")
    for i, spec in enumerate(layers):
        kind, _, ffkind = spec.partition("+")
        mix_off = kind.endswith("!mix")
        kind = kind.replace("!mix", "")
        p = f"l{i}."
        norm(p + "norm1")
        if kind in ("attention", "attention_2"):
            rd = rot_dims if rot_dims is not None else dim
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
                 "rot": {"base": base if kind == "attention" else base2, "dims": rd}}
            if v_mix and not mix_off:
                m["v_mix"] = True
                t[p + "mix.vmix"] = bf(np.float32(rng.uniform(0.2, 0.7)))
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = r(heads * dim, width), r(kv_heads * dim, width), r(kv_heads * vdim, width)
            t[p + "mix.o"] = r(width, heads * vdim)
            if kind == "attention":
                t[p + "mix.q.norm"], t[p + "mix.k.norm"] = bf(1 + 0.2 * rng.normal(size=dim)), bf(1 + 0.2 * rng.normal(size=dim))
                t[p + "mix.g"] = r(heads, width)
            else:
                for nm, rows in (("q", heads * dim), ("k", kv_heads * dim), ("v", kv_heads * vdim)):
                    t[p + f"mix.{nm}.b"] = bf(0.2 * rng.normal(size=rows))
                m["softcap"] = softcap
                if scaling:
                    m["rot"]["scaling"] = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}
        elif kind == "gla":
            m = {"heads": gla_heads, "dim": gla_dim, "vdim": gla_vdim, "tau": tau}
            t[p + "mix.q"], t[p + "mix.k"] = r(gla_heads * gla_dim, width), r(gla_heads * gla_dim, width)
            t[p + "mix.v"], t[p + "mix.g"] = r(gla_heads * gla_vdim, width), r(gla_heads * gla_vdim, width)
            t[p + "mix.o"], t[p + "mix.norm"] = r(width, gla_heads * gla_vdim), bf(1 + 0.2 * rng.normal(size=gla_vdim))
            t[p + "mix.a1"], t[p + "mix.a2"] = r(gla_rank, width), r(gla_heads * gla_dim, gla_rank, sd=1.0)
            t[p + "mix.a2.b"] = bf(rng.normal(1.0, 1.0, gla_heads * gla_dim))
        else:
            raise ValueError(spec)
        layer = {"type": kind, "mixer": m, "mlp": None}
        if ffkind == "dense":
            layer["mlp"] = {"kind": "dense", "ff": ff}
            t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = r(ff, width), r(ff, width), r(width, ff)
        elif ffkind == "moe":
            layer["mlp"] = {"kind": "moe", "expert": {"ff": expert_ff_size, "limit": limit}, "router": {"experts": experts, "top": top}}
            for e in range(experts):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"] = r(expert_ff_size, width, sd=2.0 / math.sqrt(width)), r(expert_ff_size, width, sd=2.0 / math.sqrt(width))
                t[p + f"mlp.e{e}.down"] = r(width, expert_ff_size)
            t[p + "mlp.router"], t[p + "mlp.router.b"] = r(experts, width, sd=2.0 / math.sqrt(width)), bf(0.3 * rng.normal(size=experts))
        cfg["layers"].append(layer)
    return cfg, t
