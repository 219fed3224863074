"""Plain, slow float64 restatement of the sequence engine's mechanisms, one function per mechanism, token by token where
the mechanism is sequential.  Test infrastructure only: shares no code with the product path (numpy, no kernels).

Notation: h [n, width] the rows of ONE sequence in order; weights are numpy arrays as the checkpoint stores them ([out, in])."""
import math

import numpy as np


def rms_norm(x, w, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * np.asarray(w, np.float64)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    erf = np.vectorize(math.erf)
    return 0.5 * z * (1.0 + erf(z / math.sqrt(2.0)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def embedding(tokens, embed, bigram=None, buckets=0, mul_prev=0, mul_cur=0):
    out = []
    for i, t in enumerate(tokens):
        x = np.asarray(embed[t], np.float64).copy()
        if bigram is not None:
            row = buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets
            x += np.asarray(bigram[row], np.float64)
        out.append(x)
    return np.stack(out)


def sink_softmax_window(scores, values, sink):
    """one query: scores [m], values [m, d], sink a number or None -> weighted sum [d]"""
    mx = max(float(np.max(scores)), -np.inf if sink is None else float(sink))
    e = np.exp(scores - mx)
    den = e.sum() + (0.0 if sink is None else math.exp(float(sink) - mx))
    return (e[:, None] * values).sum(0) / den


def latent_attention_rows(q, c, uk, uv, heads, dim, vdim, window, scale, sink):
    """q [n, heads*dim] queries, c [n, rank] the sequence's latents: keys and values are formed per head from c."""
    n = q.shape[0]
    k = (c @ uk.T).reshape(n, heads, dim)
    v = (c @ uv.T).reshape(n, heads, vdim)
    out = np.zeros((n, heads * vdim))
    for i in range(n):
        lo = 0 if not window else max(0, i - window + 1)
        for h in range(heads):
            s = (k[lo:i + 1, h] @ q[i].reshape(heads, dim)[h]) * scale
            out[i, h * vdim:(h + 1) * vdim] = sink_softmax_window(s, v[lo:i + 1, h], None if sink is None else sink[h])
    return out


def latent_attention(h, w, heads, dim, vdim, window, scale, eps, latent=None):
    """the whole mixer; latent: another layer's latents [n, rank] to use instead of this layer's own.  -> (out, latents)"""
    f = lambda name: np.asarray(w[name], np.float64)
    cq = rms_norm(h @ f("dq").T, f("dq.norm"), eps)
    q = cq @ f("uq").T
    c = latent if latent is not None else rms_norm(h @ f("dkv").T, f("dkv.norm"), eps)
    a = latent_attention_rows(q, c, f("uk"), f("uv"), heads, dim, vdim, window, scale, f("sink") if "sink" in w else None)
    a = a * sigmoid(h @ f("g").T)
    return a @ f("o").T, c


def causal_conv(x, conv, bias):
    """x [n, C], conv [C, taps] (last column = the current row), zeros before the start"""
    n, taps = x.shape[0], conv.shape[1]
    out = np.zeros_like(x)
    for t in range(n):
        acc = np.asarray(bias, np.float64).copy()
        for k in range(taps):
            src = t - (taps - 1 - k)
            if src >= 0:
                acc += conv[:, k] * x[src]
        out[t] = acc
    return out


def gated_recurrence(u, r, i, lam, decay):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t from S = 0;  a_t = exp(-decay r_t softplus(lam))"""
    S = np.zeros(u.shape[1])
    out = np.zeros_like(u)
    sp = softplus(np.asarray(lam, np.float64))
    for t in range(u.shape[0]):
        a = np.exp(-decay * r[t] * sp)
        S = a * S + np.sqrt(1.0 - a * a) * i[t] * u[t]
        out[t] = S
    return out


def rglru(h, w, blocks, decay=8.0):
    f = lambda name: np.asarray(w[name], np.float64)
    y = gelu_tanh(h @ f("y").T + f("y.b"))
    u = causal_conv(h @ f("x").T + f("x.b"), f("conv"), f("conv.b"))
    n, C = u.shape
    bs = C // blocks
    r, i = np.zeros_like(u), np.zeros_like(u)
    for b in range(blocks):
        ub = u[:, b * bs:(b + 1) * bs]
        r[:, b * bs:(b + 1) * bs] = sigmoid(ub @ f("ra")[b].T + f("ra.b")[b])
        i[:, b * bs:(b + 1) * bs] = sigmoid(ub @ f("ri")[b].T + f("ri.b")[b])
    return (gated_recurrence(u, r, i, f("lam"), decay) * y) @ f("o").T


def dense_mlp(h, up, down):
    return gelu_erf(h @ np.asarray(up, np.float64).T) @ np.asarray(down, np.float64).T


def modanex_forward(config, tensors, tokens, layer_streams=None):
    """tensors: name -> numpy array (any float type).  -> logits [n, vocab] (float64)"""
    eps = config["norm"]["eps"]
    f = lambda name: np.asarray(tensors[name], np.float64)
    bg = (config.get("embedding") or {}).get("bigram")
    x = embedding(tokens, f("embed"), f("bigram") if bg else None, *((bg["buckets"], bg["mul_prev"], bg["mul_cur"]) if bg else ()))
    X, latents = [x], {}
    for li, lc in enumerate(config["layers"]):
        p, m = "l%d." % li, lc["mixer"]
        w = {k[len(p) + 4:]: v for k, v in tensors.items() if k.startswith(p + "mix.")}
        if lc["type"] == "latent_attention":
            mo, c = latent_attention(x, w, m["heads"], m["dim"], m["vdim"], (m.get("mask") or {}).get("size"), m["scale"], eps,
                                     latents[m["kv_from"]] if "kv_from" in m else None)
            if "kv_from" not in m:
                latents[li] = c
        else:
            mo = rglru(x, w, m["blocks"])
        x = x + rms_norm(mo, f(p + "norm1"), eps)
        if lc.get("mlp") is not None:
            x = x + rms_norm(dense_mlp(x, f(p + "mlp.up"), f(p + "mlp.down")), f(p + "norm2"), eps)
        X.append(x)
        if p + "dwa" in tensors:
            d = f(p + "dwa")
            x = sum(d[j] * X[j] for j in range(li + 2))
        if layer_streams is not None:
            layer_streams.append(x)
    return rms_norm(x, f("final.norm"), eps) @ f("head").T


def random_modanex(rng, width=72, vocab=97, layers=("rglru", "latent_attention", "latent_attention:share", "rglru+mlp"), heads=3, dim=24, vdim=40,
                   kv_rank=48, q_rank=40, window=37, scale=0.2, rec_width=96, blocks=3, taps=4, ff=120, buckets=53, eps=1e-5,
                   bigram=True, std=None):
    """A small random model: (config, tensors as float32 numpy arrays rounded to bf16 values).  Layer specs: 'rglru' or
    'latent_attention', ':share' = reads the latent cache of the closest earlier layer that owns one, '+mlp' = with a feed-forward."""
    def bf(a):
        u = np.asarray(a, np.float32).view(np.uint32)
        u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
        return u.astype(np.uint32).view(np.float32)
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else (std or 1.0 / math.sqrt(s[-1])), s))
    cfg = {"architecture": "Modanex", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": [],
           "embedding": {"bigram": {"buckets": buckets, "mul_prev": 31, "mul_cur": 5}} if bigram else {}}
    t = {"embed": r(vocab, width, sd=1.0), "final.norm": bf(1 + 0.1 * rng.normal(size=width)), "head": r(vocab, width)}
    if bigram:
        t["bigram"] = r(buckets + 1, width, sd=0.5)
    owner = None
    for i, spec in enumerate(layers):
        kind, mlp = spec.replace("+mlp", ""), "+mlp" in spec
        p = "l%d." % i
        if kind.startswith("latent_attention"):
            m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "mask": {"size": window}, "scale": scale}
            share = kind.endswith(":share")
            if share:
                assert owner is not None
                m["kv_from"] = owner
            else:
                owner = i
                t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = r(kv_rank, width), bf(1 + 0.1 * rng.normal(size=kv_rank))
            t[p + "mix.dq"], t[p + "mix.dq.norm"] = r(q_rank, width), bf(1 + 0.1 * rng.normal(size=q_rank))
            t[p + "mix.uq"], t[p + "mix.uk"], t[p + "mix.uv"] = r(heads * dim, q_rank), r(heads * dim, kv_rank), r(heads * vdim, kv_rank)
            t[p + "mix.sink"] = bf(rng.normal(0, 1.0, heads))
            t[p + "mix.g"], t[p + "mix.o"] = r(heads * vdim, width), r(width, heads * vdim)
            cfg["layers"].append({"type": "latent_attention", "mixer": m, "mlp": None})
        else:
            bs = rec_width // blocks
            t[p + "mix.y"], t[p + "mix.y.b"] = r(rec_width, width), bf(0.1 * rng.normal(size=rec_width))
            t[p + "mix.x"], t[p + "mix.x.b"] = r(rec_width, width), bf(0.1 * rng.normal(size=rec_width))
            t[p + "mix.conv"], t[p + "mix.conv.b"] = r(rec_width, taps, sd=0.5), bf(0.1 * rng.normal(size=rec_width))
            t[p + "mix.ra"], t[p + "mix.ra.b"] = r(blocks, bs, bs), bf(0.3 * rng.normal(size=(blocks, bs)))
            t[p + "mix.ri"], t[p + "mix.ri.b"] = r(blocks, bs, bs), bf(0.3 * rng.normal(size=(blocks, bs)))
            t[p + "mix.lam"], t[p + "mix.o"] = bf(rng.normal(-1.0, 1.0, rec_width)), r(width, rec_width)
            cfg["layers"].append({"type": "rglru", "mixer": {"width": rec_width, "blocks": blocks, "conv": taps}, "mlp": None})
        t[p + "norm1"] = bf(1 + 0.1 * rng.normal(size=width))
        if mlp:
            cfg["layers"][-1]["mlp"] = {"kind": "dense", "ff": ff}
            t[p + "mlp.up"], t[p + "mlp.down"], t[p + "norm2"] = r(ff, width), r(width, ff), bf(1 + 0.1 * rng.normal(size=width))
        t[p + "dwa"] = bf(rng.normal(0.5, 0.5, i + 2))
    return cfg, t
