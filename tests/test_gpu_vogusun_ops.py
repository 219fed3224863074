"""The mechanisms of the Vogusun design, each alone, against the float64 restatement in oracle/vogusun.py: the norm without
statistics and the parallel residual step, grouped-query attention in both of its forms (norm, rotation layouts, sink, cap, gate,
value mixing, pages), gated linear attention (state, portions, chunks), the gated and the routed feed-forward."""
import math

import numpy as np
import pytest
import torch

from oracle import vogusun as ov
from tests.conftest import load_pkg
from tests.seq_helpers import MixerRig, dev_weights, rel_err

pytestmark = pytest.mark.gpu
bf = ov.bf16_values


@pytest.fixture(scope="module")
def so():
    load_pkg()
    from dash_infer_amd import seq_ops
    return seq_ops


def dev(a, dt=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dt).cuda()


def i32(a):
    return torch.tensor(a, dtype=torch.int32, device="cuda")


# ---------------------------------------------------------------------------------------------------------------- norm + residual
def test_add_dyt_residual_norm_and_row_index(so):
    rng = np.random.default_rng(0)
    T, K = 37, 100
    x, a, b = (rng.normal(0, 1.5, (T, K)).astype(np.float32) for _ in range(3))
    w, bias, alpha = bf(1 + 0.2 * rng.normal(size=K)), bf(0.2 * rng.normal(size=K)), 0.71875
    xs = x.astype(np.float64) + (a.astype(np.float64) + b)
    want = ov.dyt_norm(xs, alpha, w, bias)
    xd = dev(x)
    wide = dev(np.concatenate([a, b], 1))                    # sublayer outputs as column slices of a wider buffer
    h, h16 = so.add_dyt(xd, wide[:, :K], wide[:, K:], norm=(alpha, dev(w, torch.bfloat16), dev(bias, torch.bfloat16)), x_out=xd)
    assert h16 is None and rel_err(xd.cpu().numpy(), xs) < 1e-6 and rel_err(h.cpu().numpy(), want) < 2e-6
    _, h16 = so.add_dyt(xd, norm=(alpha, dev(w, torch.bfloat16), dev(bias, torch.bfloat16)), want16=True)
    assert torch.equal(h16.cpu(), h.cpu().to(torch.bfloat16))
    rows = [5, 0, 36, 5]
    hr, _ = so.add_dyt(xd, norm=(alpha, dev(w, torch.bfloat16), dev(bias, torch.bfloat16)), row_idx=i32(rows))
    assert torch.equal(hr.cpu(), h.cpu()[rows])
    only, _ = so.add_dyt(dev(x), dev(a), None, norm=(alpha, dev(w), dev(bias)))      # one sublayer, f32 weights, no stream written
    assert rel_err(only.cpu().numpy(), ov.dyt_norm(x.astype(np.float64) + a, alpha, w, bias)) < 2e-6


# ---------------------------------------------------------------------------------------------------------------- attention
def attention_weights(rng, kind, width, H, G, D, V):
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else 1.0 / math.sqrt(s[-1]), s))
    w = {"q": r(H * D, width), "k": r(G * D, width), "v": r(G * V, width), "o": r(width, H * V), "vmix": bf(np.float32(0.375))}
    if kind == "attention":
        w.update({"q.norm": bf(1 + 0.2 * rng.normal(size=D)), "k.norm": bf(1 + 0.2 * rng.normal(size=D)), "g": r(H, width)})
    else:
        w.update({"q.b": bf(0.2 * rng.normal(size=H * D)), "k.b": bf(0.2 * rng.normal(size=G * D)), "v.b": bf(0.2 * rng.normal(size=G * V))})
    return w


def attention_rig(kind, w, m, dtype, value_mix=None, **kw):
    load_pkg()
    from dash_infer_amd import mixers
    rot = m["rot"]
    extra = dict(rot_layout="pairs", qk_norm=True, sink="zero", head_gate=True) if kind == "attention" else \
        dict(rot_layout="halves", softcap=m.get("softcap"))
    build = lambda state, dt: mixers.GroupedQueryAttention("t", m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], dev_weights(w), state,
                                                           dt, rot_dims=rot["dims"], rot_base=rot["base"], rot_scaling=rot.get("scaling"),
                                                           value_mix=value_mix, **extra)
    return MixerRig(build, dtype, **kw)


SHAPES = [  # width, heads, kv heads, dim, vdim, rotated dims
    (72, 6, 2, 24, 16, 24),      # head sizes that are no multiple of 32 / 16
    (64, 4, 4, 32, 32, 16),      # as many key/value heads as query heads, half of the head rotated
    (80, 5, 1, 40, 8, 40),       # one key/value head, an odd number of query heads
    (64, 2, 1, 128, 64, 64),     # wide heads
    (48, 3, 3, 20, 12, 8),       # head sizes the matrix-core kernel does not serve
    (64, 2, 1, 160, 128, 32),    # the widest tiles of the matrix-core kernel
]


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
@pytest.mark.parametrize("shape", SHAPES)
def test_attention_whole_decoded_and_in_portions(kind, shape):
    width, H, G, D, V, rd = shape
    rng = np.random.default_rng(H * 100 + D)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 1.7 / math.sqrt(D), "rot": {"base": 3000.0, "dims": rd}}
    if kind == "attention_2":
        m["softcap"] = 4.0     # low enough to bend many scores
        m["rot"]["scaling"] = {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0}
    w = attention_weights(rng, kind, width, H, G, D, V)
    n = 150
    h = rng.normal(0, 1, (n, width)).astype(np.float32)
    want, _ = ov.attention(h, w, m, 1e-5, kind)
    rig = attention_rig(kind, w, m, torch.float32)
    whole = rig.step([("w", h)])[0]
    assert rel_err(whole, want) < 2e-5
    dec = np.concatenate([rig.step([("d", h[i:i + 1])])[0] for i in range(n)])
    assert rel_err(dec, whole) < 1e-6
    parts, at = [], 0
    for size in [2, 61, 3, 1, 64, 2, 17]:                       # ends inside a page, at its border, one row into the next
        parts.append(rig.step([("p", h[at:at + size])])[0])
        at += size
    assert at == n and rel_err(np.concatenate(parts), whole) < 1e-6
    rig16 = attention_rig(kind, w, m, torch.bfloat16)
    h16 = bf(h)
    want16, _ = ov.attention(h16, w, m, 1e-5, kind)
    whole16 = rig16.step([("w", h16)])[0]
    assert rel_err(whole16, want16) < 0.03
    dec16 = np.concatenate([rig16.step([("d", h16[:100])])[0]] + [rig16.step([("d", h16[i:i + 1])])[0] for i in range(100, n)])
    assert rel_err(dec16, want16) < 0.03


def test_attention_value_mixing_between_layers():
    rng = np.random.default_rng(3)
    width, H, G, D, V = 64, 4, 2, 16, 24
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.25, "rot": {"base": 100.0, "dims": D}, "v_mix": True}
    w1, w2 = attention_weights(rng, "attention", width, H, G, D, V), attention_weights(rng, "attention_2", width, H, G, D, V)
    h1, h2 = rng.normal(0, 1, (70, width)).astype(np.float32), rng.normal(0, 1, (70, width)).astype(np.float32)
    want1, v1 = ov.attention(h1, w1, m, 1e-5, "attention", None)
    want2, _ = ov.attention(h2, w2, m, 1e-5, "attention_2", v1)
    plain2, _ = ov.attention(h2, w2, m, 1e-5, "attention_2", None)
    assert rel_err(plain2, want2) > 0.05                         # the comparison below sees whether the values were mixed
    load_pkg()
    from dash_infer_amd import mixers

    def build(state, dt):      # both layers in one step: the second reads the values the first one left for it
        mk = lambda key, w, vm, **kw: mixers.GroupedQueryAttention(key, H, G, D, V, 0.25, dev_weights(w), state, dt, rot_dims=D, rot_base=100.0,
                                                                   value_mix=vm, **kw)
        first = mk("a", w1, ("source", "v"), rot_layout="pairs", qk_norm=True, sink="zero", head_gate=True)
        second = mk("b", w2, ("mix", "v", 0.375), rot_layout="halves")
        return lambda ctx, h, h16=None: torch.cat([first(ctx, h[:, :width].contiguous()), second(ctx, h[:, width:].contiguous())], 1)
    rig = MixerRig(build)
    both = np.concatenate([h1, h2], 1)
    for lo, hi in ((0, 33), (33, 34), (34, 70)):
        o = rig.step([("s", both[lo:hi])])[0]
        assert rel_err(o[:, :width], want1[lo:hi]) < 2e-5 and rel_err(o[:, width:], want2[lo:hi]) < 2e-5


@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sink_one", [True, False])
def test_attention_far_keys_page_borders_and_the_sink(so, cdt, sink_one):
    """keys and values are written by hand: one key far back stands out for some queries; for others every score is low, so that
    the sink's share of the softmax decides the result"""
    load_pkg()
    from dash_infer_amd.seq_state import SequenceStateManager
    rng = np.random.default_rng(11)
    H, G, D, V, n = 4, 2, 32, 16, 200
    q = rng.normal(0, 0.3, (n, H, D))
    k = rng.normal(0, 0.3, (n, G, D))
    v = rng.normal(0, 1, (n, G, V))
    far = {199: 3, 130: 63, 129: 64, 128: 127, 70: 0}            # query position -> the key it must find (page borders at 64, 128)
    for qp, kp in far.items():
        k[kp] = rng.normal(0, 0.3, (G, D))
        q[qp] = np.repeat(k[kp], H // G, 0) * 60.0               # a score far above all others
    low = [5, 66, 150]
    for qp in low:
        q[qp] = -np.repeat(k[:qp + 1].mean(0), H // G, 0) * 30 - 3.0 * np.sign(np.repeat(k[:qp + 1].mean(0), H // G, 0))
    q, k, v = bf(q), bf(k), bf(v)
    want = ov.causal_attention_rows(q.astype(np.float64), k, v, 0.5, sink_one=sink_one).reshape(n, H * V)
    other = ov.causal_attention_rows(q.astype(np.float64), k, v, 0.5, sink_one=not sink_one).reshape(n, H * V)
    assert max(rel_err(other[p], want[p]) for p in low) > 0.2    # a sink left out (or put in) shows
    for qp, kp in far.items():
        assert rel_err(want[qp].reshape(H, V), np.repeat(v[kp], H // G, 0)) < (0.6 if sink_one else 1e-3)
    st = SequenceStateManager(512, 2, 64, "cuda")
    kt, vt = st.add_span_cache("k", G * D, cdt), st.add_span_cache("v", G * V, cdt)
    st.admit("a")
    st.reserve("a", n)
    st.upload()
    slot = st.live["a"].index
    rows = dev(np.concatenate([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], 1))
    so.qkv_prep_append(rows, 0, H * D, (H + G) * D, H, G, D, V, None, None, 1e-5, None, 0, 0, 1.0, 0.0, None, None, kt, vt,
                       i32([slot] * n), i32(list(range(n))))
    mode = so.SINK_ZERO if sink_one else so.SINK_NONE
    got = so.gqa_attn(rows, kt, vt, i32([slot] * n), i32(list(range(n))), H, G, D, V, 0.5, sink_mode=mode).cpu().numpy()
    assert rel_err(got, want) < (2e-5 if cdt == torch.float32 else 2e-5)
    one = so.gqa_attn(rows[199:200], kt, vt, i32([slot]), i32([199]), H, G, D, V, 0.5, sink_mode=mode).cpu().numpy()   # decoded alone
    assert np.array_equal(one[0], got[199])
    if cdt == torch.bfloat16:
        for nsplit in (1, 3):
            mc = so.gqa_attn_mc(rows, kt, vt, i32(list(range(n))), i32([slot]), i32([0]), i32([n]), n, n - 1, H, G, D, V, 0.5, sink_mode=mode,
                                nsplit=nsplit).cpu().numpy()
            assert rel_err(mc, want) < 0.01
            for p in low + list(far):
                assert rel_err(mc[p], want[p]) < 0.02, (p, nsplit)
        for p in (199, 129, 66):                                  # decoded alone: one row, the key walk split
            mc1 = so.gqa_attn_mc(rows[p:p + 1], kt, vt, i32([p]), i32([slot]), i32([0]), i32([1]), 1, p, H, G, D, V, 0.5, sink_mode=mode).cpu().numpy()
            assert rel_err(mc1[0], want[p]) < 0.02


# ---------------------------------------------------------------------------------------------------------------- gated linear attention
def gla_weights(rng, width, H, D, V, rank, decay_bias=1.0):
    r = lambda *s, sd=None: bf(rng.normal(0, sd if sd is not None else 1.0 / math.sqrt(s[-1]), s))
    return {"q": r(H * D, width), "k": r(H * D, width), "v": r(H * V, width), "g": r(H * V, width), "o": r(width, H * V),
            "norm": bf(1 + 0.2 * rng.normal(size=V)), "a1": r(rank, width), "a2": r(H * D, rank, sd=1.0),
            "a2.b": bf(rng.normal(decay_bias, 1.0, H * D))}


def gla_rig(w, m, dtype, **kw):
    load_pkg()
    from dash_infer_amd import mixers
    return MixerRig(lambda state, dt: mixers.GatedLinearAttention("t", m["heads"], m["dim"], m["vdim"], m["tau"], dev_weights(w), state), dtype, **kw)


@pytest.mark.parametrize("shape", [(72, 3, 20, 24, 8, 8.0), (64, 1, 64, 64, 4, 1.0), (96, 2, 72, 130, 16, 12.0), (64, 2, 8, 200, 1, 2.0),
                                   (64, 1, 136, 40, 4, 4.0)])
def test_gla_whole_decoded_portions_and_chunks(shape):
    width, H, D, V, rank, tau = shape
    rng = np.random.default_rng(D + V)
    m = {"heads": H, "dim": D, "vdim": V, "tau": tau}
    w = gla_weights(rng, width, H, D, V, rank, decay_bias=3.0 if tau < 4 else 0.0)
    n = 330
    h = rng.normal(0, 1, (n, width)).astype(np.float32)
    want = ov.gla(h, w, m, 1e-5)
    rig = gla_rig(w, m, torch.float32)
    whole = rig.step([("w", h)])[0]                              # long enough for the chunks that run side by side
    assert rel_err(whole, want) < 3e-5
    dec = np.concatenate([rig.step([("d", h[i:i + 1])])[0] for i in range(n)])     # long decoding through the state
    assert rel_err(dec, want) < 3e-5
    parts, at = [], 0
    for size in [2, 100, 1, 129, 64, 3, 31]:
        parts.append(rig.step([("p", h[at:at + size])])[0])
        at += size
    assert at == n and rel_err(np.concatenate(parts), want) < 3e-5
    rig.release("w")
    again = rig.step([("w2", h[:40])])[0]                         # a slot that held a state starts from zero again
    assert rel_err(again, want[:40]) < 3e-5
    rig16 = gla_rig(w, m, torch.bfloat16)
    h16 = bf(h)
    assert rel_err(rig16.step([("w", h16)])[0], ov.gla(h16, w, m, 1e-5)) < 0.03


def test_gla_sequences_side_by_side():
    rng = np.random.default_rng(21)
    m = {"heads": 2, "dim": 24, "vdim": 40, "tau": 4.0}
    w = gla_weights(rng, 64, 2, 24, 40, 8)
    hs = [rng.normal(0, 1, (n, 64)).astype(np.float32) for n in (140, 9, 1)]
    want = [ov.gla(h, w, m, 1e-5) for h in hs]
    rig = gla_rig(w, m, torch.float32)
    a = rig.step([("a", hs[0][:130]), ("b", hs[1][:2]), ("c", hs[2])])     # a chunked portion beside short ones
    b = rig.step([("b", hs[1][2:]), ("a", hs[0][130:])])
    assert rel_err(np.concatenate([a[0], b[1]]), want[0]) < 3e-5
    assert rel_err(np.concatenate([a[1], b[0]]), want[1]) < 3e-5 and rel_err(a[2], want[2]) < 3e-5


# ---------------------------------------------------------------------------------------------------------------- feed-forward
def test_gated_mlp():
    load_pkg()
    from dash_infer_amd import mixers
    rng = np.random.default_rng(31)
    width, ff = 72, 100
    w = {"gate": bf(rng.normal(0, 0.2, (ff, width))), "up": bf(rng.normal(0, 0.2, (ff, width))), "down": bf(rng.normal(0, 0.1, (width, ff)))}
    h = rng.normal(0, 1, (70, width)).astype(np.float32)
    dw = dev_weights(w)
    rig = MixerRig(lambda state, dt: mixers.GatedMlp(dw["gate"], dw["up"], dw["down"], "gelu_tanh"))
    assert rel_err(rig.step([("a", h)])[0], ov.dense_ff(h, w)) < 1e-5


@pytest.mark.parametrize("experts,top,T", [(5, 2, 1), (5, 2, 70), (10, 3, 300), (4, 4, 9), (3, 1, 40), (40, 6, 130)])
def test_routed_experts(so, experts, top, T):
    load_pkg()
    from dash_infer_amd import mixers
    rng = np.random.default_rng(experts * 10 + top)
    width, ff, limit = 64, 24, 0.75                                # a limit that clips many units
    w = {"router": bf(rng.normal(0, 0.5, (experts, width))), "router.b": bf(rng.normal(0, 0.5, experts))}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"] = bf(rng.normal(0, 0.25, (ff, width))), bf(rng.normal(0, 0.25, (ff, width)))
        w[f"e{e}.down"] = bf(rng.normal(0, 0.2, (width, ff)))
    h = bf(rng.normal(0, 1, (T, width)))
    chosen = []
    want = ov.moe_ff(h, w, experts, top, limit, chosen)
    dw = dev_weights(w)
    build = lambda state, dt: mixers.ExpertMlp(dw["router"], dw["router.b"], [dw[f"e{e}.gate"] for e in range(experts)],
                                               [dw[f"e{e}.up"] for e in range(experts)], [dw[f"e{e}.down"] for e in range(experts)], top, limit)
    rig = MixerRig(build)
    got = rig.step([("a", h)])[0]
    z = dev(h.astype(np.float64) @ w["router"].astype(np.float64).T + w["router.b"])
    ids, wts, seg, src, dst = so.moe_route(z, top)
    assert ids.cpu().tolist() == chosen and abs(float(wts.sum()) - T) < 1e-4
    seg = seg.cpu().tolist()
    assert seg[0] == 0 and seg[-1] == T * top and all(a <= b for a, b in zip(seg, seg[1:]))
    assert rel_err(got, want) < 1e-5
    rig16 = MixerRig(build, torch.bfloat16)
    assert rel_err(rig16.step([("a", h)])[0], want) < 0.03
    if T > 1:                                                     # a token's result does not depend on the others of the batch
        assert rel_err(rig.step([("b", h[T // 2:T // 2 + 1])])[0], got[T // 2:T // 2 + 1]) < 1e-6


@pytest.mark.parametrize("T,N,K", [(100, 12, 192), (300, 5, 64), (40, 64, 1000), (17, 1, 8)])
def test_router_logits_many_rows_few_columns(so, T, N, K):
    """the f32 product of many rows with few output columns: unrounded operands, the same bits for a row whatever the batch"""
    rng = np.random.default_rng(T + N)
    x = rng.normal(0, 1, (T, K)).astype(np.float32)
    w, b = bf(rng.normal(0, 0.3, (N, K))), bf(rng.normal(0, 0.3, N))
    want = x.astype(np.float64) @ w.astype(np.float64).T + b
    got = so.linear(dev(x), dev(w, torch.bfloat16), dev(b, torch.bfloat16), math=so.MATH_F32_STREAM)
    assert rel_err(got.cpu().numpy(), want) < 2e-6
    part = so.linear(dev(x[T // 2:T // 2 + 20]), dev(w, torch.bfloat16), dev(b, torch.bfloat16), math=so.MATH_F32_STREAM)
    assert torch.equal(part.cpu(), got.cpu()[T // 2:T // 2 + 20])
    x16 = dev(x, torch.bfloat16)
    got16 = so.linear(x16, dev(w, torch.bfloat16), dev(b, torch.bfloat16), math=so.MATH_F32_STREAM)
    assert rel_err(got16.cpu().numpy(), x16.double().cpu().numpy() @ w.astype(np.float64).T + b) < 2e-6
