"""Host-side parts of the Vogusun design (no GPU): the registry, the rotary frequency table, and the oracle against itself
(its recurrence against the closed form, its routed feed-forward against dense evaluation)."""
import math

import numpy as np

from oracle import vogusun as ov
from tests.conftest import load_pkg


def test_registry_knows_the_design():
    load_pkg()
    from dash_infer_amd import models
    cls = models.resolve({"architecture": "Vogusun"})
    assert cls.engine == "sequence" and "Vogusun" in models.known()


def test_rotary_frequency_table_matches_the_oracle():
    load_pkg()
    from dash_infer_amd.mixers import rotary_frequencies
    for dims, base, sc in ((16, 10000.0, None), (48, 3000.0, {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0}),
                           (64, 1e6, {"factor": 32.0, "original": 4096, "fast": 32.0, "slow": 1.0}), (2, 7.0, {"factor": 2.0, "original": 8, "fast": 4.0, "slow": 2.0})):
        f, mag = rotary_frequencies(dims, base, sc)
        rot = {"dims": dims, "base": base}
        if sc:
            rot["scaling"] = sc
        want, wmag = ov.rotary_frequencies(rot)
        assert np.allclose(f.numpy(), want.astype(np.float32), rtol=1e-7, atol=0) and abs(mag - wmag) < 1e-12
        if sc:      # the fastest pair keeps its frequency, the slowest is slowed down by the factor (where the ramp reaches them)
            assert want[0] <= base ** 0 and want[-1] >= base ** (-2.0 * (dims // 2 - 1) / dims) / sc["factor"] * (1 - 1e-12)


def test_oracle_recurrence_against_its_closed_form():
    rng = np.random.default_rng(0)
    n, H, D, V = 9, 2, 3, 4
    q, k, a = rng.normal(size=(n, H, D)), rng.normal(size=(n, H, D)), rng.uniform(0.3, 1.0, (n, H, D))
    v = rng.normal(size=(n, H, V))
    got = ov.gla_recurrence(q, k, v, a)
    for t in range(n):
        want = np.zeros((H, V))
        for s in range(t + 1):
            decay = np.prod(a[s + 1:t + 1], axis=0)                     # [H, D]: what is left of step s at step t
            want += np.einsum("hd,hd,hv->hv", q[t], decay * k[s], v[s])
        assert np.allclose(got[t], want)


def test_oracle_routing_weights_and_clamps():
    rng = np.random.default_rng(1)
    width, E, ff = 16, 4, 6
    w = {"router": rng.normal(size=(E, width)), "router.b": rng.normal(size=E)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.normal(size=(ff, width)), rng.normal(size=(ff, width)), rng.normal(size=(width, ff))
    h = rng.normal(size=(5, width))
    chosen = []
    out = ov.moe_ff(h, w, E, E, 0.5, chosen)                             # every expert: a plain softmax over all logits
    z = h @ w["router"].T + w["router.b"]
    p = np.exp(z - z.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    dense = sum(p[:, e:e + 1] * ov.expert_ff(h, w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], 0.5) for e in range(E))
    assert np.allclose(out, dense) and all(sorted(c) == list(range(E)) for c in chosen)
    one = ov.expert_ff(h, w["e0.gate"], w["e0.up"], w["e0.down"], 1e-9)  # everything clipped: g = min(., tiny), u in [-tiny, tiny]
    g = np.minimum(h @ w["e0.gate"].T, 1e-9)
    assert np.allclose(one, (g * ov.sigmoid(1.702 * g) * (np.clip(h @ w["e0.up"].T, -1e-9, 1e-9) + 1)) @ w["e0.down"].T)


def test_oracle_sink_takes_its_share():
    q, k, v = np.zeros((1, 1, 2)), np.zeros((1, 1, 2)), np.ones((1, 1, 3))
    assert np.allclose(ov.causal_attention_rows(q, k, v, 1.0, sink_one=True), 0.5)     # one key of score 0 beside the sink of score 0
    assert np.allclose(ov.causal_attention_rows(q, k, v, 1.0, sink_one=False), 1.0)
    big = ov.causal_attention_rows(np.full((1, 1, 2), 10.0), np.full((1, 1, 2), 10.0), v, 1.0, softcap=2.0)
    assert np.allclose(big, 1.0) and math.isclose(2.0 * math.tanh(200.0 / 2.0), 2.0)
