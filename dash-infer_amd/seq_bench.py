"""bench.py --workload modanex_layers: prefill and decode throughput of the sequence engine on random Modanex models of
layer sizes that resemble real models', per-operator times against their rooflines, and the quantised decode runner's
Qwen2 layers of equal width / depth / feed-forward size beside them (int8 per-channel weights: its closest weight form to
16-bit weights)."""
import math
import time

import torch

HBM_BW = 8.0e12          # bytes / s
MFMA_BF16 = 2.5e15       # dense bf16 flop / s
VALU_F32 = 1.57e14       # f32 flop / s of the vector units (256 CUs x 4 SIMD x 16 lanes x 2 x 2.4 GHz packed pairs)

SIZES = {
    # width, heads, dim, vdim, kv_rank, q_rank, window, rec_width, blocks, taps, ff, vocab
    "2k": dict(width=2048, heads=16, dim=128, vdim=128, kv_rank=256, q_rank=768, window=1024, rec_width=2560, blocks=10, taps=4, ff=8192, vocab=32000),
    "4k": dict(width=4096, heads=32, dim=128, vdim=128, kv_rank=512, q_rank=1536, window=2048, rec_width=4096, blocks=16, taps=4, ff=14336, vocab=32000),
}
PATTERN = ("rglru", "latent_attention+mlp", "rglru", "latent_attention:share+mlp", "rglru+mlp", "latent_attention+mlp")


def random_model(size, device="cuda", seed=0):
    """config + bf16 tensors on the device (torch generator: nothing of it is trained or loaded)"""
    s = SIZES[size]
    g = torch.Generator(device=device).manual_seed(seed)
    W = s["width"]

    def r(*shape, sd=None):
        sd = sd if sd is not None else 1.0 / math.sqrt(shape[-1])
        return (torch.randn(*shape, generator=g, device=device) * sd).to(torch.bfloat16)

    def one(n):
        return (1 + 0.1 * torch.randn(n, generator=g, device=device)).to(torch.bfloat16)
    cfg = {"architecture": "Modanex", "width": W, "vocab": s["vocab"], "norm": {"eps": 1e-6}, "layers": [],
           "embedding": {"bigram": {"buckets": 8191, "mul_prev": 1009, "mul_cur": 13}}}
    t = {"embed": r(s["vocab"], W, sd=1.0), "bigram": r(8192, W, sd=0.5), "final.norm": one(W), "head": r(s["vocab"], W)}
    owner = None
    for i, spec in enumerate(PATTERN):
        p = f"l{i}."
        kind = spec.replace("+mlp", "")
        H, D, V, R, Q = s["heads"], s["dim"], s["vdim"], s["kv_rank"], s["q_rank"]
        if kind.startswith("latent_attention"):
            m = {"heads": H, "dim": D, "vdim": V, "kv_rank": R, "q_rank": Q, "mask": {"size": s["window"]}, "scale": 1.0 / math.sqrt(D)}
            if kind.endswith(":share"):
                m["kv_from"] = owner
            else:
                owner = i
                t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = r(R, W), one(R)
            t[p + "mix.dq"], t[p + "mix.dq.norm"], t[p + "mix.uq"] = r(Q, W), one(Q), r(H * D, Q)
            t[p + "mix.uk"], t[p + "mix.uv"], t[p + "mix.sink"] = r(H * D, R), r(H * V, R), r(H, sd=1.0)
            t[p + "mix.g"], t[p + "mix.o"] = r(H * V, W), r(W, H * V)
            cfg["layers"].append({"type": "latent_attention", "mixer": m, "mlp": None})
        else:
            C, B = s["rec_width"], s["blocks"]
            bs = C // B
            for n_ in ("y", "x"):
                t[p + "mix." + n_], t[p + "mix." + n_ + ".b"] = r(C, W), r(C, sd=0.1)
            t[p + "mix.conv"], t[p + "mix.conv.b"] = r(C, s["taps"], sd=0.5), r(C, sd=0.1)
            for n_ in ("ra", "ri"):
                t[p + "mix." + n_], t[p + "mix." + n_ + ".b"] = r(B, bs, bs), r(B, bs, sd=0.3)
            t[p + "mix.lam"], t[p + "mix.o"] = (torch.randn(C, generator=g, device=device) - 1).to(torch.bfloat16), r(W, C)
            cfg["layers"].append({"type": "rglru", "mixer": {"width": C, "blocks": B, "conv": s["taps"]}, "mlp": None})
        t[p + "norm1"] = one(W)
        if "+mlp" in spec:
            cfg["layers"][-1]["mlp"] = {"kind": "dense", "ff": s["ff"]}
            t[p + "mlp.up"], t[p + "mlp.down"], t[p + "norm2"] = r(s["ff"], W), r(W, s["ff"]), one(W)
        t[p + "dwa"] = (0.5 + 0.5 * torch.randn(i + 2, generator=g, device=device)).to(torch.bfloat16)
    return cfg, t


def _time(fn, reps):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e-3


def engine_throughput(eng, vocab, prompt_len, decode_batches=(1, 4), decode_steps=32):
    gen = torch.Generator().manual_seed(3)
    toks = torch.randint(0, vocab, (8, prompt_len + decode_steps + 8), generator=gen).tolist()

    def prefill():
        eng.step([("p", toks[0][:prompt_len], [prompt_len - 1])])
        eng.release("p")
    out = {"prefill_tokens_per_s": round(prompt_len / _time(prefill, 3), 1)}
    for b in decode_batches:
        eng.step([(("d", k), toks[k][:prompt_len - 4], []) for k in range(b)])
        for i in range(-4, 0):       # the first decode step of a shape launches eagerly and is captured: not timed
            eng.step([(("d", k), [toks[k][prompt_len + i]], [0]) for k in range(b)])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(decode_steps):
            lg = eng.step([(("d", k), [toks[k][prompt_len + i]], [0]) for k in range(b)])
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / decode_steps
        for k in range(b):
            eng.release(("d", k))
        out[f"decode_b{b}_tokens_per_s"] = round(b / dt, 1)
        out[f"decode_b{b}_ms_per_step"] = round(dt * 1e3, 3)
    return out


def operator_table(size, prompt_len):
    """every operator of the layers alone, at the prompt's row count and at one row: seconds, and the fraction of its bound
    (matrix products at T rows: the bf16 matrix-core peak; everything else: 8 TB/s over the bytes it must move)"""
    from . import seq_ops as so
    from .seq_state import SequenceStateManager
    s = SIZES[size]
    W, H, D, V, R, Q, C, B, ff = s["width"], s["heads"], s["dim"], s["vdim"], s["kv_rank"], s["q_rank"], s["rec_width"], s["blocks"], s["ff"]
    dev = "cuda"
    rows = []
    bf = lambda *sh: (torch.randn(*sh, device=dev) * 0.05).to(torch.bfloat16)
    for T in (prompt_len, 1):
        x = torch.randn(T, max(W, ff, C, H * V, H * R, H * D), device=dev)
        x16 = x.to(torch.bfloat16)      # the engine hands bf16 copies to the products wherever their producer can write one
        for name, N, K in (("attn in-proj", Q + R + H * V, W), ("attn uq", H * D, Q), ("attn o", W, H * V), ("rglru in-proj", 2 * C, W),
                           ("rglru o (f32 rows)", W, C), ("mlp up", ff, W), ("mlp down", W, ff), ("head", s["vocab"], W)):
            if name == "head" and T > 1:
                continue
            w = bf(N, K)
            y = torch.empty(T, N, device=dev)
            xin = x if "f32 rows" in name or name == "head" else x16
            sec = _time(lambda: so.linear(xin[:, :K], w, out=y, math=so.MATH_BF16), 5)
            fl, by = 2.0 * T * N * K, 2.0 * N * K + 4.0 * T * N + xin.element_size() * T * K
            bound = max(fl / MFMA_BF16, by / HBM_BW)
            rows.append({"op": f"linear {name} [{T}x{K}]x[{N}]", "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 1),
                         "gbps": round(by / sec / 1e9), "of_bound": round(bound / sec, 3)})
        for name, G, N, K, xg in (("attn q absorb", H, R, D, H), ("attn uv", H, V, R, H), ("rglru gates (f32)", 2 * B, C // B, C // B, B)):
            w = bf(G, N, K)
            y = torch.empty(T, G * N, device=dev)
            mth = so.MATH_F32_STREAM if "gates" in name else so.MATH_BF16
            sec = _time(lambda: so.linear(x[:, :xg * K], w, out=y, math=mth, groups=G, x_groups=xg), 5)
            fl, by = 2.0 * T * G * N * K, 2.0 * G * N * K + 4.0 * T * (G * N + xg * K)
            bound = max(fl / (VALU_F32 if mth != so.MATH_BF16 else MFMA_BF16), by / HBM_BW)
            rows.append({"op": f"grouped linear {name} {G}x[{T}x{K}]x[{N}]", "us": round(sec * 1e6, 1), "tflops": round(fl / sec / 1e12, 2),
                         "of_bound": round(bound / sec, 3)})
        # attention over the cache: prompt rows at positions 0 .. T-1, or one row at position prompt_len - 1
        st = SequenceStateManager(prompt_len + 64, 1, 64, dev)
        tab = st.add_span_cache("c", R, torch.bfloat16)
        st.admit("a")
        st.reserve("a", prompt_len)
        st.upload()
        tab.pool.pool.view(torch.bfloat16).normal_(0, 0.3)
        pos = torch.arange(T, dtype=torch.int32, device=dev) if T > 1 else torch.tensor([prompt_len - 1], dtype=torch.int32, device=dev)
        slot = torch.zeros(T, dtype=torch.int32, device=dev)
        q = torch.randn(T, H * R, device=dev) * 0.1
        o = torch.empty(T, H * R, device=dev)
        sink = bf(H)
        one = lambda v: torch.tensor([v], dtype=torch.int32, device=dev)
        e_slot, e_row0, e_cnt = one(0), one(0), one(T)
        sec = _time(lambda: so.latent_window_attn_mc(q, tab, sink, pos, e_slot, e_row0, e_cnt, T, int(pos[-1]), H, s["window"], 0.1, out=o), 3)
        keys = sum(min(int(p) + 1, s["window"]) for p in pos.tolist())
        fl = 4.0 * keys * H * R
        by = (2.0 * R * min(prompt_len, s["window"] + T) + 8.0 * T * H * R)
        bound = max(fl / MFMA_BF16, by / HBM_BW)
        rows.append({"op": f"latent window attention T={T} H={H} R={R} window={s['window']}", "us": round(sec * 1e6, 1),
                     "tflops": round(fl / sec / 1e12, 2), "of_bound": round(bound / sec, 3)})
        # recurrence, convolution, norms: bytes
        es, er, ec = (torch.tensor([v], dtype=torch.int32, device=dev) for v in (0, 0, T))
        off = torch.arange(T, dtype=torch.int32, device=dev)
        g2, u, yv, out = torch.rand(T, 2 * C, device=dev), torch.randn(T, C, device=dev), torch.randn(T, C, device=dev), torch.empty(T, C, device=dev)
        lam, state, tail = bf(C), torch.zeros(1, C, device=dev), torch.zeros(1, s["taps"] - 1, C, device=dev)
        sec = _time(lambda: so.gated_recurrence(g2[:, :C], g2[:, C:], u, yv, lam, 8.0, state, es, er, ec, out=out, max_count=T), 3)
        rows.append({"op": f"gated recurrence T={T} C={C}", "us": round(sec * 1e6, 1), "of_bound": round(20.0 * T * C / HBM_BW / sec, 3)})
        cw, cb = bf(C, s["taps"]), bf(C)
        sec = _time(lambda: so.causal_conv_state(u, cw, cb, tail, slot, off, out=out), 3)
        rows.append({"op": f"causal conv T={T} C={C} taps={s['taps']}", "us": round(sec * 1e6, 1), "of_bound": round(8.0 * T * C / HBM_BW / sec, 3)})
        L = len(PATTERN)
        stack, xo, xm, gam, dwa = torch.randn(L + 1, T, W, device=dev), torch.empty(T, W, device=dev), torch.empty(T, W, device=dev), bf(W), bf(L + 1)
        n_mix = L // 2 + 1
        sec = _time(lambda: so.norm_residual_mix(stack[0], x[:, :W], gam, 1e-6, xo, stack, dwa, n_mix, xm), 3)
        rows.append({"op": f"norm + residual + depth mix of {n_mix} T={T}", "us": round(sec * 1e6, 1),
                     "of_bound": round(4.0 * T * W * (n_mix + 4) / HBM_BW / sec, 3)})
    return rows


def qwen2_equal_size(size, prompt_len, decode_steps=32):
    """the quantised decode runner on Qwen2 layers of the same width, depth and feed-forward parameter count (SwiGLU of 2/3 the width),
    int8 per-channel weights, 16-bit KV spans: prompt tokens / s and decode tokens / s at batch 1"""
    from . import decoder
    s = SIZES[size]
    inter = (s["ff"] * 2 // 3 + 127) // 128 * 128
    cfg = decoder.ModelConfig(f"qwen2-like-{size}", s["width"], len(PATTERN), s["heads"], max(1, s["heads"] // 8), s["dim"], inter, s["vocab"])
    model = decoder.build_random_model(cfg, decoder.QuantSpec(8, -1), seed=5)
    sess = decoder.DecodeSession(model, 1, max_len=prompt_len + decode_steps + 64, span_len=128)
    gen = torch.Generator().manual_seed(11)
    prompt = [int(t) for t in torch.randint(0, cfg.vocab, (prompt_len,), generator=gen)]
    out = {"model": f"{len(PATTERN)} Qwen2 layers, hidden {cfg.hidden}, {cfg.n_heads}/{cfg.n_kv} heads, SwiGLU {inter}, int8 per-channel weights"}
    out["prefill_tokens_per_s"] = round(prompt_len / _time(lambda: sess.prefill([prompt]), 3), 1)
    sess.prefill([prompt])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(decode_steps):
        sess.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / decode_steps
    out["decode_b1_tokens_per_s"], out["decode_b1_ms_per_step"] = round(1 / dt, 1), round(dt * 1e3, 3)
    return out


def run(args):
    from . import models
    from .engine import SeqEngine
    prompt_len = 2048
    res = {"metric": "prefill / decode throughput of the sequence engine (random Modanex models) beside Qwen2 layers of equal size",
           "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "prompt_len": prompt_len, "sizes": {}}
    for size in SIZES:
        cfg, t = random_model(size)
        eng = SeqEngine(models.resolve(cfg), cfg, t, dtype=torch.bfloat16, max_tokens=4 * (prompt_len + 128), max_slots=4)
        entry = {"layers": list(PATTERN), **{k: v for k, v in SIZES[size].items()}}
        entry["engine"] = engine_throughput(eng, cfg["vocab"], prompt_len)
        del eng, t
        torch.cuda.empty_cache()
        entry["operators"] = operator_table(size, prompt_len)
        try:
            entry["qwen2_equal_size"] = qwen2_equal_size(size, prompt_len)
        except Exception as e:  # noqa: BLE001  the line is still printed
            entry["qwen2_equal_size"] = {"error": f"{type(e).__name__}: {e}"[:300]}
        res["sizes"][size] = entry
    res["value"] = res["sizes"]["4k"]["engine"]["prefill_tokens_per_s"]
    return res
