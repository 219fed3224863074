"""Modanex: a decoder-only model of mixed layers on a depth-weighted residual stream.

  embedding      x = embed[token] (+ bigram[(prev * mul_prev + token * mul_cur) mod buckets]; the row after the buckets for a
                 sequence's first token)
  layer i        x <- x + norm1(mixer(x));  x <- x + norm2(mlp(x)) where the layer has one: RMS norms on the sublayers'
                 OUTPUTS, the sublayers read the stream itself.  mixer: latent window attention or a gated linear recurrence
  depth average  with X_0 the embedding and X_(i+1) the result of layer i, the next layer (or the head) reads
                 sum_{j <= i+1} dwa_i[j] X_j
  head           logits = head . rmsnorm(x; final.norm)
Sizes, layer order and constants come from config.json; tensor names are those of the checkpoint ('l<i>.mix.*', ...).
"""
import torch

from .. import mixers
from .. import seq_ops as so
from . import register

RECURRENCE_DECAY = 8.0   # log a = -8 * r * softplus(lam): fixed by the design


def _sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


@register("Modanex")
class Modanex:
    engine = "sequence"

    def __init__(self, config, tensors, state, dtype):
        self.config = config
        self.width, self.vocab = int(config["width"]), int(config["vocab"])
        self.eps = float(config["norm"]["eps"])
        self.dtype = dtype
        self.math = so.MATH_BF16 if dtype == torch.bfloat16 else so.MATH_F32
        self.embed = tensors["embed"]
        assert self.embed.shape == (self.vocab, self.width)
        bg = (config.get("embedding") or {}).get("bigram")
        self.bigram = None
        if bg:
            self.bigram = tensors["bigram"]
            self.buckets, self.mul_prev, self.mul_cur = int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])
            assert self.bigram.shape == (self.buckets + 1, self.width)
        self.final_norm, self.head = tensors["final.norm"], tensors["head"].contiguous()
        self.layers = []
        for i, lc in enumerate(config["layers"]):
            w, m = _sub(tensors, f"l{i}."), lc["mixer"]
            mw = _sub(w, "mix.")
            if lc["type"] == "latent_attention":
                src = m.get("kv_from")
                if src is not None:
                    sm = config["layers"][src]
                    if sm["type"] != "latent_attention" or "kv_from" in sm["mixer"] or int(sm["mixer"]["kv_rank"]) != int(m["kv_rank"]):
                        raise ValueError(f"layer {i}: kv_from {src} is not a layer with a latent cache of rank {m['kv_rank']}")
                mixer = mixers.LatentWindowAttention(
                    f"l{i}.latent", int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), int(m["q_rank"]),
                    (m.get("mask") or {}).get("size"), m["scale"], mw, state, dtype, None if src is None else f"l{src}.latent")
            elif lc["type"] == "rglru":
                mixer = mixers.GatedLinearRecurrence(f"l{i}.rglru", int(m["width"]), int(m["blocks"]), int(m["conv"]), RECURRENCE_DECAY, mw, state)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
            mlp = None
            if lc.get("mlp") is not None:
                if lc["mlp"].get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {lc['mlp']['kind']!r}")
                mlp = mixers.DenseMlp(w["mlp.up"], w["mlp.down"], "gelu_erf")
                assert w["mlp.up"].shape == (int(lc["mlp"]["ff"]), self.width)
            self.layers.append((mixer, w["norm1"], mlp, w.get("norm2"), w.get("dwa")))

    @classmethod
    def from_config(cls, config, tensors, state, dtype):
        return cls(config, tensors, state, dtype)

    # -- host side of the embedding: the second table's row of every token ------------------------------------------
    uses_previous_token = True

    def second_rows(self, prev, tokens):
        """prev: the sequence's last token before `tokens` (None at its start)"""
        if self.bigram is None:
            return None
        rows, p = [], prev
        for t in tokens:
            rows.append(self.buckets if p is None else (p * self.mul_prev + t * self.mul_cur) % self.buckets)
            p = t
        return rows

    # -- device side ----------------------------------------------------------------------------------------------------
    def forward(self, ctx):
        """-> the stream the head reads, [T, width] f32"""
        T, W, L = ctx.T, self.width, len(self.layers)
        dev = self.embed.device
        stack = torch.empty(L + 1, T, W, dtype=torch.float32, device=dev)
        so.embed_sum(ctx.ids, self.embed, ctx.rows2, self.bigram, out=stack[0])
        cur, cur16 = stack[0], None
        bf = self.math == so.MATH_BF16      # bf16 copies of what the products read, written by the kernel that makes the f32 rows
        xr = torch.empty(T, W, dtype=torch.float32, device=dev)
        xr16 = torch.empty(T, W, dtype=torch.bfloat16, device=dev) if bf else None
        mixed = [torch.empty(T, W, dtype=torch.float32, device=dev) for _ in range(2)]
        mixed16 = [torch.empty(T, W, dtype=torch.bfloat16, device=dev) if bf else None for _ in range(2)]
        for i, (mixer, norm1, mlp, norm2, dwa) in enumerate(self.layers):
            n_mix = i + 2 if dwa is not None else 0
            nxt, nxt16 = (mixed[i & 1], mixed16[i & 1]) if n_mix else (xr, xr16)
            mo = mixer(ctx, cur, cur16)
            if mlp is None:
                so.norm_residual_mix(cur, mo, norm1, ctx.eps, xr, stack, dwa, n_mix, nxt if n_mix else None, next16=nxt16)
            else:
                so.norm_residual_mix(cur, mo, norm1, ctx.eps, xr, next16=xr16)
                f = mlp(ctx, xr, xr16)
                so.norm_residual_mix(xr, f, norm2, ctx.eps, xr, stack, dwa, n_mix, nxt if n_mix else None, next16=nxt16)
            if not n_mix:      # no depth average: the layer's result goes on as it is
                xr = torch.empty(T, W, dtype=torch.float32, device=dev)
                xr16 = torch.empty(T, W, dtype=torch.bfloat16, device=dev) if bf else None
            cur, cur16 = nxt, nxt16
            if ctx.taps is not None:
                ctx.taps[i] = cur.clone()
        return cur

    def logits(self, ctx, x, rows):
        """rows: int32 device tensor of the row indices whose logits are wanted -> f32 [len(rows), vocab]"""
        xn = so.rmsnorm(x, self.final_norm, ctx.eps, row_idx=rows)
        return so.linear(xn, self.head, math=ctx.math)
