"""Vogusun: a decoder-only model whose layers run their token mixer and their feed-forward side by side.

  embedding   x = embed[token]
  layer i     h = dyt(x) = tanh(alpha x) * w + b  (a norm without statistics);  x <- x + (mixer(h) + ff(h))
              mixer: 'attention'    grouped-query attention, unit-RMS norm of queries and keys, rotary positions on pairs of
                                    neighbouring dimensions, a softmax sink of score 0, a sigmoid gate per head
                     'attention_2'  grouped-query attention with biases, rotary positions on the two halves of the rotated part with
                                    frequencies rescaled for longer contexts, tanh-capped scores
                     'gla'          gated linear attention: a decay per key channel, a matrix state per head
                     layers that say v_mix blend their values with those of the first such layer (same token)
              ff:    dense (gelu(gate h) * up h -> down) or a mixture of experts (top-k of the router's logits, clamped gated
                     units, weights = softmax over the chosen logits), or none
  head        logits = head . dyt(x; final.norm)
Sizes, layer order and constants come from config.json; tensor names are those of the checkpoint ('l<i>.mix.*', 'l<i>.mlp.*').
"""
import torch

from .. import mixers
from .. import seq_ops as so
from . import register


def _sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def _norm(tensors, name):
    """(alpha, weight, bias) of a dyt norm; the scalar is read once at load"""
    return float(tensors[name + ".alpha"].float().item()), tensors[name].contiguous(), tensors[name + ".b"].contiguous()


@register("Vogusun")
class Vogusun:
    engine = "sequence"
    VALUES_KEY = "values.first"

    def __init__(self, config, tensors, state, dtype):
        self.config = config
        self.width, self.vocab = int(config["width"]), int(config["vocab"])
        self.eps = float(config["norm"]["eps"])
        self.dtype = dtype
        self.math = so.MATH_BF16 if dtype == torch.bfloat16 else so.MATH_F32
        self.embed = tensors["embed"]
        assert self.embed.shape == (self.vocab, self.width)
        self.final_norm, self.head = _norm(tensors, "final.norm"), tensors["head"].contiguous()
        self.layers = []
        values_source = None     # the first layer that mixes values: the others blend with what it computed
        for i, lc in enumerate(config["layers"]):
            w, m, kind = _sub(tensors, f"l{i}."), lc["mixer"], lc["type"]
            mw = _sub(w, "mix.")
            if kind in ("attention", "attention_2"):
                vm = None
                if m.get("v_mix"):
                    if values_source is None:
                        values_source, vm = i, ("source", self.VALUES_KEY)
                    else:
                        sm = config["layers"][values_source]["mixer"]
                        if int(sm["kv_heads"]) * int(sm["vdim"]) != int(m["kv_heads"]) * int(m["vdim"]):
                            raise ValueError(f"layer {i}: its values cannot be mixed with those of layer {values_source} (other shape)")
                        vm = ("mix", self.VALUES_KEY, float(mw["vmix"].float().item()))
                rot = m.get("rot") or {}
                common = dict(rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_scaling=rot.get("scaling"),
                              value_mix=vm)
                if kind == "attention":
                    extra = dict(rot_layout="pairs", qk_norm=True, sink="zero", head_gate=True)
                else:
                    extra = dict(rot_layout="halves", softcap=m.get("softcap"))
                mixer = mixers.GroupedQueryAttention(f"l{i}.attn", int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                                     float(m["scale"]), mw, state, dtype, **common, **extra)
            elif kind == "gla":
                mixer = mixers.GatedLinearAttention(f"l{i}.gla", int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"]), mw, state)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            ff, fc = None, lc.get("mlp")
            if fc is not None:
                fw = _sub(w, "mlp.")
                if fc["kind"] == "dense":
                    ff = mixers.GatedMlp(fw["gate"], fw["up"], fw["down"], "gelu_tanh")
                    assert fw["gate"].shape == (int(fc["ff"]), self.width)
                elif fc["kind"] == "moe":
                    n = int(fc["router"]["experts"])
                    ff = mixers.ExpertMlp(fw["router"], fw["router.b"], [fw[f"e{e}.gate"] for e in range(n)], [fw[f"e{e}.up"] for e in range(n)],
                                          [fw[f"e{e}.down"] for e in range(n)], int(fc["router"]["top"]), float(fc["expert"]["limit"]))
                    assert fw["e0.gate"].shape == (int(fc["expert"]["ff"]), self.width)
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {fc['kind']!r}")
            self.layers.append((_norm(w, "norm1"), mixer, ff))

    @classmethod
    def from_config(cls, config, tensors, state, dtype):
        return cls(config, tensors, state, dtype)

    def second_rows(self, prev, tokens):
        return None      # one embedding table

    def forward(self, ctx):
        """-> the residual stream after the last layer, [T, width] f32"""
        bf = self.math == so.MATH_BF16        # bf16 products read a bf16 copy of the norm's output: the same bits at half the traffic
        x = so.embed_sum(ctx.ids, self.embed)
        h, h16 = so.add_dyt(x, norm=self.layers[0][0], want16=bf) if self.layers else (None, None)
        for i, (_, mixer, ff) in enumerate(self.layers):
            mo = mixer(ctx, h, h16)
            fo = ff(ctx, h, h16) if ff is not None else None
            nxt = self.layers[i + 1][0] if i + 1 < len(self.layers) else None
            h, h16 = so.add_dyt(x, mo, fo, norm=nxt, x_out=x, want16=bf)
            if ctx.taps is not None:
                ctx.taps[i] = x.clone()
        return x

    def logits(self, ctx, x, rows):
        """rows: int32 device tensor of the row indices whose logits are wanted -> f32 [len(rows), vocab]"""
        h, h16 = so.add_dyt(x, norm=self.final_norm, row_idx=rows, want16=self.math == so.MATH_BF16)
        return so.linear(h16 if h16 is not None else h, self.head, math=ctx.math)
