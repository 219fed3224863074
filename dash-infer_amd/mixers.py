"""Token mixers and feed-forward blocks of the sequence engine, each with its constants as parameters.

A mixer maps the rows h [T, width] (f32) of one step -- portions of several sequences, described by the step context --
to rows of the same shape, reading and updating what its sequences left in the state manager:
  LatentWindowAttention  attention through a low-rank latent that alone is cached (paged), sliding window, softmax sink,
                         sigmoid output gate; a layer may read the latent cache another layer writes
  GatedLinearRecurrence  two-branch recurrent block: gelu branch x (short causal convolution -> block-diagonal gates ->
                         real-gated diagonal recurrence), f32 state and convolution tail per slot
  DenseMlp               down(act(up(h)))
Matrix products run in ctx.math (seq_ops.MATH_F32 / MATH_BF16); norms, scores, gates of the recurrence, decays and
state are f32 in both.
"""
import torch

from . import seq_ops as so


class StepContext:
    """One step's flat batch on the device.  ids / rows2: token and second-table rows; tok_*: per row; ent_*: per portion."""

    def __init__(self, T, E, ids, rows2, tok_slot, tok_pos, tok_off, ent_slot, ent_row0, ent_count, want_rows, math, eps):
        self.T, self.E = T, E
        self.ids, self.rows2, self.tok_slot, self.tok_pos, self.tok_off = ids, rows2, tok_slot, tok_pos, tok_off
        self.ent_slot, self.ent_row0, self.ent_count, self.want_rows = ent_slot, ent_row0, ent_count, want_rows
        self.math, self.eps = math, eps
        self.max_count, self.max_pos = T, 0     # host numbers: the largest portion and the last position of the step
        self.taps = None    # layer index -> [T, .] intermediate (diagnostics; None: off)

    def act_buffer(self, n, dtype=None):
        """[T, n] for an activation that only a product reads: bf16 under bf16 products (the product would round it anyway), else f32"""
        dt = dtype or (torch.bfloat16 if self.math == so.MATH_BF16 else torch.float32)
        return torch.empty(self.T, n, dtype=dt, device=self.ids.device)


class LatentWindowAttention:
    def __init__(self, key, heads, dim, vdim, kv_rank, q_rank, window, scale, w, state, cache_dtype, kv_from_key=None):
        """w: dq [q_rank, width], dq.norm, uq [heads*dim, q_rank], dkv [kv_rank, width] + dkv.norm (absent with kv_from_key),
        uk [heads*dim, kv_rank], uv [heads*vdim, kv_rank], sink [heads] (optional), g [heads*vdim, width], o [width, heads*vdim]"""
        self.H, self.D, self.V, self.R, self.Q, self.window, self.scale = heads, dim, vdim, kv_rank, q_rank, int(window or 0), float(scale)
        self.owns_cache = kv_from_key is None
        parts = [w["dq"]] + ([w["dkv"]] if self.owns_cache else []) + [w["g"]]
        self.w_in = torch.cat(parts, 0).contiguous()          # one product for everything that reads h
        self.c_lo = q_rank
        self.g_lo = q_rank + (kv_rank if self.owns_cache else 0)
        self.n_in = self.g_lo + heads * vdim
        self.dq_norm, self.uq = w["dq.norm"], w["uq"].contiguous()
        self.dkv_norm = w.get("dkv.norm")
        # scores against the latent itself: q' = W_uk[h]^T q_h, so that k = W_uk c never has to be formed
        self.uk_t = w["uk"].view(heads, dim, kv_rank).transpose(1, 2).contiguous()   # [H, R, D]
        self.uv = w["uv"].view(heads, vdim, kv_rank).contiguous()                      # [H, V, R]
        self.sink, self.o = w.get("sink"), w["o"].contiguous()
        assert self.uq.shape == (heads * dim, q_rank) and self.o.shape[1] == heads * vdim
        if self.owns_cache:
            self.table = state.add_span_cache(key, kv_rank, cache_dtype)
        else:
            self.table = state.tables[kv_from_key]
            assert self.table.row_elems == kv_rank, "a shared latent cache must have this layer's rank"
        self.mc = so.latent_attn_mc_supported(self.table) and (heads * kv_rank) % 4 == 0

    def __call__(self, ctx, h, h16=None):
        """h16: the bf16 copy of h where the producer made one (bf16 products read it: the same bits at half the traffic)"""
        a = so.linear(h16 if h16 is not None else h, self.w_in, act="sigmoid", act_cols=(self.g_lo, self.n_in), math=ctx.math)
        cq = so.rmsnorm(a[:, : self.Q], self.dq_norm, ctx.eps, out=ctx.act_buffer(self.Q))
        q = so.linear(cq, self.uq, math=ctx.math, out=ctx.act_buffer(self.H * self.D))
        if self.owns_cache:
            so.norm_span_append(self.table, a[:, self.c_lo: self.g_lo], self.dkv_norm, ctx.eps, ctx.tok_slot, ctx.tok_pos)
        ql = so.linear(q, self.uk_t, groups=self.H, math=ctx.math)
        if ctx.math == so.MATH_BF16 and self.mc:
            ol = so.latent_window_attn_mc(ql, self.table, self.sink, ctx.tok_pos, ctx.ent_slot, ctx.ent_row0, ctx.ent_count, ctx.max_count,
                                          ctx.max_pos, self.H, self.window, self.scale)
        else:
            ol = so.latent_window_attn(ql, self.table, self.sink, ctx.tok_slot, ctx.tok_pos, self.H, self.window, self.scale, math=ctx.math)
        og = so.linear(ol, self.uv, groups=self.H, mul=a[:, self.g_lo:], math=ctx.math, out=ctx.act_buffer(self.H * self.V))
        return so.linear(og, self.o, math=ctx.math)


class GatedLinearRecurrence:
    def __init__(self, key, width, blocks, taps, decay, w, state):
        """w: y [width, model], y.b, x [width, model], x.b, conv [width, taps], conv.b, ra / ri [blocks, bs, bs], ra.b / ri.b
        [blocks, bs], lam [width], o [model, width]"""
        assert width % blocks == 0 and w["conv"].shape == (width, taps)
        self.C, self.B, self.taps, self.decay = width, blocks, taps, float(decay)
        self.w_in = torch.cat([w["y"], w["x"]], 0).contiguous()
        self.b_in = torch.cat([w["y.b"], w["x.b"]], 0).contiguous()
        self.conv, self.conv_b = w["conv"].contiguous(), w["conv.b"].contiguous()
        self.w_gate = torch.cat([w["ra"], w["ri"]], 0).contiguous()           # [2B, bs, bs]: recurrence gates, then input gates
        self.b_gate = torch.cat([w["ra.b"], w["ri.b"]], 0).contiguous()
        self.lam, self.o = w["lam"].contiguous(), w["o"].contiguous()
        self.S = state.add_state(key + ".S", (width,))
        self.tail = state.add_state(key + ".tail", (taps - 1, width)) if taps > 1 else None

    def __call__(self, ctx, h, h16=None):
        C = self.C
        a = so.linear(h16 if h16 is not None else h, self.w_in, self.b_in, act="gelu_tanh", act_cols=(0, C), math=ctx.math)     # [y | x]
        y, x = a[:, :C], a[:, C:]
        u = so.causal_conv_state(x, self.conv, self.conv_b, self.tail, ctx.tok_slot, ctx.tok_off)
        if self.tail is not None:
            so.conv_tail_update(self.tail, x, self.taps, ctx.ent_slot, ctx.ent_row0, ctx.ent_count)
        g = so.linear(u, self.w_gate, self.b_gate, act="sigmoid", groups=2 * self.B, x_groups=self.B,
                      math=so.MATH_F32 if ctx.math == so.MATH_F32 else so.MATH_F32_STREAM)    # f32 products in both engines
        sy = so.gated_recurrence(g[:, :C], g[:, C:], u, y, self.lam, self.decay, self.S, ctx.ent_slot, ctx.ent_row0, ctx.ent_count,
                                 max_count=ctx.max_count)
        return so.linear(sy, self.o, math=ctx.math)


class DenseMlp:
    def __init__(self, up, down, act):
        self.up, self.down, self.act = up.contiguous(), down.contiguous(), act

    def __call__(self, ctx, h, h16=None):
        act = so.linear(h16 if h16 is not None else h, self.up, act=self.act, math=ctx.math, out=ctx.act_buffer(self.up.shape[0]))
        return so.linear(act, self.down, math=ctx.math)
