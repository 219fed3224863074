"""Tensor-level wrappers over libdashinfer_hip_seq.so (torch: device memory and streams only).

Activations between operators are f32 tensors, possibly column slices of a wider buffer (row stride = stride(0)); weights
stay in the type the checkpoint stores (bf16 or f32: both widen to f32 exactly).  `math` selects how dihip_linear
multiplies: seq_capi.MATH_F32 (every product and sum in f32) or MATH_BF16 (bf16 operands, f32 accumulation).
"""
import ctypes as C

import torch

from . import seq_capi
from .seq_capi import ACT, MATH_BF16, MATH_F32, MATH_F32_STREAM, check, lib

_DT = {torch.float32: seq_capi.F32, torch.bfloat16: seq_capi.BF16}


def dt(t):
    return _DT[t.dtype]


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _rows(t):
    assert t.dim() == 2 and t.stride(1) == 1, "row-major rows (a column slice of a wider buffer is fine)"
    return t.stride(0)


def linear(x, w, bias=None, out=None, act=None, act_cols=None, mul=None, math=MATH_F32, groups=1, x_groups=None):
    """y = epilogue(x . w^T + bias).  w: [N, K] (groups == 1) or [groups, N, K]; x: [T, x_groups * K] (group g reads the K
    columns from (g % x_groups) * K); y: [T, groups * N].  act on the output columns act_cols = (lo, hi) (default: all);
    mul: f32 [T, groups * N] multiplied on the output."""
    if w.dim() == 2:
        N, K = w.shape
    else:
        assert w.shape[0] == groups
        _, N, K = w.shape
    xg = groups if x_groups is None else x_groups
    T = x.shape[0]
    assert x.shape[1] == xg * K and w.is_contiguous() and (bias is None or (bias.is_contiguous() and bias.dtype == w.dtype))
    y = out if out is not None else torch.empty(T, groups * N, dtype=torch.float32, device=x.device)
    assert y.shape == (T, groups * N)
    lo, hi = (0, groups * N) if act_cols is None else act_cols
    if act is None:
        lo = hi = 0
    check(lib().dihip_linear(stream(), ptr(x), dt(x), _rows(x), K, xg, ptr(w), dt(w), ptr(bias), ptr(y), dt(y), _rows(y), N,
                             ptr(mul), _rows(mul) if mul is not None else 0, T, N, K, groups, ACT[act], lo, hi, math), "dihip_linear")
    return y


def embed_sum(ids, table, rows2=None, table2=None, out=None):
    T, K = ids.shape[0], table.shape[1]
    h = out if out is not None else torch.empty(T, K, dtype=torch.float32, device=table.device)
    assert table2 is None or (table2.dtype == table.dtype and table2.shape[1] == K)
    check(lib().dihip_embed_sum(stream(), ptr(h), ptr(ids), ptr(table), ptr(rows2), ptr(table2), dt(table), T, K), "dihip_embed_sum")
    return h


def rmsnorm(x, gamma, eps, row_idx=None, out=None):
    M = x.shape[0] if row_idx is None else row_idx.shape[0]
    K = gamma.shape[0]
    assert x.shape[1] == K and x.dtype == torch.float32
    y = out if out is not None else torch.empty(M, K, dtype=torch.float32, device=x.device)
    check(lib().dihip_rmsnorm_strided(stream(), ptr(y), dt(y), _rows(y), ptr(x), _rows(x), ptr(row_idx), ptr(gamma), dt(gamma), float(eps),
                                      M, K), "dihip_rmsnorm_strided")
    return y


def norm_span_append(table, x, gamma, eps, tok_slot, tok_pos):
    """table: a SpanTable (seq_state) of rows of x.shape[1] elements"""
    T, K = x.shape
    assert K == table.row_elems and x.dtype == torch.float32
    check(lib().dihip_norm_span_append(stream(), ptr(table.ptrs), table.max_spans, table.span_len, _DT[table.dtype], ptr(x), _rows(x),
                                       ptr(gamma), dt(gamma), float(eps), ptr(tok_slot), ptr(tok_pos), T, K), "dihip_norm_span_append")


def norm_residual_mix(x_in, m, gamma, eps, x_out, stack=None, mix_w=None, n_mix=0, x_mix=None, next16=None):
    """next16: optional bf16 [T, K] copy of what the next product reads (x_mix where n_mix > 0, else x_out)"""
    T, K = x_in.shape
    assert x_in.is_contiguous() and x_out.is_contiguous() and m.shape == (T, K)
    assert next16 is None or (next16.dtype == torch.bfloat16 and next16.is_contiguous() and next16.shape == (T, K))
    if n_mix:
        assert stack.is_contiguous() and stack.shape[0] >= n_mix and x_mix.is_contiguous() and mix_w.shape[0] >= n_mix
    check(lib().dihip_norm_residual_mix(stream(), ptr(x_out), ptr(x_in), ptr(m), _rows(m), ptr(gamma), dt(gamma), float(eps),
                                        ptr(stack), stack.stride(0) if n_mix else 0, ptr(mix_w), n_mix, ptr(x_mix), ptr(next16), T, K),
          "dihip_norm_residual_mix")
    return x_out


def latent_window_attn(q, table, sink, tok_slot, tok_pos, H, window, scale, math=MATH_F32, out=None):
    T = q.shape[0]
    R = table.row_elems
    assert q.shape[1] == H * R and q.dtype == torch.float32
    o = out if out is not None else torch.empty(T, H * R, dtype=torch.float32, device=q.device)
    check(lib().dihip_latent_window_attn(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(table.ptrs), table.max_spans, table.span_len,
                                         _DT[table.dtype], ptr(sink), dt(sink) if sink is not None else 0, ptr(tok_slot), ptr(tok_pos),
                                         T, H, R, int(window), float(scale), math), "dihip_latent_window_attn")
    return o


def latent_attn_mc_supported(table):
    return bool(lib().dihip_latent_window_attn_mc_supported(table.row_elems, table.span_len, _DT[table.dtype]))


def latent_window_attn_mc(q, table, sink, tok_pos, ent_slot, ent_row0, ent_count, max_count, max_pos, H, window, scale, out=None, nsplit=None):
    """the matrix-core form (bf16 cache): rows as portions; max_count / max_pos: the largest portion and position of the step
    (host numbers: they size the grid and the split of the key walk)"""
    T, R, E = q.shape[0], table.row_elems, ent_slot.shape[0]
    o = out if out is not None else torch.empty(T, H * R, dtype=torch.float32, device=q.device)
    if nsplit is None:       # fill the chip: ~2 workgroups per CU; at least 2 key tiles (64 keys) per workgroup
        blocks = max(1, E * ((max_count * H + 63) // 64))
        keys = min(max_pos + 1, window) if window > 0 else max_pos + 1
        nsplit = max(1, min(512 // blocks, (keys + 63) // 64))
    ws = None
    if nsplit > 1:
        ws = torch.empty(int(lib().dihip_latent_window_attn_mc_workspace_bytes(T, H, R, nsplit)), dtype=torch.uint8, device=q.device)
    check(lib().dihip_latent_window_attn_mc(stream(), ptr(o), _rows(o), ptr(q), _rows(q), ptr(table.ptrs), table.max_spans, table.span_len,
                                            ptr(sink), dt(sink) if sink is not None else 0, ptr(tok_pos), ptr(ent_slot), ptr(ent_row0),
                                            ptr(ent_count), E, int(max_count), T, H, R, int(window), float(scale), int(nsplit), ptr(ws),
                                            ws.numel() if ws is not None else 0), "dihip_latent_window_attn_mc")
    return o


def causal_conv_state(x, w, bias, tail, tok_slot, tok_off, out=None):
    T, Cn = x.shape
    taps = w.shape[1]
    u = out if out is not None else torch.empty(T, Cn, dtype=torch.float32, device=x.device)
    check(lib().dihip_causal_conv_state(stream(), ptr(u), _rows(u), ptr(x), _rows(x), ptr(w), ptr(bias), dt(w), ptr(tail), ptr(tok_slot),
                                        ptr(tok_off), T, Cn, taps), "dihip_causal_conv_state")
    return u


def conv_tail_update(tail, x, taps, ent_slot, ent_row0, ent_count):
    check(lib().dihip_conv_tail_update(stream(), ptr(tail), ptr(x), _rows(x), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                       ent_slot.shape[0], x.shape[1], taps), "dihip_conv_tail_update")


CHUNKED_RECURRENCE_ROWS = 256   # portions from this length on run as chunks side by side


def gated_recurrence(r, i, u, y, lam, decay, state, ent_slot, ent_row0, ent_count, out=None, max_count=None):
    """max_count: the step's largest portion (a host number); given and >= CHUNKED_RECURRENCE_ROWS: the chunk-parallel form"""
    T, Cn = u.shape
    assert _rows(r) == _rows(i)
    o = out if out is not None else torch.empty(T, Cn, dtype=torch.float32, device=u.device)
    if max_count is not None and max_count >= CHUNKED_RECURRENCE_ROWS:
        E = ent_slot.shape[0]
        ws = torch.empty(int(lib().dihip_gated_recurrence_chunked_workspace_bytes(E, max_count, Cn)), dtype=torch.uint8, device=u.device)
        check(lib().dihip_gated_recurrence_chunked(stream(), ptr(o), _rows(o), ptr(r), ptr(i), _rows(r), ptr(u), _rows(u), ptr(y), _rows(y),
                                                   ptr(lam), dt(lam), float(decay), ptr(state), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                                   E, int(max_count), Cn, ptr(ws), ws.numel()), "dihip_gated_recurrence_chunked")
        return o
    check(lib().dihip_gated_recurrence(stream(), ptr(o), _rows(o), ptr(r), ptr(i), _rows(r), ptr(u), _rows(u), ptr(y), _rows(y), ptr(lam),
                                       dt(lam), float(decay), ptr(state), ptr(ent_slot), ptr(ent_row0), ptr(ent_count),
                                       ent_slot.shape[0], Cn), "dihip_gated_recurrence")
    return o
