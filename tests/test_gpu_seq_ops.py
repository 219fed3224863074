"""Every operator of libdashinfer_hip_seq.so alone against the float64 restatement in oracle/seq_model.py."""
import numpy as np
import pytest
import torch

from tests.conftest import load_pkg
from oracle import seq_model as om
from tests.seq_helpers import rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def so():
    load_pkg()
    from dash_infer_amd import seq_ops
    return seq_ops


def bf(a):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16)


def dev(a, dt=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dt).cuda()


@pytest.mark.parametrize("T,N,K,groups", [(1, 40, 64, 1), (3, 33, 100, 1), (5, 130, 72, 1), (17, 96, 256, 1), (200, 150, 152, 1),
                                          (4, 24, 32, 3), (70, 20, 28, 5), (130, 128, 128, 2)])
@pytest.mark.parametrize("wdt", [torch.bfloat16, torch.float32])
def test_linear_f32_and_bf16(so, T, N, K, groups, wdt):
    rng = np.random.default_rng(T * 1000 + N + K)
    x = rng.normal(0, 1, (T, groups * K)).astype(np.float32)
    w = bf(rng.normal(0, 1 / np.sqrt(K), (groups, N, K))).float().numpy()
    b = bf(rng.normal(0, 0.3, (groups, N))).float().numpy()
    mul = rng.normal(0, 1, (T, groups * N)).astype(np.float32)
    lo, hi = N // 3, groups * N - 2
    def ref(xr, wr):
        y = np.stack([xr[:, g * K:(g + 1) * K].astype(np.float64) @ wr[g].astype(np.float64).T + b[g] for g in range(groups)], 1).reshape(T, groups * N)
        y[:, lo:hi] = om.gelu_tanh(y[:, lo:hi])
        return y * mul
    wt, bt = dev(w.reshape(groups * N, K) if groups == 1 else w, wdt), dev(b, wdt)
    if groups == 1:
        wt, bt = wt.view(N, K), bt.view(N)
    y = so.linear(dev(x), wt, bt, act="gelu_tanh", act_cols=(lo, hi), mul=dev(mul), math=so.MATH_F32, groups=groups)
    assert rel_err(y.cpu().numpy(), ref(x, w)) < 2e-6
    y16 = so.linear(dev(x), wt, bt, act="gelu_tanh", act_cols=(lo, hi), mul=dev(mul), math=so.MATH_BF16, groups=groups)
    xr = bf(x).float().numpy()
    assert rel_err(y16.cpu().numpy(), ref(xr, w)) < 2e-5      # same rounded operands, f32 accumulation


def test_linear_rows_do_not_depend_on_the_batch(so):
    rng = np.random.default_rng(5)
    K, N = 192, 100
    x, w = dev(rng.normal(0, 1, (150, K))), dev(rng.normal(0, 0.1, (N, K)), torch.bfloat16)
    full = so.linear(x, w, math=so.MATH_F32)
    for lo, hi in ((0, 1), (7, 9), (64, 131), (149, 150)):
        assert torch.equal(so.linear(x[lo:hi].contiguous(), w, math=so.MATH_F32), full[lo:hi])
    full16 = so.linear(x, w, math=so.MATH_BF16)
    for lo, hi in ((0, 1), (7, 12), (30, 47)):     # the streaming kernel sums in another order than the matrix cores
        assert rel_err(so.linear(x[lo:hi].contiguous(), w, math=so.MATH_BF16).cpu(), full16[lo:hi].cpu()) < 1e-5
    assert torch.equal(so.linear(x[3:40].contiguous(), w, math=so.MATH_BF16), full16[3:40])


def test_linear_strided_input_and_output(so):
    rng = np.random.default_rng(6)
    big = dev(rng.normal(0, 1, (9, 200)))
    w = dev(rng.normal(0, 0.1, (48, 72)), torch.bfloat16)
    out = torch.zeros(9, 100, device="cuda")
    so.linear(big[:, 56:128], w, out=out[:, 8:56], math=so.MATH_F32)
    want = big[:, 56:128].double().cpu().numpy() @ w.double().cpu().numpy().T
    assert rel_err(out[:, 8:56].cpu().numpy(), want) < 2e-6 and float(out[:, :8].abs().max()) == 0 and float(out[:, 56:].abs().max()) == 0


def test_embed_sum(so):
    rng = np.random.default_rng(7)
    e, b2 = bf(rng.normal(0, 1, (50, 72))), bf(rng.normal(0, 1, (11, 72)))
    ids, rows = [3, 49, 0, 7], [10, 0, 5, 5]
    h = so.embed_sum(torch.tensor(ids, dtype=torch.int32).cuda(), e.cuda(), torch.tensor(rows, dtype=torch.int32).cuda(), b2.cuda())
    assert torch.equal(h.cpu(), e[ids].float() + b2[rows].float())
    assert torch.equal(so.embed_sum(torch.tensor(ids, dtype=torch.int32).cuda(), e.cuda()).cpu(), e[ids].float())


def test_rmsnorm_strided_with_row_index(so):
    rng = np.random.default_rng(8)
    x, g = rng.normal(0, 3, (6, 300)).astype(np.float32), bf(1 + 0.1 * rng.normal(size=100))
    idx = [4, 0, 5]
    y = so.rmsnorm(dev(x)[:, 100:200], g.cuda(), 1e-3, row_idx=torch.tensor(idx, dtype=torch.int32).cuda())
    assert rel_err(y.cpu().numpy(), om.rms_norm(x[idx, 100:200], g.float().numpy(), 1e-3)) < 2e-6
    tiny = np.full((1, 100), 1e-4, np.float32)      # eps inside the root decides here
    assert rel_err(so.rmsnorm(dev(tiny), g.cuda(), 1e-3).cpu().numpy(), om.rms_norm(tiny, g.float().numpy(), 1e-3)) < 2e-6


def test_norm_residual_mix(so):
    rng = np.random.default_rng(9)
    T, K, n = 5, 72, 4
    stack = rng.normal(0, 1, (n, T, K)).astype(np.float32)
    m, x_in, g = rng.normal(0, 2, (T, 80)).astype(np.float32), rng.normal(0, 1, (T, K)).astype(np.float32), bf(1 + 0.1 * rng.normal(size=K))
    wmix = bf(rng.normal(0.5, 0.5, n))
    st, xo, xm = dev(stack), torch.empty(T, K, device="cuda"), torch.empty(T, K, device="cuda")
    so.norm_residual_mix(dev(x_in), dev(m)[:, 3:75], g.cuda(), 1e-5, xo, st, wmix.cuda(), n, xm)
    want = x_in + om.rms_norm(m[:, 3:75], g.float().numpy(), 1e-5)
    assert rel_err(xo.cpu().numpy(), want) < 2e-6 and rel_err(st[n - 1].cpu().numpy(), want) < 2e-6
    mix = sum(float(wmix[j]) * (stack[j].astype(np.float64) if j < n - 1 else want) for j in range(n))
    assert rel_err(xm.cpu().numpy(), mix) < 2e-6
    xo2 = torch.empty(T, K, device="cuda")
    so.norm_residual_mix(dev(x_in), dev(m)[:, 3:75], g.cuda(), 1e-5, xo2)
    assert torch.equal(xo2, xo)


# ---- attention over the paged latent cache ------------------------------------------------------------------------------------
def filled_cache(rows, dtype, slots=2, slot_of=1, span_len=64):
    """a state manager whose slot `slot_of` holds `rows` [n, R] in pages that are NOT consecutive"""
    load_pkg()
    from dash_infer_amd.seq_state import SequenceStateManager
    n, R = rows.shape
    st = SequenceStateManager(max_tokens=2 * n + 4 * span_len, max_slots=slots, span_len=span_len)
    tab = st.add_span_cache("t", R, dtype)
    for s in range(slot_of):     # other requests take the first slots and every other page
        st.admit(("x", s))
    st.admit("a")
    for k in range(st.pages_for(n)):
        st.reserve(("x", 0), (k + 1) * span_len) if slot_of else None
        st.reserve("a", min(n, (k + 1) * span_len))
    slot = st.live["a"]
    assert slot.index == slot_of
    for k, p in enumerate(slot.pages):
        v = tab.pool.span_view(p).view(dtype).view(span_len, R)
        part = rows[k * span_len:(k + 1) * span_len]
        v[: len(part)] = torch.from_numpy(part).to(dtype).cuda()
    st.upload()
    return st, tab, slot


def attn_ref(q, rows, pos, H, window, scale, sink):
    R = rows.shape[1]
    out = np.zeros((len(pos), H * R))
    for t, p in enumerate(pos):
        lo = max(0, p - window + 1) if window else 0
        for h in range(H):
            s = rows[lo:p + 1].astype(np.float64) @ q[t, h * R:(h + 1) * R].astype(np.float64) * scale
            out[t, h * R:(h + 1) * R] = om.sink_softmax_window(s, rows[lo:p + 1].astype(np.float64), None if sink is None else sink[h])
    return out


@pytest.mark.parametrize("cdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("R,H,window", [(48, 3, 37), (64, 1, 64), (80, 5, 130), (128, 2, 0), (200, 4, 65)])
def test_latent_window_attn_edges_pages_and_far_keys(so, cdt, R, H, window):
    """One cached row stands out (its score dominates and its content is recognisable): queries that must just see it, just
    not see it, see it across page borders or from hundreds of positions away -- as a prompt's rows and as single rows."""
    rng = np.random.default_rng(R + window)
    n = 400
    rows = rng.normal(0, 0.3, (n, R)).astype(np.float32)
    spikes = [0, 63, 64, 130, 255]
    qdir = rng.normal(0, 1, R).astype(np.float32)
    qdir /= np.linalg.norm(qdir)
    for j in spikes:
        rows[j] = 3.0 * qdir + rng.normal(0, 0.05, R)
    if cdt == torch.bfloat16:
        rows = torch.from_numpy(rows).to(torch.bfloat16).float().numpy()
    st, tab, slot = filled_cache(rows, cdt)
    sink = bf(rng.normal(0, 1, H))
    w = window or n
    pos = sorted({p for j in spikes for p in (j, j + 1, j + w - 2, j + w - 1, j + w, j + w + 1) if 0 <= p < n} | {n - 1, 1, 2, 65, 127, 128, 129})
    q = (rng.normal(0, 0.2, (len(pos), H * R)) + np.tile(4.0 * qdir, H)).astype(np.float32)
    want = attn_ref(q, rows, pos, H, window, 0.5, sink.float().numpy())
    tslot = torch.full((len(pos),), slot.index, dtype=torch.int32).cuda()
    got = so.latent_window_attn(dev(q), tab, sink.cuda(), tslot, torch.tensor(pos, dtype=torch.int32).cuda(), H, window, 0.5)
    assert rel_err(got.cpu().numpy(), want) < 1e-5
    # the spike really decides: leaving the window's last key out (or taking one more in) would be seen
    shifted = attn_ref(q, rows, pos, H, (window + 1) if window else 0, 0.5, sink.float().numpy())
    if window:
        assert rel_err(shifted, want) > 0.05
    for k in (0, len(pos) // 2, len(pos) - 1):      # single rows (decoding) give the same numbers
        one = so.latent_window_attn(dev(q[k:k + 1]), tab, sink.cuda(), tslot[:1], torch.tensor(pos[k:k + 1], dtype=torch.int32).cuda(), H, window, 0.5)
        assert torch.equal(one[0], got[k])
    nosink = so.latent_window_attn(dev(q), tab, None, tslot, torch.tensor(pos, dtype=torch.int32).cuda(), H, window, 0.5)
    assert rel_err(nosink.cpu().numpy(), attn_ref(q, rows, pos, H, window, 0.5, None)) < 1e-5
    assert rel_err(nosink.cpu().numpy(), want) > 1e-3   # a sink that is left out shows


def test_norm_span_append_at_page_borders(so):
    rng = np.random.default_rng(3)
    R = 48
    st, tab, slot = filled_cache(np.zeros((200, R), np.float32), torch.float32)
    x, g = rng.normal(0, 2, (6, 100)).astype(np.float32), bf(1 + 0.1 * rng.normal(size=R))
    pos = [62, 63, 64, 65, 127, 128]
    so.norm_span_append(tab, dev(x)[:, 10:58], g.cuda(), 1e-4, torch.full((6,), slot.index, dtype=torch.int32).cuda(),
                        torch.tensor(pos, dtype=torch.int32).cuda())
    got = tab.rows(slot.index, slot.pages, 200).cpu().numpy()
    assert rel_err(got[pos], om.rms_norm(x[:, 10:58], g.float().numpy(), 1e-4)) < 2e-6
    rest = np.delete(got, pos, 0)
    assert float(np.abs(rest).max()) == 0


# ---- convolution and recurrence with per-slot state ---------------------------------------------------------------------------
def entries(portions, slots):
    """flat batch of portions [(slot, n)]: tok_slot, tok_off, ent_slot, ent_row0, ent_count on the device"""
    ts, to, es, er, ec, row = [], [], [], [], [], 0
    for s, n in portions:
        ts += [s] * n
        to += range(n)
        es.append(s)
        er.append(row)
        ec.append(n)
        row += n
    i32 = lambda a: torch.tensor(a, dtype=torch.int32).cuda()
    return i32(ts), i32(to), i32(es), i32(er), i32(ec)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_causal_conv_in_portions_of_two_sequences(so, taps):
    rng = np.random.default_rng(taps)
    C, n = 70, 40
    xa, xb = rng.normal(0, 1, (n, C)).astype(np.float32), rng.normal(0, 1, (n, C)).astype(np.float32)
    w, b = bf(rng.normal(0, 0.5, (C, taps))), bf(rng.normal(0, 0.1, C))
    want_a, want_b = om.causal_conv(xa.astype(np.float64), w.double().numpy(), b.double().numpy()), om.causal_conv(xb.astype(np.float64), w.double().numpy(), b.double().numpy())
    tail = torch.zeros(3, max(taps - 1, 1), C, device="cuda")
    got_a, got_b, at_a, at_b = [], [], 0, 0
    for na, nb in ((1, 5), (1, 2), (2, 1), (6, 1), (1, 1), (3, 9), (26, 21)):
        ts, to, es, er, ec = entries([(2, na), (0, nb)], 3)
        x = dev(np.concatenate([xa[at_a:at_a + na], xb[at_b:at_b + nb]]))
        u = so.causal_conv_state(x, w.cuda(), b.cuda(), tail if taps > 1 else None, ts, to)
        if taps > 1:
            so.conv_tail_update(tail, x, taps, es, er, ec)
        got_a.append(u[:na].cpu().numpy())
        got_b.append(u[na:].cpu().numpy())
        at_a, at_b = at_a + na, at_b + nb
    assert rel_err(np.concatenate(got_a), want_a) < 2e-6 and rel_err(np.concatenate(got_b), want_b) < 2e-6


def test_gated_recurrence_portions_long_decode_and_state(so):
    rng = np.random.default_rng(11)
    C, n = 100, 300
    u, y = rng.normal(0, 1, (n, C)).astype(np.float32), rng.normal(0, 1, (n, C)).astype(np.float32)
    r, i = rng.uniform(0, 1, (n, C)).astype(np.float32), rng.uniform(0, 1, (n, C)).astype(np.float32)
    lam = bf(rng.normal(-2, 2, C))       # decays from almost 1 to almost 0
    want = om.gated_recurrence(u.astype(np.float64), r, i, lam.double().numpy(), 8.0) * y
    state = torch.zeros(2, C, device="cuda")
    state[0] = 7.0                        # another slot's state is not touched
    got, at = [], 0
    for k in [50, 2, 1, 9, 17] + [1] * 221:
        ts, to, es, er, ec = entries([(1, k)], 2)
        sl = slice(at, at + k)
        got.append(so.gated_recurrence(dev(r[sl]), dev(i[sl]), dev(u[sl]), dev(y[sl]), lam.cuda(), 8.0, state, es, er, ec).cpu().numpy())
        at += k
    assert at == n and rel_err(np.concatenate(got), want) < 5e-6
    assert float((state[0] - 7.0).abs().max()) == 0
    whole = torch.zeros(2, C, device="cuda")
    ts, to, es, er, ec = entries([(1, n)], 2)
    one = so.gated_recurrence(dev(r), dev(i), dev(u), dev(y), lam.cuda(), 8.0, whole, es, er, ec)
    assert torch.equal(one.cpu(), torch.from_numpy(np.concatenate(got))) and torch.equal(whole[1], state[1])


@pytest.mark.parametrize("R,H,window,nsplit", [(64, 3, 37, 1), (64, 1, 64, 3), (128, 5, 130, 1), (96, 2, 0, 4), (256, 4, 65, 2), (512, 2, 200, 1), (32, 7, 33, None)])
def test_latent_window_attn_on_the_matrix_cores(so, R, H, window, nsplit):
    """the same edges, page borders and far keys through the matrix-core kernel: two portions of two slots and single rows,
    with and without a split key walk, against the float64 restatement (bf16 operands: tolerance of their rounding)"""
    rng = np.random.default_rng(R + window + H)
    n = 330
    rows = rng.normal(0, 0.3, (n, R)).astype(np.float32)
    qdir = rng.normal(0, 1, R).astype(np.float32)
    qdir /= np.linalg.norm(qdir)
    spikes = [0, 31, 32, 63, 64, 130, 255]
    for j in spikes:
        rows[j] = 3.0 * qdir + rng.normal(0, 0.05, R)
    rows = torch.from_numpy(rows).to(torch.bfloat16).float().numpy()
    st, tab, slot = filled_cache(rows, torch.bfloat16)
    assert so.latent_attn_mc_supported(tab)
    sink = bf(rng.normal(0, 1, H))
    w = window or n
    for start, count in ((0, 70), (60, 150), (200, 130), (129, 1), (n - 1, 1), (0, 1), (spikes[3] + w - 1, 2)):
        if start + count > n:
            continue
        pos = list(range(start, start + count))
        q = (rng.normal(0, 0.2, (count, H * R)) + np.tile(4.0 * qdir, H)).astype(np.float32)
        qr = torch.from_numpy(q).to(torch.bfloat16).float().numpy()
        want = attn_ref(qr, rows, pos, H, window, 0.5, sink.float().numpy())
        i32 = lambda a: torch.tensor(a, dtype=torch.int32).cuda()
        got = so.latent_window_attn_mc(dev(q), tab, sink.cuda(), i32(pos), i32([slot.index]), i32([0]), i32([count]), count, pos[-1], H, window,
                                       0.5, nsplit=nsplit)
        assert rel_err(got.cpu().numpy(), want) < 6e-3, (start, count)     # P is rounded to bf16 for the second product
        exact = so.latent_window_attn(dev(qr), tab, sink.cuda(), torch.full((count,), slot.index, dtype=torch.int32).cuda(), i32(pos), H, window, 0.5)
        assert rel_err(got.cpu().numpy(), exact.cpu().numpy()) < 6e-3
        if window:
            shifted = attn_ref(qr, rows, pos, H, window + 1, 0.5, sink.float().numpy())
            if rel_err(shifted, want) > 0.05:
                assert rel_err(got.cpu().numpy(), shifted) > 0.03


def test_gated_recurrence_in_chunks_side_by_side(so):
    """long portions cut into chunks that run in parallel: two portions of unequal length (one shorter than a chunk) that start
    from states an earlier step left"""
    rng = np.random.default_rng(12)
    C, na, nb, pre = 70, 333, 40, 9
    mk = lambda n: (rng.normal(0, 1, (n, C)).astype(np.float32), rng.normal(0, 1, (n, C)).astype(np.float32),
                    rng.uniform(0, 1, (n, C)).astype(np.float32), rng.uniform(0, 1, (n, C)).astype(np.float32))
    lam = bf(rng.normal(-2, 2, C))
    seqs = [mk(pre + na), mk(pre + nb)]
    want = [om.gated_recurrence(u.astype(np.float64), r, i, lam.double().numpy(), 8.0) * y for u, y, r, i in seqs]
    state = torch.zeros(3, C, device="cuda")
    cat = lambda k, lo, hi: dev(np.concatenate([seqs[0][k][lo[0]:hi[0]], seqs[1][k][lo[1]:hi[1]]]))
    ts, to, es, er, ec = entries([(2, pre), (0, pre)], 3)
    so.gated_recurrence(cat(2, (0, 0), (pre, pre)), cat(3, (0, 0), (pre, pre)), cat(0, (0, 0), (pre, pre)), cat(1, (0, 0), (pre, pre)), lam.cuda(),
                        8.0, state, es, er, ec)
    ts, to, es, er, ec = entries([(2, na), (0, nb)], 3)
    lo, hi = (pre, pre), (pre + na, pre + nb)
    got = so.gated_recurrence(cat(2, lo, hi), cat(3, lo, hi), cat(0, lo, hi), cat(1, lo, hi), lam.cuda(), 8.0, state, es, er, ec, max_count=na)
    seq_state = state.clone()
    assert rel_err(got[:na].cpu().numpy(), want[0][pre:]) < 5e-6 and rel_err(got[na:].cpu().numpy(), want[1][pre:]) < 5e-6
    # the states it leaves are those of the row-by-row form
    state2 = torch.zeros(3, C, device="cuda")
    for (s, n), k in (((2, pre + na), 0), ((0, pre + nb), 1)):
        ts, to, es, er, ec = entries([(s, n)], 3)
        so.gated_recurrence(dev(seqs[k][2]), dev(seqs[k][3]), dev(seqs[k][0]), dev(seqs[k][1]), lam.cuda(), 8.0, state2, es, er, ec)
    assert rel_err(seq_state.cpu().numpy(), state2.cpu().numpy()) < 5e-6 and float(seq_state[1].abs().max()) == 0


@pytest.mark.parametrize("T", [1, 3, 4, 9, 40])
def test_linear_f32_stream_mode(so, T):
    """f32 products of the unrounded rows whichever kernel serves the row count (block-diagonal weights with bias and sigmoid)"""
    rng = np.random.default_rng(T)
    G, N, K = 6, 40, 40
    x = rng.normal(0, 1, (T, 3 * K)).astype(np.float32)
    w, b = bf(rng.normal(0, 0.2, (G, N, K))), bf(rng.normal(0, 0.3, (G, N)))
    y = so.linear(dev(x), w.cuda(), b.cuda(), act="sigmoid", groups=G, x_groups=3, math=so.MATH_F32_STREAM)
    want = np.concatenate([om.sigmoid(x[:, (g % 3) * K:(g % 3 + 1) * K].astype(np.float64) @ w[g].double().numpy().T + b[g].double().numpy())
                           for g in range(G)], 1)
    assert rel_err(y.cpu().numpy(), want) < 2e-6
