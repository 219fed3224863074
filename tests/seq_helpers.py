"""Helpers of the sequence-engine tests: engines from random small models, cache filling."""
import numpy as np
import torch

from tests.conftest import load_pkg


def to_torch(tensors, device="cuda"):
    return {k: torch.from_numpy(np.ascontiguousarray(v)).to(torch.bfloat16).to(device) for k, v in tensors.items()}


def make_engine(cfg, tensors, dtype=torch.float32, max_tokens=1024, max_slots=4, device="cuda"):
    load_pkg()
    from dash_infer_amd import models
    from dash_infer_amd.engine import SeqEngine
    return SeqEngine(models.resolve(cfg), cfg, to_torch(tensors, device), dtype=dtype, max_tokens=max_tokens, max_slots=max_slots, device=device)


def rel_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / (np.abs(want).max() + 1e-30))


def rows_close(got, want, tol, share=0.95):
    """for engines that round to 16 bits: a rounding can tip a routing decision that the exact computation makes narrowly, and
    that row (and, weakly, later ones) then differs by more than rounding.  True when `share` of the rows are within tol of the
    reference, relative to its largest value."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    err = np.abs(got - want).max(axis=1) / (np.abs(want).max() + 1e-30)
    return float(np.mean(err < tol)) >= share


def run_whole(eng, rid, tokens):
    out = eng.step([(rid, tokens, list(range(len(tokens))))]).cpu().numpy()
    eng.release(rid)
    return out


def run_portions(eng, rid, tokens, sizes, release=True):
    """the prompt in portions of the given sizes (the last size repeats), all logits"""
    out, at, k = [], 0, 0
    while at < len(tokens):
        n = min(sizes[min(k, len(sizes) - 1)], len(tokens) - at)
        out.append(eng.step([(rid, tokens[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
        k += 1
    if release:
        eng.release(rid)
    return np.concatenate(out)


class MixerRig:
    """One mixer (or feed-forward) of dash_infer_amd.mixers on a state manager of its own: feeds rows of hidden states as
    portions of named sequences, as the engine's step does, and returns the mixer's output rows."""

    def __init__(self, build, dtype=torch.float32, max_tokens=2048, slots=4, eps=1e-5):
        load_pkg()
        from dash_infer_amd import seq_ops
        from dash_infer_amd.seq_state import SequenceStateManager
        self.so, self.dtype, self.eps = seq_ops, dtype, eps
        self.state = SequenceStateManager(max_tokens, slots, 64, "cuda")
        self.mixer = build(self.state, dtype)
        self.state.upload()

    def step(self, portions):
        """portions: [(sequence name, rows [n, width] numpy)] -> [output rows numpy]"""
        from dash_infer_amd.mixers import StepContext
        st = self.state
        tslot, tpos, toff, eslot, erow0, ecnt, hs = [], [], [], [], [], [], []
        for name, rows in portions:
            if name not in st.live:
                st.admit(name)
            n = rows.shape[0]
            s = st.reserve(name, st.live[name].length + n)
            erow0.append(len(tslot))
            tslot += [s.index] * n
            tpos += range(s.length, s.length + n)
            toff += range(n)
            eslot.append(s.index)
            ecnt.append(n)
            s.length += n
            hs.append(rows)
        st.upload()
        i32 = lambda a: torch.tensor(a, dtype=torch.int32, device="cuda")
        T = len(tslot)
        math = self.so.MATH_BF16 if self.dtype == torch.bfloat16 else self.so.MATH_F32
        ctx = StepContext(T, len(eslot), i32([0] * T), i32([0] * T), i32(tslot), i32(tpos), i32(toff), i32(eslot), i32(erow0), i32(ecnt),
                          i32([]), math, self.eps)
        ctx.max_count, ctx.max_pos = max(ecnt), max(tpos)
        self.ctx = ctx
        h = torch.from_numpy(np.concatenate(hs).astype(np.float32)).cuda()
        out = self.mixer(ctx, h, h.to(torch.bfloat16) if self.dtype == torch.bfloat16 else None).cpu().numpy()
        return [out[r:r + n] for r, n in zip(erow0, ecnt)]

    def release(self, name):
        self.state.release(name)


def dev_weights(w, device="cuda"):
    """name -> numpy array (bf16 values)  ->  name -> bf16 device tensor"""
    return {k: torch.from_numpy(np.ascontiguousarray(v, dtype=np.float32)).to(torch.bfloat16).to(device) for k, v in w.items()}
