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
