"""Host side of the sequence engine (no GPU): state manager, scheduler, checkpoint reader, model registry."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from tests.conftest import load_pkg

load_pkg()
from dash_infer_amd import models, safetensors_io  # noqa: E402
from dash_infer_amd.engine import Request, Scheduler  # noqa: E402
from dash_infer_amd.seq_state import SequenceStateManager  # noqa: E402


def test_state_manager_hands_pages_and_slots_out_again():
    st = SequenceStateManager(max_tokens=300, max_slots=2, span_len=64, device="cpu")
    assert st.num_pages == 5
    tab = st.add_span_cache("k", 8, torch.float32)
    s = st.add_state("s", (3,))
    a = st.admit("a")
    st.reserve("a", 65)
    assert len(a.pages) == 2 and st.used_pages() == 2
    st.reserve("a", 128)
    assert len(a.pages) == 2
    b = st.admit("b")
    s[b.index] = 5.0
    st.reserve("b", 130)
    assert st.used_pages() == 5 and not st.can_admit()
    with pytest.raises(RuntimeError):
        st.reserve("a", 129)
    with pytest.raises(RuntimeError):
        st.admit("c")
    with pytest.raises(KeyError):
        st.admit("a")
    ptr_b0 = int(tab.host[b.index, 0])
    pages_b = list(b.pages)
    st.release("b")
    assert st.used_pages() == 2 and st.can_admit(64 * 3)
    c = st.admit("c")
    assert c.index == b.index and float(s[c.index].abs().max()) == 0      # the slot's state starts at zero again
    st.reserve("c", 64 * 3)
    assert c.pages == pages_b and int(tab.host[c.index, 0]) == ptr_b0
    assert len({int(x) for x in tab.host[c.index, :3]} | {int(x) for x in tab.host[a.index, :2]}) == 5   # no span twice


class FakeState:
    def __init__(self, pages, slots, span=64):
        self.num_pages, self.max_slots, self.span = pages, slots, span

    def pages_for(self, n):
        return (n + self.span - 1) // self.span


def test_scheduler_budget_chunks_and_admission():
    sch = Scheduler(FakeState(pages=2, slots=2), token_budget=40, max_chunk=32)
    reqs = [Request(0, list(range(50)), 4), Request(1, list(range(10)), 4), Request(2, list(range(100)), 4)]
    for r in reqs:
        sch.add(r)
    b = sch.next_batch()
    assert [(r.index, len(t), s) for r, t, s in b] == [(0, 32, False), (1, 8, False)]      # the budget cuts the second portion
    for r, t, _ in b:
        r.fed += len(t)
    b = sch.next_batch()
    assert [(r.index, len(t), s) for r, t, s in b] == [(0, 18, True), (1, 2, True)]
    for r, t, s in b:
        r.fed += len(t)
        r.out.append(7)
    b = sch.next_batch()
    assert [(r.index, t, s) for r, t, s in b] == [(0, [7], True), (1, [7], True)]         # decoding: the sampled token alone
    assert len(sch.waiting) == 1                                                           # no slot for the third
    sch.finish(reqs[1])
    b = sch.next_batch()
    assert [r.index for r, _, _ in b] == [0]      # a slot is free, but the third request needs two pages and one is left
    sch.finish(reqs[0])
    b = sch.next_batch()
    assert [(r.index, len(t)) for r, t, _ in b] == [(2, 32)]


def write_safetensors(path, tensors):
    head, blobs, at = {}, [], 0
    for k, (dt, arr) in tensors.items():
        raw = arr.tobytes()
        head[k] = {"dtype": dt, "shape": list(arr.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    h = json.dumps(head).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + b"".join(blobs))


def test_safetensors_reader(tmp_path):
    rng = np.random.default_rng(0)
    a = rng.normal(size=(3, 5)).astype(np.float32)
    b16 = (a.view(np.uint32) >> 16).astype(np.uint16)
    tab = np.arange(7, dtype=np.int32)
    p = str(tmp_path / "model.safetensors")
    write_safetensors(p, {"a": ("F32", a), "b": ("BF16", b16), "t": ("I32", tab), "e": ("F32", np.zeros((0, 4), np.float32))})
    got = safetensors_io.load(p)
    assert torch.equal(got["a"], torch.from_numpy(a)) and got["b"].dtype == torch.bfloat16 and got["b"].shape == (3, 5)
    assert torch.equal(got["b"].view(torch.int16), torch.from_numpy(b16.view(np.int16)))
    assert torch.equal(got["t"], torch.from_numpy(tab)) and got["e"].shape == (0, 4)
    assert set(safetensors_io.load(p, names={"t"})) == {"t"}
    with open(p, "r+b") as f:
        f.write(struct.pack("<Q", 1 << 40))
    with pytest.raises(ValueError):
        safetensors_io.load(p)


def test_registry_resolves_by_config():
    assert "Modanex" in models.known() and "Qwen2ForCausalLM" in models.known()
    assert models.resolve({"architecture": "Modanex"}).engine == "sequence"
    q = models.resolve({"architectures": ["Qwen2ForCausalLM"]})
    mc = q.model_config({"hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4, "num_hidden_layers": 28,
                         "intermediate_size": 18944, "vocab_size": 152064, "rms_norm_eps": 1e-6, "rope_theta": 1e6})
    assert (mc.hidden, mc.n_heads, mc.n_kv, mc.head_dim, mc.inter) == (3584, 28, 4, 128, 18944)
    with pytest.raises(KeyError):
        models.resolve({"architecture": "NoSuchModel"})
    with pytest.raises(KeyError):
        models.resolve({})


def test_seq_library_exports_every_header_symbol():
    """libdashinfer_hip_seq.so exports what include/dashinfer_hip_seq.h declares, and the ctypes table covers the header"""
    import ctypes
    import re
    from dash_infer_amd import REPO_ROOT, seq_capi
    assert os.path.exists(seq_capi.SEQ_LIB_PATH), "build with __graft_entry__.build()"
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(REPO_ROOT, "include", "dashinfer_hip_seq.h")).read(), flags=re.S)
    syms = sorted(set(re.findall(r"\b(dihip_[a-z0-9_]+)\s*\(", text)))
    l = ctypes.CDLL(seq_capi.SEQ_LIB_PATH)
    assert len(syms) >= 15 and not [s for s in syms if not hasattr(l, s)]
    assert set(syms) == set(seq_capi._SIGS), set(syms) ^ set(seq_capi._SIGS)
    lib = seq_capi.lib()
    assert b"gfx950" in lib.dihip_seq_version()
    assert lib.dihip_latent_window_attn_mc_supported(512, 64, seq_capi.BF16) == 1
    assert lib.dihip_latent_window_attn_mc_supported(48, 64, seq_capi.BF16) == 0 and lib.dihip_latent_window_attn_mc_supported(64, 64, seq_capi.F32) == 0
    assert lib.dihip_latent_window_attn_mc_workspace_bytes(4, 32, 512, 16) == 16 * 4 * 32 * 516 * 4
    assert lib.dihip_gated_recurrence_chunked_workspace_bytes(2, 130, 100) == 2 * 3 * 2 * 100 * 4
