"""The sequence engine: ragged-batch step function, scheduler and generation loop for the models of models/ whose
`engine` is "sequence".

    eng = SeqEngine.from_pretrained(folder, dtype=torch.bfloat16, max_tokens=4096, max_slots=4)
    logits = eng.step([("a", [5, 17, 3], [0, 2]), ("b", [9], [0])])       # portions of prompts beside decoded tokens
    eng.release("a")
    outs = eng.generate([[1, 2, 3], [4, 5]], max_new_tokens=16)             # scheduler + sampling on top of step()

One step runs the tokens it is given, all requests as ONE flat batch, from what earlier steps left in the state manager
(seq_state.SequenceStateManager): the logits of a position do not depend on how its prompt was cut, on the other requests
of the batch or on the pages and slots it got.
"""
from collections import deque

import torch

from . import models, safetensors_io, seq_ops
from .mixers import StepContext
from .seq_state import SequenceStateManager


class SeqEngine:
    def __init__(self, model_cls, config, tensors, dtype=torch.bfloat16, max_tokens=4096, max_slots=4, span_len=64, device="cuda"):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("the sequence engine computes in bfloat16 or float32")
        self.device, self.dtype = device, dtype
        self.state = SequenceStateManager(max_tokens, max_slots, span_len, device)
        self.model = model_cls.from_config(config, tensors, self.state, dtype)
        self.vocab = self.model.vocab
        self.state.upload()
        # decode steps (one token of every request, every one's logits wanted) replay a captured hipGraph per (requests, length
        # bucket): the launches of a step are fixed once its sizes are, its numbers (tokens, positions, slots) lie in a device
        # buffer that is refilled before the replay.  DIHIP_SEQ_GRAPH=0: eager launches.
        import os
        self.use_graphs = dtype == torch.bfloat16 and os.environ.get("DIHIP_SEQ_GRAPH", "1") != "0"
        self._graphs = {}

    @classmethod
    def from_pretrained(cls, path, dtype=torch.bfloat16, device="cuda", **kw):
        import os
        config = models.read_config(path)
        model_cls = models.resolve(config)
        if getattr(model_cls, "engine", None) != "sequence":
            raise ValueError(f"{models.architecture_of(config)} is not served by the sequence engine")
        tensors = safetensors_io.load(os.path.join(path, "model.safetensors"), device)
        return cls(model_cls, config, tensors, dtype=dtype, device=device, **kw)

    # -- one step ---------------------------------------------------------------------------------------------------------
    def step(self, entries, taps=None):
        """entries: (request id, tokens, wanted indices among these tokens) per request, a request at most once.  A request is
        admitted at its first entry.  -> f32 [wanted, vocab] on the device in the order of the entries (None: nothing wanted)."""
        st, model = self.state, self.model
        ids, rows2, tslot, tpos, toff, eslot, erow0, ecnt, want = [], [], [], [], [], [], [], [], []
        seen = set()
        for rid, tokens, wanted in entries:
            if rid in seen:
                raise ValueError(f"request {rid!r} twice in one step")
            seen.add(rid)
            tokens = [int(t) for t in tokens]
            if not tokens:
                continue
            if min(tokens) < 0 or max(tokens) >= self.vocab:
                raise ValueError(f"request {rid!r}: token outside the vocabulary")
            if rid not in st.live:
                st.admit(rid)
            s = st.reserve(rid, st.live[rid].length + len(tokens))
            r2 = model.second_rows(s.last_token, tokens)
            row0 = len(ids)
            ids += tokens
            if r2 is not None:
                rows2 += r2
            tslot += [s.index] * len(tokens)
            tpos += range(s.length, s.length + len(tokens))
            toff += range(len(tokens))
            eslot.append(s.index)
            erow0.append(row0)
            ecnt.append(len(tokens))
            for k in wanted:
                if not 0 <= k < len(tokens):
                    raise ValueError(f"request {rid!r}: wanted index {k} outside its {len(tokens)} tokens")
                want.append(row0 + k)
            s.length += len(tokens)
            s.last_token = tokens[-1]
        T, E = len(ids), len(eslot)
        if T == 0:
            return None
        st.upload()
        if not rows2:
            rows2 = [0] * T
        flat = ids + rows2 + tslot + tpos + toff + eslot + erow0 + ecnt + want
        host = torch.tensor(flat, dtype=torch.int32)
        cut = [T, T, T, T, T, E, E, E, len(want)]
        if self.use_graphs and taps is None and T == E and want == list(range(E)):
            return self._decode_step(host, cut, T, max(tpos))
        if torch.cuda.is_available():
            host = host.pin_memory()
        # the split of the attention's key walk follows the length bucket, as in the captured decode steps: the same step gives the
        # same bits whether it is launched or replayed
        ctx = self._context(host.to(self.device, non_blocking=True), cut, T, E, max(ecnt), self._bucket(max(tpos)))
        ctx.taps = taps
        x = model.forward(ctx)
        if not want:
            return None
        return model.logits(ctx, x, ctx.want_rows)

    def _context(self, dev, cut, T, E, max_count, max_pos):
        parts, o = [], 0
        for n in cut:
            parts.append(dev[o:o + n])
            o += n
        ctx = StepContext(T, E, *parts, math=self.model.math, eps=self.model.eps)
        ctx.max_count, ctx.max_pos = max_count, max_pos
        return ctx

    @staticmethod
    def _bucket(max_pos):
        """the last position of the 512-position bucket max_pos lies in: the split of the attention's key walk follows this, not the exact length"""
        return (max_pos + 512) // 512 * 512 - 1

    def _decode_step(self, host, cut, E, max_pos):
        """one token of each of E requests: the first step of a (E, length bucket) runs eagerly and is then captured, later ones
        replay.  The returned logits are the graph's own buffer: valid until the next step."""
        bucket = self._bucket(max_pos)
        g = self._graphs.get((E, bucket))
        if g is None:
            g = {"host": torch.empty(host.numel(), dtype=torch.int32, pin_memory=True),
                 "meta": torch.empty(host.numel(), dtype=torch.int32, device=self.device), "graph": None}
            if len(self._graphs) < 64:
                self._graphs[(E, bucket)] = g
        if "copied" in g:
            g["copied"].synchronize()      # the staging block is free again once the step before has read it
        g["host"].copy_(host)
        g["meta"].copy_(g["host"], non_blocking=True)
        g["copied"] = torch.cuda.Event()
        g["copied"].record()
        if g["graph"] is not None:
            g["graph"].replay()
            return g["logits"]
        ctx = self._context(g["meta"], cut, E, E, 1, bucket)
        logits = self.model.logits(ctx, self.model.forward(ctx), ctx.want_rows)
        if (E, bucket) in self._graphs:
            torch.cuda.synchronize()
            try:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):      # records the same launches; nothing runs, the state is not touched
                    g["logits"] = self.model.logits(ctx, self.model.forward(ctx), ctx.want_rows)
                g["graph"] = graph
            except Exception as e:  # noqa: BLE001  a capture that fails costs speed only: this step has run, later ones launch eagerly
                import sys
                print(f"sequence engine: hipGraph capture failed ({type(e).__name__}: {e}); decode steps launch eagerly", file=sys.stderr)
                self.use_graphs = False
                self._graphs.clear()
                torch.cuda.synchronize()
        return logits

    def release(self, rid):
        if rid in self.state.live:
            self.state.release(rid)

    # -- generation ---------------------------------------------------------------------------------------------------------
    def generate(self, prompts, max_new_tokens=16, sampling=None, eos=None, token_budget=2048, max_chunk=512):
        """Continuous batching over step(): prompts are admitted while slots and pages last, prefilled in portions of at most
        max_chunk tokens under a per-step token budget beside the running requests' decode tokens.  sampling: None (greedy)
        or a dict top_k / top_p / temperature / seed (ops.sample).  -> the generated token ids per prompt."""
        sched = Scheduler(self.state, token_budget, max_chunk)
        reqs = [Request(i, list(p), max_new_tokens) for i, p in enumerate(prompts)]
        for r in reqs:
            if not r.prompt:
                raise ValueError("empty prompt")
            sched.add(r)
        while sched.busy():
            batch = sched.next_batch()
            if not batch:
                raise RuntimeError("the scheduler could not place any request: the cache pool is too small for one of them")
            logits = self.step([(("gen", r.index), toks, [len(toks) - 1] if sample else []) for r, toks, sample in batch])
            sampled = [r for r, _, sample in batch if sample]
            if sampled:
                nxt = self._sample(logits, sampled, sampling)
                for r, t in zip(sampled, nxt):
                    r.out.append(t)
                    if len(r.out) >= r.max_new or (eos is not None and t == eos):
                        r.done = True
            for r, toks, _ in batch:
                r.fed += len(toks)
                if r.done:
                    sched.finish(r)
                    self.release(("gen", r.index))
        return [r.out for r in reqs]

    def _sample(self, logits, reqs, sampling):
        from . import ops   # the sampling kernels live in the decode library
        if not sampling:
            return ops.argmax(logits.contiguous()).tolist()
        M = logits.shape[0]
        pos = torch.tensor([len(r.prompt) + len(r.out) for r in reqs], dtype=torch.int32, device=logits.device)
        seed = [int(sampling.get("seed", 0)) + r.index for r in reqs]
        return ops.sample(logits.contiguous(), [int(sampling.get("top_k", 0))] * M, [float(sampling.get("top_p", 1.0))] * M,
                          [float(sampling.get("temperature", 1.0))] * M, seed, position=pos).tolist()


class Request:
    def __init__(self, index, prompt, max_new):
        self.index, self.prompt, self.max_new = index, prompt, max_new
        self.out, self.fed, self.done = [], 0, False

    def pending(self):
        """tokens not yet run: the rest of the prompt, then the last sampled token"""
        seq = self.prompt + self.out
        return seq[self.fed:]


class Scheduler:
    """Which requests run in the next step, and how many tokens of each.  Running requests come first (one decode token, or the
    next portion of their prompt), then waiting ones are admitted in arrival order while a slot is free and the pool holds the
    pages of their whole prompt and generation (no preemption: an admitted request always finishes)."""

    def __init__(self, state, token_budget=2048, max_chunk=512):
        self.state, self.token_budget, self.max_chunk = state, int(token_budget), int(max_chunk)
        self.waiting, self.running = deque(), []
        self.reserved_pages = 0

    def add(self, r):
        self.waiting.append(r)

    def busy(self):
        return bool(self.waiting or self.running)

    def _pages(self, r):
        return self.state.pages_for(len(r.prompt) + r.max_new)

    def next_batch(self):
        while self.waiting and len(self.running) < self.state.max_slots:
            r = self.waiting[0]
            if self.reserved_pages + self._pages(r) > self.state.num_pages:
                break
            self.reserved_pages += self._pages(r)
            self.running.append(self.waiting.popleft())
        batch, budget = [], self.token_budget
        for r in self.running:
            pend = r.pending()
            n = min(len(pend), self.max_chunk, budget)
            if n <= 0:
                continue
            budget -= n
            batch.append((r, pend[:n], n == len(pend)))   # the last pending token's logits give the next token
        return batch

    def finish(self, r):
        self.running.remove(r)
        self.reserved_pages -= self._pages(r)
