"""Serving engine for models that run ragged steps (hybrid.HybridModel): cache manager + step builder + continuous-batching scheduler.

  * ``run_step(entries)`` is the step function: every entry brings the next tokens of one sequence (a portion of a prompt or one decoded
    token); all entries run as ONE batch against the pages and state slots the sequences hold, and the logits of the asked rows come back.
    A sequence is admitted at its first entry, may sit out steps, and gives its pages and slot back on ``release``.
  * ``add_request`` / ``step`` / ``generate`` schedule requests over it: decode tokens of running requests first, then prompt portions of
    admitted and waiting requests up to a token budget per step; a request is admitted when a state slot is free and the pool can hold its
    prompt and everything it may generate.  New tokens come from the framework's sampler (sampler.sample_greedy: greedy, or temperature /
    top-k / top-p with explicit uniforms).
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .kvcache import CacheManager
from .mixers import StepBatch


@dataclass
class Request:
    rid: object
    prompt: List[int]
    max_new_tokens: int
    top_k: int = 1
    top_p: float = 1.0
    temperature: float = 1.0
    eos_id: Optional[int] = None
    seed: int = 0
    fed: int = 0                                   # prompt tokens already run
    output: List[int] = field(default_factory=list)
    done: bool = False


class ServingEngine:
    def __init__(self, model, *, max_tokens: int, max_seqs: int = 4, max_step_tokens: int = 2048):
        """max_tokens: tokens the page pool holds (every live sequence rounded up to whole pages); max_seqs: state slots = live sequences."""
        self.model, self.page = model, model.page
        self.device = model.device
        num_pages = max(1, (max_tokens + self.page - 1) // self.page)
        self.cache = CacheManager(num_pages, self.page, max_seqs)
        self.tensors = model.alloc_cache(num_pages, max_seqs)
        self.max_step_tokens = max_step_tokens
        # decode-only steps (one token per entry, its logits wanted) replay a captured HIP graph per (sequences, block-table width)
        self.use_graphs = False
        self._graphs = {}
        self.waiting: List[Request] = []
        self.running: List[Request] = []

    # ------------------------------------------------------------------ the step function
    def build_batch(self, entries: Sequence[Tuple[object, Sequence[int], Sequence[int]]]) -> StepBatch:
        """entries: (sequence id, its next tokens, indices among them whose logits are wanted).  Admits new sequences and takes pages."""
        tokens, pos, seq, row_start, slot, first, want, tables, prev = [], [], [], [0], [], [], [], [], []
        seen, admitted = set(), []
        try:
            return self._build(entries, tokens, pos, seq, row_start, slot, first, want, tables, seen, admitted, prev)
        except Exception:
            for sid in admitted:                      # a step that cannot run leaves no half-admitted sequence behind
                self.cache.release(sid)
            raise

    def _build(self, entries, tokens, pos, seq, row_start, slot, first, want, tables, seen, admitted, prev):
        for sid, toks, wants in entries:
            if sid in seen:
                raise ValueError(f"sequence {sid!r} appears twice in one step")
            seen.add(sid)
            if not len(toks):
                raise ValueError(f"sequence {sid!r}: an entry without tokens")
            if sid not in self.cache.live:
                self.cache.admit(sid)
                admitted.append(sid)
            sc = self.cache.grow(sid, len(toks))
            s = len(slot)
            base = len(tokens)
            tokens += [int(t) for t in toks]
            prev += [sc.last_token if sc.length else -1] + [int(t) for t in toks[:-1]]
            pos += list(range(sc.length, sc.length + len(toks)))
            seq += [s] * len(toks)
            row_start.append(len(tokens))
            slot.append(sc.slot)
            first.append(sc.length)
            for w in wants:
                if not 0 <= int(w) < len(toks):
                    raise ValueError(f"sequence {sid!r}: wanted row {w} of {len(toks)}")
                want.append(base + int(w))
            tables.append(sc.pages)
        width = max(8, -(-max(len(t) for t in tables) // 8) * 8)
        t0, tn = [], []
        for a, b in zip(row_start[:-1], row_start[1:]):           # tiles of at most 16 consecutive rows of one sequence
            t0 += list(range(a, b, 16))
            tn += [min(16, b - r) for r in range(a, b, 16)]
        bt = []
        for t in tables:
            bt += t + [0] * (width - len(t))
        # every index array of the step travels in ONE pinned int32 buffer and one copy; the fields are views into the device copy
        parts = [tokens, pos, seq, row_start, slot, first, bt, want, t0, tn, prev]
        offs = [0]
        for part in parts:
            offs.append(offs[-1] + (len(part) + 3) // 4 * 4)      # 16-byte aligned fields
        host = torch.zeros(offs[-1], dtype=torch.int32, pin_memory=self.device.type == "cuda")
        for o, part in zip(offs, parts):
            if part:
                host[o:o + len(part)] = torch.tensor(part, dtype=torch.int32)
        batch = self.batch_views(host.to(self.device, non_blocking=True), [len(part) for part in parts], len(tables), width)
        batch.host = host
        batch.max_rows = max(b - a for a, b in zip(row_start[:-1], row_start[1:]))
        return batch

    @staticmethod
    def batch_views(buf: torch.Tensor, sizes, nseq: int, width: int) -> StepBatch:
        """The StepBatch whose fields are views of `buf` (layout of _build: fields in StepBatch order, each padded to 4 elements)."""
        views, o = [], 0
        for n in sizes:
            views.append(buf[o:o + n])
            o += (n + 3) // 4 * 4
        views[6] = views[6].view(nseq, width)
        return StepBatch(*views)

    def run_step(self, entries, collect: Optional[list] = None) -> Optional[torch.Tensor]:
        """Run the entries as one batch; -> fp32 logits [wanted rows, vocab] in the order of the entries and their wants (None if none)."""
        entries = [(sid, list(toks), list(wants)) for sid, toks, wants in entries]
        if not entries:
            return None
        batch = self.build_batch(entries)
        if self.use_graphs and collect is None and all(len(t) == 1 and list(w) == [0] for _, t, w in entries):
            logits = self._replay_decode(batch)
        else:
            logits = self.model.forward(batch, self.tensors, collect)
        for sid, toks, _ in entries:
            self.cache.advance(sid, len(toks), toks[-1])
        return logits if batch.want.numel() else None

    def _replay_decode(self, batch: StepBatch) -> torch.Tensor:
        """The decode step as a graph: captured once per shape over static input tensors (capture runs nothing, so the recurrent states
        move only on replay), then fed by copies into those tensors."""
        key = (batch.slot.numel(), batch.block_table.shape[1])
        ent = self._graphs.get(key)
        if ent is None:
            buf = torch.empty_like(batch.host, device=self.device)
            buf.copy_(batch.host)
            nseq, width = key
            static = self.batch_views(buf, [nseq, nseq, nseq, nseq + 1, nseq, nseq, nseq * width, nseq, nseq, nseq, nseq], nseq, width)
            static.max_rows = 1
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                out = self.model.forward(static, self.tensors)
            ent = self._graphs[key] = (g, buf, out)
        g, buf, out = ent
        buf.copy_(batch.host, non_blocking=True)              # one copy feeds every index array of the captured step
        g.replay()
        return out.clone()

    def release(self, sid):
        self.cache.release(sid)

    # ------------------------------------------------------------------ scheduling
    def add_request(self, prompt: Sequence[int], max_new_tokens: int, *, rid=None, top_k: int = 1, top_p: float = 1.0, temperature: float = 1.0,
                    eos_id: Optional[int] = None, seed: int = 0) -> Request:
        if not len(prompt) or max_new_tokens < 1:
            raise ValueError("add_request: an empty prompt or nothing to generate")
        total = len(prompt) + max_new_tokens
        if self.cache.pages_for(total) > self.cache.pages.num_pages:
            raise ValueError(f"add_request: {total} tokens do not fit the pool of {self.cache.pages.num_pages} pages of {self.page}")
        r = Request(rid if rid is not None else object(), [int(t) for t in prompt], int(max_new_tokens), int(top_k), float(top_p), float(temperature),
                    eos_id, int(seed))
        self.waiting.append(r)
        return r

    def _admit_waiting(self):
        while self.waiting:
            r = self.waiting[0]
            if not self.cache.can_admit(len(r.prompt) + r.max_new_tokens):
                break
            self.cache.admit(r.rid, reserve_tokens=len(r.prompt) + r.max_new_tokens)
            self.running.append(self.waiting.pop(0))

    def step(self) -> List[Tuple[Request, int]]:
        """One scheduled step: -> the (request, new token) pairs it produced."""
        from . import sampler
        self._admit_waiting()
        budget = self.max_step_tokens
        entries, owners = [], []
        for r in self.running:                                    # decode rows first: one token each
            if r.fed == len(r.prompt) and budget > 0:
                entries.append((r.rid, [r.output[-1]], [0])); owners.append(r); budget -= 1
        for r in self.running:                                    # then portions of prompts, first come first served
            if r.fed < len(r.prompt) and budget > 0:
                n = min(budget, len(r.prompt) - r.fed)
                last = r.fed + n == len(r.prompt)
                entries.append((r.rid, r.prompt[r.fed:r.fed + n], [n - 1] if last else []))
                if last:
                    owners.append(r)
                budget -= n
        if not entries:
            return []
        logits = self.run_step(entries)
        by_id = {r.rid: r for r in self.running}
        for sid, toks, _ in entries:
            r = by_id[sid]
            if r.fed < len(r.prompt):
                r.fed += len(toks)
        produced = []
        if owners:
            B = len(owners)
            step_col = max(len(r.prompt) + len(r.output) for r in owners)
            hist = torch.zeros(B, step_col + 1, dtype=torch.int32)
            lens = torch.zeros(B, dtype=torch.int32)
            for i, r in enumerate(owners):
                t = r.prompt + r.output
                hist[i, : len(t)] = torch.tensor(t, dtype=torch.int32)
                lens[i] = len(t)
            u = torch.tensor([torch.rand(1, generator=torch.Generator().manual_seed(r.seed * 1000003 + len(r.output))).item() for r in owners])
            params = sampler.GreedyParams(logits=logits.contiguous(), input_lengths=lens, sequence_lengths=lens, token_ids=hist, step=step_col,
                                          top_k=torch.tensor([r.top_k for r in owners], dtype=torch.int32),
                                          top_p=torch.tensor([r.top_p for r in owners], dtype=torch.float32),
                                          temperature=torch.tensor([r.temperature for r in owners], dtype=torch.float32), uniform=u)
            ids = sampler.sample_greedy(params).cpu().tolist()
            for r, t in zip(owners, ids):
                r.output.append(int(t))
                produced.append((r, int(t)))
                if len(r.output) >= r.max_new_tokens or (r.eos_id is not None and t == r.eos_id):
                    r.done = True
        for r in [x for x in self.running if x.done]:
            self.running.remove(r)
            self.release(r.rid)
        return produced

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, **sampling) -> List[List[int]]:
        """Generate for every prompt (more prompts than state slots queue up and join as slots and pages free up)."""
        reqs = [self.add_request(p, max_new_tokens, rid=("gen", i, id(prompts)), **sampling) for i, p in enumerate(prompts)]
        while any(not r.done for r in reqs):
            if not self.step() and not self.running and self.waiting:
                raise MemoryError("generate: a waiting request can never be admitted")
        return [r.output for r in reqs]
