"""The serving loop over a paged cache: admission, page and slot bookkeeping, batching of unequal requests, sampling.

`Engine.step(entries)` is the one step function: every entry is (request id, its next tokens, places whose logits are wanted);
all entries of a step are one batch -- portions of prompts beside single decoded tokens -- flattened into rows that carry their
sequence slot and position, so a position's logits do not depend on how its request was cut into steps or on what else ran
beside it.  `Generator` drives the same step for generation: prompts are fed in portions while other requests decode,
tokens are chosen by the library's device sampler."""
from __future__ import annotations

import random

import torch

from .cache import PAGE_SIZE, PagePool
from .layered import SPAN_CHUNK, StepBatch

PROMPT_TILE = 64                                          # rows per tile of a prompt portion (csrc/window_attn.hip: 16 query rows per wave)


class Engine:
    def __init__(self, model, max_tokens: int, max_seqs: int = 4, page_size: int = PAGE_SIZE, graphs: bool | None = None):
        """The pool is made for `max_tokens` live tokens over at most `max_seqs` live requests, each holding whole pages.
        graphs (default: on a GPU): steps that bring one token per request -- decoding -- replay ONE HIP graph per batch size; their
        inputs (tokens, slots, positions, block table) live in device buffers the graph reads."""
        self.model = model
        pages = -(-int(max_tokens) // page_size) + max_seqs
        self.pool = PagePool(pages, page_size, max_seqs, model.device)
        self.cache = model.make_cache(self.pool)
        self.slots = {}                                           # request id -> slot
        self.graphs = ((model.device.type == "cuda") if graphs is None else bool(graphs)) and getattr(model, "graph_safe_step", False)
        self._decode = {}                                         # batch size -> captured decode step
        self._stream = torch.cuda.Stream(device=model.device) if self.graphs and model.device.type == "cuda" else None

    def live(self):
        return list(self.slots)

    def length(self, rid) -> int:
        return self.pool.seq_len[self.slots[rid]]

    def step(self, entries, end=()):
        """entries: iterable of (request id, tokens, want) -- `want` = indices into `tokens` whose logits are returned, in the order
        of the entries and of `want`.  A request is admitted at its first entry.  `end`: requests whose pages and slot are given
        back after the step.  Returns fp32 logits [n wanted, vocab] on the device, or None."""
        ids, seq, pos, want_rows = [], [], [], []
        t16_row0, t16_rows, t1_row0, t1_maxpos = [], [], [], 0
        prompt_spans = []
        spans = []
        seen = set()
        for rid, tokens, want in entries:
            if rid in seen:
                raise RuntimeError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            n = len(tokens)
            if n == 0:
                continue
            if rid not in self.slots:
                self.slots[rid] = self.pool.open()
            slot = self.slots[rid]
            start = self.pool.extend(slot, n)
            base = len(ids)
            spans.append((base, n, slot, start))
            if n > 1:
                prompt_spans.append((base, n))
            if n == 1:
                t1_row0.append(base)
                t1_maxpos = max(t1_maxpos, start)
            else:
                for i in range(0, n, 16):
                    t16_row0.append(base + i)
                    t16_rows.append(min(16, n - i))
            ids.extend(int(t) for t in tokens)
            seq.extend([slot] * n)
            pos.extend(range(start, start + n))
            for w in want:
                if not 0 <= w < n:
                    raise RuntimeError(f"request {rid!r}: wanted place {w} outside its {n} tokens")
                want_rows.append(base + w)
        logits = None
        if ids and self.graphs and not t16_row0 and len(want_rows) == len(ids):
            logits = self._decode_step(ids, seq, pos)
        elif ids:
            dev = self.model.device
            packed = torch.tensor([ids, seq, pos], dtype=torch.int32).to(dev)
            lr = torch.tensor(want_rows or [0], dtype=torch.int32).to(dev)
            batch = StepBatch(packed[0], packed[1], packed[2], self.pool.device_table(), lr, len(ids), len(want_rows), spans=spans,
                              logits_all_rows=want_rows == list(range(len(ids))))
            chunk0, total = [], 0
            for s in spans:                                       # recurrent mixers unroll long spans in chunks of SPAN_CHUNK rows
                chunk0.append(total)
                total += -(-s[1] // SPAN_CHUNK)
            sp = torch.tensor([[s[0] for s in spans], [s[1] for s in spans], chunk0], dtype=torch.int32).to(dev)
            batch.spans_dev = (sp[0], sp[1], len(spans), max(s[1] for s in spans))
            batch.span_chunks = (sp[2], SPAN_CHUNK, total)
            if prompt_spans:
                # tiles of consecutive positions for the tiled attention kernels
                size = PROMPT_TILE
                row0 = [b + i for b, n in prompt_spans for i in range(0, n, size)]
                nrow = [min(size, n - i) for b, n in prompt_spans for i in range(0, n, size)]
                tl = torch.tensor([row0, nrow], dtype=torch.int32).to(dev)
                batch.prompt_tiles = (tl[0], tl[1], len(row0), size)
            if t16_row0:
                t16 = torch.tensor([t16_row0, t16_rows], dtype=torch.int32).to(dev)
                batch.tiles16 = (t16[0], t16[1], len(t16_row0))
            if t1_row0:
                batch.tiles1 = (torch.tensor(t1_row0, dtype=torch.int32).to(dev), len(t1_row0), t1_maxpos)
            logits = self.model.step(batch, self.cache)
            if logits is not None:
                logits = logits.clone()                          # the step's own buffer is reused by the next step
        for rid in end:
            self.finish(rid)
        return logits

    def _decode_step(self, ids, seq, pos):
        """One token per request, every row's logits wanted: the step's launches are the same for every such step of this batch
        size (the split of the attention keys is fixed by the pool's capacity), so they are captured once -- after a first eager
        run that sizes the scratch arena -- and replayed with new inputs."""
        m, ext, b = self.model, self.model.ext, len(ids)
        st = self._decode.get(b)
        if st is None:
            dev = m.device
            ar = torch.arange(b, dtype=torch.int32, device=dev)
            st = {"inputs": torch.zeros((3, b), dtype=torch.int32, device=dev), "rows": ar, "graph": None, "runs": 0}
            cap = self.pool.num_pages * self.pool.page_size
            st["batch"] = StepBatch(st["inputs"][0], st["inputs"][1], st["inputs"][2], self.pool.device_table(), ar, b, b,
                                    tiles1=(ar, b, cap - 1), spans_dev=(ar, torch.ones_like(ar), b, 1), logits_all_rows=True)
            self._decode[b] = st
        if st["graph"] is not None and st.get("epoch") != getattr(m, "scratch_epoch", 0):
            # a larger step has moved a scratch buffer since the capture: the graph holds the old addresses
            ext.graph_free(st["graph"])
            st["graph"], st["runs"] = None, 1
        host = torch.tensor([ids, seq, pos], dtype=torch.int32)
        if self._stream is None:                                   # (no GPU: the same batch, eagerly)
            st["inputs"].copy_(host)
            self.pool.device_table()
            return m.step(st["batch"], self.cache).clone()
        cur = torch.cuda.current_stream(m.device)
        self._stream.wait_stream(cur)
        with torch.cuda.stream(self._stream):
            st["inputs"].copy_(host)
            self.pool.device_table()
            if st["graph"] is None:
                logits = m.step(st["batch"], self.cache)          # eager: valid result, and every scratch buffer gets its size
                st["runs"] += 1
                if st["runs"] >= 2:                                # a batch size seen twice is worth a graph
                    self._stream.synchronize()
                    m.frozen = True
                    ext.graph_begin_capture(self._stream.cuda_stream)
                    try:
                        st["logits"] = m.step(st["batch"], self.cache)    # recorded, not run
                    finally:
                        st["graph"] = ext.graph_end_capture(self._stream.cuda_stream)
                        st["epoch"] = getattr(m, "scratch_epoch", 0)
                        m.frozen = False
            else:
                ext.graph_launch(st["graph"], self._stream.cuda_stream)
                logits = st["logits"]
            out = logits.clone()
        cur.wait_stream(self._stream)
        return out

    def close(self) -> None:
        for st in self._decode.values():
            if st.get("graph") is not None:
                self.model.ext.graph_free(st["graph"])
                st["graph"] = None

    def finish(self, rid) -> None:
        slot = self.slots.pop(rid, None)
        if slot is not None:
            self.pool.close(slot)


class Generator:
    """Continuous batching over Engine.step: up to the pool's slot count of requests are live; a request's prompt is fed in
    portions of at most `chunk` tokens beside the single tokens of requests that already decode; the next token of a row comes
    from the library's device sampler (csrc/sampling.hip; temperature 0 = greedy)."""

    def __init__(self, engine: Engine, chunk: int = 512):
        self.engine, self.chunk = engine, chunk

    def generate(self, prompts, max_new_tokens: int, temperature: float = 0.0, top_k: int = 1, top_p: float = 0.0,
                 min_p: float = 0.0, seed: int = 0, stop_token: int | None = None):
        """prompts: list of token-id lists; returns the list of generated token lists (greedy by default)"""
        eng, ext = self.engine, self.engine.model.ext
        rng = random.Random(seed)
        waiting = list(range(len(prompts)))[::-1]
        state = {}                                               # request -> [tokens not yet fed, generated]
        out = [[] for _ in prompts]
        dev, vocab = eng.model.device, eng.model.vocab
        while waiting or state:
            while waiting and len(state) < eng.pool.max_seqs:
                r = waiting.pop()
                if not prompts[r]:
                    raise RuntimeError("generate: empty prompt")
                state[r] = [list(prompts[r]), 0]
            entries, sampled = [], []
            for r, (todo, _n) in state.items():
                part = todo[:self.chunk]
                del todo[:len(part)]
                last = not todo
                entries.append((r, part, [len(part) - 1] if last else []))
                if last:
                    sampled.append(r)
            logits = eng.step(entries)
            if not sampled:
                continue
            toks = torch.empty((len(sampled),), dtype=torch.int32, device=dev)
            probs = torch.empty((len(sampled),), dtype=torch.float32, device=dev)
            ext.sample_rows(logits, temperature, top_k, top_p, min_p, rng.random(), toks, probs, vocab=vocab)
            for r, t in zip(sampled, toks.cpu().tolist()):
                out[r].append(int(t))
                state[r][1] += 1
                if state[r][1] >= max_new_tokens or (stop_token is not None and t == stop_token):
                    eng.finish(r)
                    del state[r]
                else:
                    state[r][0] = [int(t)]
        return out
