"""Serving loop above the executors: paged-cache block manager, sequence state, step function, scheduler, sampling.

The executors of the library take a step's tokens with explicit cache slots and block tables and leave their bookkeeping to the
caller; this file is that caller.  `Engine.step` runs one batch (prompts, prompt portions or decode tokens of any mix of
sequences) through the model and returns the logits rows that were asked for; `Engine.generate` drives it from a scheduler
(first come, first served: waiting prompts are admitted while blocks and the step's token budget last, running sequences decode
together) and samples with the library's sampling kernels.  Nothing here computes on tensors: arrays of ids go in, logits or
token ids come out.
"""
from __future__ import annotations

import collections
import dataclasses

import numpy as np
import torch

from ._lib import check, lib


class BlockManager:
    """Free list of cache blocks.  Freed blocks are handed out again first, last freed first, so reuse (in another order than
    the first owner's) is the common case, not the corner."""

    def __init__(self, num_blocks: int, block_size: int):
        self.num_blocks, self.block_size = num_blocks, block_size
        self.free = list(range(num_blocks - 1, -1, -1))

    def blocks_for(self, tokens: int) -> int:
        return (tokens + self.block_size - 1) // self.block_size

    def can_allocate(self, n: int) -> bool:
        return n <= len(self.free)

    def allocate(self, n: int) -> list:
        if n > len(self.free):
            raise MemoryError(f"cache exhausted: {n} blocks wanted, {len(self.free)} free of {self.num_blocks}")
        return [self.free.pop() for _ in range(n)]

    def release(self, blocks: list) -> None:
        self.free.extend(blocks)


class StateSlots:
    """Free list of recurrent-state slots: a model with recurrent layers keeps each live sequence's state (convolution inputs,
    matrix memories) in one slot of fixed size.  A slot is not cleared when it changes hands: the executor starts a sequence whose
    step begins at position 0 from zeros.  Like the blocks, freed slots are handed out again first."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free = list(range(num_slots - 1, -1, -1))

    def allocate(self) -> int:
        if not self.free:
            raise MemoryError(f"all {self.num_slots} state slots are in use")
        return self.free.pop()

    def release(self, slot: int) -> None:
        self.free.append(slot)


@dataclasses.dataclass
class Sequence:
    """What a request holds between steps: its cache blocks, how many tokens they hold, its last token (the hashed bigram
    embedding of the next token needs it) and, for models with recurrent layers, its state slot."""
    seq_id: object
    blocks: list = dataclasses.field(default_factory=list)
    length: int = 0
    last_token: int = -1
    state_slot: int = -1


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 0.0      # 0: greedy
    top_k: int = 0
    top_p: float = 1.0
    max_new_tokens: int = 16
    seed: int = 0


class Engine:
    def __init__(self, model, max_tokens: int | None = None):
        """model: an executor driver with .forward(tokens, prev, positions, slots, seq_ids, block_tables, logit_rows, ...),
        .block_size, .num_blocks, .max_tokens, .vocab_size (GesutarForCausalLM, GupuvikForCausalLM; PackedQwen3 adapts the Qwen3
        executor).  A driver with .state_slots > 0 also gets seq_starts and state_slots (recurrent state per sequence)."""
        self.model = model
        self.blocks = BlockManager(model.num_blocks, model.block_size)
        self.states = StateSlots(model.state_slots) if getattr(model, "state_slots", 0) else None
        self.max_tokens = min(max_tokens or model.max_tokens, model.max_tokens)
        self.seqs: dict = {}
        self.device = model.device

    # ------------------------------------------------------------------ state
    def add(self, seq_id) -> Sequence:
        if seq_id in self.seqs:
            raise KeyError(f"sequence {seq_id!r} already exists")
        s = Sequence(seq_id)
        if self.states is not None:
            s.state_slot = self.states.allocate()
        self.seqs[seq_id] = s
        return s

    def finish(self, seq_id) -> None:
        s = self.seqs.pop(seq_id)
        self.blocks.release(s.blocks)
        s.blocks = []
        if self.states is not None and s.state_slot >= 0:
            self.states.release(s.state_slot)
            s.state_slot = -1

    def _dev(self, a) -> torch.Tensor:
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(self.device)

    # ------------------------------------------------------------------ one step
    def step(self, entries, want_logits: bool = True, want_greedy: bool = False, layer_trace: bool = False):
        """entries: [(seq_id, token ids, wanted offsets among these tokens)], unknown seq_ids start new sequences.
        All entries are one batch.  Returns (logits f32 [wanted, vocab] | None, greedy ids [wanted] | None, trace | None) with
        rows in the order of the entries and of their wanted offsets."""
        bs = self.blocks.block_size
        total = sum(len(t) for _, t, _ in entries)
        if total == 0:
            return None, None, None
        if total > self.max_tokens:
            raise ValueError(f"step of {total} tokens, the engine takes {self.max_tokens}")
        tok = np.empty(total, np.int32)
        prev = np.empty(total, np.int32)
        pos = np.empty(total, np.int32)
        slots = np.empty(total, np.int32)
        sid = np.empty(total, np.int32)
        rows = []
        at = 0
        seqs = []
        for i, (seq_id, tokens, want) in enumerate(entries):
            s = self.seqs.get(seq_id) or self.add(seq_id)
            n = len(tokens)
            need = self.blocks.blocks_for(s.length + n) - len(s.blocks)
            if need > 0:
                s.blocks.extend(self.blocks.allocate(need))
            seqs.append(s)
            t = np.asarray(tokens, np.int32)
            p = np.arange(s.length, s.length + n, dtype=np.int32)
            tok[at:at + n] = t
            prev[at] = s.last_token
            prev[at + 1:at + n] = t[:-1]
            pos[at:at + n] = p
            b = np.asarray(s.blocks, np.int32)
            slots[at:at + n] = b[p // bs] * bs + p % bs
            sid[at:at + n] = i
            rows.extend(at + int(w) for w in want)
            at += n
        width = max(len(s.blocks) for s in seqs)
        bt = np.zeros((len(seqs), width), np.int32)
        for i, s in enumerate(seqs):
            bt[i, :len(s.blocks)] = s.blocks
        extra = {}
        if self.states is not None:   # recurrent layers walk each sequence's rows in order and carry its state slot
            starts = np.zeros(len(seqs) + 1, np.int32)
            starts[1:] = np.cumsum([len(t) for _, t, _ in entries])
            extra = {"seq_starts": self._dev(starts), "state_slots": self._dev([s.state_slot for s in seqs])}
        out = self.model.forward(self._dev(tok), self._dev(prev), self._dev(pos), self._dev(slots), self._dev(sid), self._dev(bt),
                                 self._dev(rows) if rows else None, want_logits=want_logits, want_greedy=want_greedy, layer_trace=layer_trace,
                                 **extra)
        for s, (_, tokens, _) in zip(seqs, entries):
            s.length += len(tokens)
            s.last_token = int(tokens[-1])
        return out

    # ------------------------------------------------------------------ sampling
    def sample(self, logits: torch.Tensor, params: list, rng: np.random.Generator) -> np.ndarray:
        """Token ids for f32 logits rows [n, vocab] under per-row SamplingParams (temperature > 0; greedy rows are the caller's)."""
        n, V = logits.shape
        st = torch.cuda.current_stream().cuda_stream
        inv_t = torch.tensor([1.0 / max(p.temperature, 1e-6) for p in params], dtype=torch.float32, device=self.device)
        lg = logits.clone()
        check(lib.vmx_temperature_scale_f32_per_seq(lg.data_ptr(), inv_t.data_ptr(), n, V, st))
        probs = torch.empty_like(lg)
        check(lib.vmx_softmax_to_probs(probs.data_ptr(), lg.data_ptr(), 0, n, V, st))
        rv = torch.from_numpy(rng.random(n, dtype=np.float32)).to(self.device)
        tk = torch.tensor([p.top_k for p in params], dtype=torch.int32, device=self.device)
        tp = torch.tensor([p.top_p for p in params], dtype=torch.float32, device=self.device)
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        check(lib.vmx_top_k_top_p_sample(out.data_ptr(), probs.data_ptr(), rv.data_ptr(), tk.data_ptr(), tp.data_ptr(), 0, 1.0, n, V, st))
        return out.cpu().numpy()

    # ------------------------------------------------------------------ generation
    def generate(self, prompts: list, params: SamplingParams | list | None = None, prefill_chunk: int | None = None) -> list:
        """Continuous batching over `prompts` (lists of token ids); returns the generated ids per prompt.  prefill_chunk: longest
        prompt portion a sequence contributes to one step (None: whole prompts)."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        sched = Scheduler(self, prefill_chunk)
        for i, (p, sp) in enumerate(zip(prompts, params)):
            sched.submit(("gen", i), list(p), sp)
        rng = np.random.default_rng(params[0].seed if params else 0)
        while sched.busy():
            batch = sched.schedule()
            entries = [(r.seq_id, r.next_tokens, [len(r.next_tokens) - 1] if r.samples_now else []) for r in batch]
            need = [r for r in batch if r.samples_now]
            greedy = all(r.params.temperature <= 0 for r in need)
            logits, ids, _ = self.step(entries, want_logits=not greedy, want_greedy=greedy)
            if need:
                chosen = ids.cpu().numpy() if greedy else None
                if not greedy:
                    chosen = self.sample(logits, [r.params for r in need], rng)
                    for j, r in enumerate(need):
                        if r.params.temperature <= 0:
                            chosen[j] = int(torch.argmax(logits[j]).item())
            sched.update(batch, {id(r): int(chosen[j]) for j, r in enumerate(need)} if need else {})
        return [sched.done[("gen", i)] for i in range(len(prompts))]


@dataclasses.dataclass
class Request:
    seq_id: object
    prompt: list
    params: SamplingParams
    fed: int = 0                 # prompt tokens already in the cache
    output: list = dataclasses.field(default_factory=list)
    next_tokens: list = dataclasses.field(default_factory=list)
    samples_now: bool = False


class Scheduler:
    """First come, first served.  A step is either a prefill step (waiting or partly fed prompts, as many as the token budget and
    the free blocks allow) or a decode step of every running sequence; prompts go first so that new requests join the decode batch
    early.  A request that cannot get blocks waits until running ones finish."""

    def __init__(self, engine: Engine, prefill_chunk: int | None = None):
        self.engine, self.prefill_chunk = engine, prefill_chunk
        self.waiting: collections.deque = collections.deque()
        self.running: list = []
        self.done: dict = {}

    def submit(self, seq_id, prompt: list, params: SamplingParams) -> None:
        if not prompt:
            raise ValueError("empty prompt")
        self.waiting.append(Request(seq_id, prompt, params))

    def busy(self) -> bool:
        return bool(self.waiting or self.running)

    def schedule(self) -> list:
        eng = self.engine
        budget, batch = eng.max_tokens, []
        free = len(eng.blocks.free)
        # prompt portions: requests already admitted but not fully fed come first, then new ones in arrival order
        feeding = [r for r in self.running if r.fed < len(r.prompt)]
        while self.waiting and len(self.running) + 1 <= eng.model.max_seqs:
            r = self.waiting[0]
            # admission: the whole prompt plus its generation must fit into what is free once the running ones have grown
            need = eng.blocks.blocks_for(len(r.prompt) + r.params.max_new_tokens)
            reserved = sum(eng.blocks.blocks_for(len(q.prompt) + q.params.max_new_tokens) - len(eng.seqs[q.seq_id].blocks) if q.seq_id in eng.seqs
                           else eng.blocks.blocks_for(len(q.prompt) + q.params.max_new_tokens) for q in self.running)
            if need + reserved > free:
                break
            self.waiting.popleft()
            self.running.append(r)
            feeding.append(r)
        for r in feeding:
            if budget <= 0:
                break
            n = len(r.prompt) - r.fed
            if self.prefill_chunk:
                n = min(n, self.prefill_chunk)
            n = min(n, budget)
            r.next_tokens = r.prompt[r.fed:r.fed + n]
            r.samples_now = r.fed + n == len(r.prompt)
            budget -= n
            batch.append(r)
        if batch:
            return batch
        if not self.running:
            raise MemoryError("no request fits into the cache")
        for r in self.running[:budget]:
            r.next_tokens = [r.output[-1]]
            r.samples_now = True
            batch.append(r)
        return batch

    def update(self, batch: list, chosen: dict) -> None:
        for r in batch:
            if r.fed < len(r.prompt):
                r.fed += len(r.next_tokens)
            if id(r) in chosen:
                r.output.append(chosen[id(r)])
                if len(r.output) >= r.params.max_new_tokens:
                    self.done[r.seq_id] = r.output
                    self.running.remove(r)
                    self.engine.finish(r.seq_id)


class PackedQwen3:
    """The Qwen3-family executor behind the packed step interface of Engine: prompt portions go through its native prompt
    pass one sequence at a time, single tokens of several sequences through its batched decode step."""

    def __init__(self, model):
        self.model, s = model, model.spec
        self.block_size, self.num_blocks, self.vocab_size, self.device = s.block_size, s.num_blocks, s.vocab_size, model.device
        self.max_tokens = max(s.max_prefill_tokens, s.max_batch)
        self.max_seqs = s.max_batch

    def forward(self, tokens, prev_tokens, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits=True, want_greedy=False,
                layer_trace=False):
        m, s = self.model, self.model.spec
        sid = seq_ids.cpu().numpy()
        pos = positions.cpu().numpy()
        rows = [] if logit_rows is None else logit_rows.cpu().numpy().tolist()
        T = len(sid)
        logits = torch.zeros((T, s.vocab_size), dtype=m.act_torch_dtype, device=self.device)
        ids = torch.zeros(T, dtype=torch.int32, device=self.device)
        starts = [i for i in range(T) if i == 0 or sid[i] != sid[i - 1]] + [T]
        single = all(starts[i + 1] - starts[i] == 1 for i in range(len(starts) - 1))
        if single and T <= s.max_batch:
            bt = block_tables[torch.from_numpy(sid).long().to(self.device)].contiguous()
            m.forward_decode_batch(tokens, positions, slots, bt, (positions + 1).contiguous(), out_ids=ids, logits=logits)
        else:
            for a, b in zip(starts[:-1], starts[1:]):
                # the native prompt pass returns the last row only: portions that want other rows go token by token
                inner = [r for r in rows if a <= r < b - 1]
                if inner or b - a > s.max_prefill_tokens:
                    i2, l2 = m.forward(tokens[a:b], int(pos[a]), block_tables[sid[a]])
                    ids[a:b], logits[a:b] = i2, l2
                else:
                    m.prefill(tokens[a:b], int(pos[a]), block_tables[sid[a]], out_id=ids[b - 1:b], logits_last=logits[b - 1])
        sel = torch.tensor(rows, dtype=torch.long, device=self.device)
        return (logits[sel].float() if want_logits and rows else None), (ids[sel] if want_greedy and rows else None), None
