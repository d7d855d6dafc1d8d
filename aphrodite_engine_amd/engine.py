"""A small serving engine around any registered model: page pool, state slots, continuous-batching scheduler with
chunked prompts, the step function, and sampling (the roles of BlockSpaceManager, Scheduler, ModelRunner.execute_model
and Sampler, aphrodite/processing/scheduler.py + task_handler/model_runner.py + modeling/layers/sampler.py, cut down to
one process and one GPU).

A step is a list of SEGMENTS -- (request, next tokens) -- run as one batch: portions of prompts beside single decoded
tokens.  ``LLMEngine.step()`` lets the scheduler choose the segments; ``LLMEngine.run_segments()`` runs segments the caller
dictates (replaying a recorded schedule) through the very same page / slot bookkeeping and ``ModelRunner.execute``.

Pages hold ``block_size`` tokens of every paged cache of the model at once (one block table per request, shared by all
layer runs); a state slot holds every recurrent state of one request.  Both are handed back when a request ends and are
reused LIFO, so a new request usually lands in memory another one has just left: a model must not read what it has not
written -- the kernels start a sequence's state from zero when its context is empty, and attention never reads past a
sequence's own length."""
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

import torch

from .step_batch import StepBatch


class NoFreePages(RuntimeError):
    pass


class FreeList:
    """LIFO pool of integer handles (pages or state slots)."""

    def __init__(self, n: int, what: str):
        self.what, self.total = what, n
        self._free = list(range(n - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, n: int = 1) -> List[int]:
        if n > len(self._free):
            raise NoFreePages(f"{n} {self.what} wanted, {len(self._free)} of {self.total} free")
        out = [self._free.pop() for _ in range(n)]
        return out

    def give(self, handles: Sequence[int]) -> None:
        for h in handles:
            if not 0 <= h < self.total or h in self._free:
                raise ValueError(f"{self.what} {h} given back twice or never taken")
            self._free.append(h)


@dataclass
class SamplingParams:
    max_tokens: int = 16
    temperature: float = 0.0          # 0: greedy
    top_k: int = -1
    top_p: float = 1.0
    seed: Optional[int] = None
    stop_token_ids: Tuple[int, ...] = ()


@dataclass
class Request:
    request_id: str
    tokens: List[int]                 # prompt, then generated tokens
    num_prompt: int
    params: SamplingParams = field(default_factory=SamplingParams)
    num_computed: int = 0             # tokens whose keys / state are in the caches
    pages: List[int] = field(default_factory=list)
    slot: int = -1
    finished: bool = False

    @property
    def output_tokens(self) -> List[int]:
        return self.tokens[self.num_prompt:]


class ModelRunner:
    """Owns the caches and turns segments into one model step."""

    def __init__(self, model, num_pages: int, block_size: int, num_slots: int, device):
        self.model, self.block_size, self.device = model, block_size, torch.device(device)
        self.caches = model.make_caches(num_pages, block_size, num_slots, self.device)

    @torch.no_grad()
    def execute(self, segments: Sequence[Tuple[Request, Sequence[int]]], want: Sequence[Sequence[int]]) -> torch.Tensor:
        """Run the segments as one batch from the caches earlier steps left; returns fp32 logits [sum(len(w)), vocab] for
        the wanted places (indices into each segment's tokens), in segment order."""
        batch = StepBatch.build([list(t) for _, t in segments], [r.num_computed for r, _ in segments],
                                [r.pages for r, _ in segments], [r.slot for r, _ in segments], self.block_size, self.device)
        rows, a = [], 0
        for (_, toks), w in zip(segments, want):
            for i in w:
                if not 0 <= i < len(toks):
                    raise ValueError("a wanted place outside its segment")
                rows.append(a + i)
            a += len(toks)
        if not rows:                  # the step still has to advance caches and states
            rows = [0]
            logits = self.model.step(batch, self.caches, torch.tensor(rows, dtype=torch.int64, device=self.device))
            return logits[:0]
        return self.model.step(batch, self.caches, torch.tensor(rows, dtype=torch.int64, device=self.device))


class Scheduler:
    """Continuous batching with chunked prompts: every running request that is past its prompt gets its one token, then
    prompt portions fill what is left of the token budget, oldest request first."""

    def __init__(self, max_num_seqs: int, max_num_batched_tokens: int):
        self.max_num_seqs, self.max_tokens = max_num_seqs, max_num_batched_tokens
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []

    def add(self, r: Request) -> None:
        self.waiting.append(r)

    def plan(self, can_admit, pages_for) -> List[Tuple[Request, int]]:
        """[(request, number of its next tokens)], prompt portions first, decoded tokens last.  ``can_admit()`` says
        whether a state slot is free; ``pages_for(request, n)`` reserves pages for n more tokens or returns False."""
        budget = self.max_tokens
        decodes, portions = [], []
        for r in self.running:
            left = len(r.tokens) - r.num_computed
            if left == 1 and r.num_computed >= r.num_prompt and budget > 0 and pages_for(r, 1):
                decodes.append((r, 1))
                budget -= 1
        for r in self.running:
            left = len(r.tokens) - r.num_computed
            if not (left == 1 and r.num_computed >= r.num_prompt) and left > 0 and budget > 0:
                n = min(left, budget)
                if pages_for(r, n):
                    portions.append((r, n))
                    budget -= n
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs and can_admit():
            r = self.waiting[0]
            n = min(len(r.tokens), budget)
            if not pages_for(r, n):
                break
            self.waiting.popleft()
            self.running.append(r)
            portions.append((r, n))
            budget -= n
        return portions + decodes

    def retire(self, r: Request) -> None:
        self.running.remove(r)


class Sampler:
    """Greedy and temperature / top-k / top-p sampling on the package's own kernels."""

    def __call__(self, logits: torch.Tensor, params: Sequence[SamplingParams], steps: Sequence[int]) -> List[int]:
        from . import _custom_ops as ops
        if all(p.temperature <= 0.0 for p in params):
            return ops.argmax_rows(logits).tolist()
        dev = logits.device
        temp = torch.tensor([p.temperature if p.temperature > 0 else 1.0 for p in params], dtype=torch.float32, device=dev)
        top_k = torch.tensor([p.top_k if p.top_k > 0 else logits.shape[1] for p in params], dtype=torch.int32, device=dev)
        top_p = torch.tensor([p.top_p for p in params], dtype=torch.float32, device=dev)
        seeds = torch.tensor([(p.seed if p.seed is not None else 0) * 1000003 + s for p, s in zip(params, steps)],
                             dtype=torch.int64, device=dev)
        drawn = ops.sample_top_k_top_p(logits, temp, top_k, top_p, seeds=seeds).tolist()
        greedy = ops.argmax_rows(logits).tolist()
        return [g if p.temperature <= 0.0 else d for p, d, g in zip(params, drawn, greedy)]


class LLMEngine:
    def __init__(self, model, max_tokens: int = 8192, max_num_seqs: int = 4, block_size: int = 16,
                 max_num_batched_tokens: int = 2048, device="cuda"):
        """``max_tokens``: the most tokens live requests hold at any time (each request's count rounded up to whole
        pages): the page pool is made for exactly that."""
        self.block_size = block_size
        self.pages = FreeList((max_tokens + block_size - 1) // block_size, "pages")
        self.slots = FreeList(max_num_seqs, "state slots")
        self.runner = ModelRunner(model, self.pages.total, block_size, max_num_seqs, device)
        self.scheduler = Scheduler(max_num_seqs, max_num_batched_tokens)
        self.sampler = Sampler()
        self.requests: Dict[str, Request] = {}

    @classmethod
    def from_pretrained(cls, model_dir: str, dtype: torch.dtype = torch.bfloat16, device="cuda", **engine_args) -> "LLMEngine":
        from .loader import load_model
        return cls(load_model(model_dir, dtype=dtype, device=device), device=device, **engine_args)

    # ---- bookkeeping shared by both ways of stepping -------------------------------------------------------------------
    def _admit(self, r: Request) -> None:
        if r.slot < 0:
            r.slot = self.slots.take()[0]

    def _reserve(self, r: Request, n: int) -> bool:
        need = (r.num_computed + n + self.block_size - 1) // self.block_size - len(r.pages)
        if need > self.pages.num_free:
            return False
        if need > 0:
            r.pages += self.pages.take(need)
        return True

    def release(self, request_id: str) -> None:
        """Give a request's pages and slot back."""
        r = self.requests.pop(request_id)
        self.pages.give(r.pages)
        if r.slot >= 0:
            self.slots.give([r.slot])
        r.pages, r.slot, r.finished = [], -1, True

    def _run(self, segments: List[Tuple[Request, List[int]]], want: Sequence[Sequence[int]]) -> torch.Tensor:
        logits = self.runner.execute(segments, want)
        for r, toks in segments:
            r.num_computed += len(toks)
        return logits

    # ---- a dictated schedule -------------------------------------------------------------------------------------------
    def run_segments(self, entries: Sequence[Tuple[str, Sequence[int], Sequence[int]]]) -> torch.Tensor:
        """entries: (request id, its next tokens, wanted places among them).  A request is admitted at its first entry
        and keeps its pages and slot until ``release``.  Returns fp32 logits of the wanted places, in order."""
        segments, want = [], []
        for rid, toks, w in entries:
            if len(toks) == 0:
                if len(w):
                    raise ValueError(f"request {rid}: logits wanted of an entry without tokens")
                continue
            r = self.requests.get(rid)
            if r is None:
                r = Request(rid, [], 0)
                self._admit(r)                 # raises before the request is known if no slot is free
                self.requests[rid] = r
            toks = [int(t) for t in toks]
            if not self._reserve(r, len(toks)):
                raise NoFreePages(f"request {rid}: no pages left for {len(toks)} more tokens")
            r.tokens += toks
            r.num_prompt = len(r.tokens)
            segments.append((r, toks))
            want.append(list(w))
        if not segments:
            return torch.empty(0, self.runner.model.vocab_size, dtype=torch.float32, device=self.runner.device)
        # prompt portions first, decoded tokens last (the order attention metadata assumes); answers keep the caller's order
        order = sorted(range(len(segments)), key=lambda i: len(segments[i][1]) == 1 and segments[i][0].num_computed > 0)
        logits = self._run([segments[i] for i in order], [want[i] for i in order])
        if order == list(range(len(order))):
            return logits
        offs, a = {}, 0
        for i in order:
            offs[i] = a
            a += len(want[i])
        idx = [offs[i] + j for i in range(len(segments)) for j in range(len(want[i]))]
        return logits[torch.tensor(idx, dtype=torch.int64, device=logits.device)] if idx else logits[:0]

    # ---- generation ----------------------------------------------------------------------------------------------------
    def add_request(self, request_id: str, prompt_token_ids: Sequence[int], params: Optional[SamplingParams] = None) -> None:
        if request_id in self.requests:
            raise ValueError(f"request {request_id} exists")
        if not prompt_token_ids:
            raise ValueError("empty prompt")
        r = Request(request_id, [int(t) for t in prompt_token_ids], len(prompt_token_ids), params or SamplingParams())
        self.requests[request_id] = r
        self.scheduler.add(r)

    def has_unfinished(self) -> bool:
        return bool(self.scheduler.waiting or self.scheduler.running)

    def step(self) -> List[Request]:
        """One scheduler-chosen batch; returns the requests that finished in it."""
        def pages_for(r, n):
            if not self._reserve(r, n):
                return False
            self._admit(r)
            return True
        plan = self.scheduler.plan(lambda: self.slots.num_free > 0, pages_for)
        if not plan:
            if self.has_unfinished():
                raise NoFreePages("nothing can be scheduled: the page pool is too small for the oldest request")
            return []
        segments = [(r, r.tokens[r.num_computed:r.num_computed + n]) for r, n in plan]
        # a segment that reaches the end of what the request holds yields the next token
        samples = [i for i, (r, toks) in enumerate(segments) if r.num_computed + len(toks) == len(r.tokens)]
        want = [[len(toks) - 1] if i in samples else [] for i, (_, toks) in enumerate(segments)]
        logits = self._run(segments, want)
        done = []
        if samples:
            rs = [segments[i][0] for i in samples]
            new = self.sampler(logits, [r.params for r in rs], [len(r.tokens) for r in rs])
            for r, tok in zip(rs, new):
                r.tokens.append(int(tok))
                if len(r.output_tokens) >= r.params.max_tokens or int(tok) in r.params.stop_token_ids:
                    done.append(r)
        for r in done:
            self.scheduler.retire(r)
            self.release(r.request_id)
        return done

    def generate(self, prompts: Sequence[Sequence[int]], params: Optional[SamplingParams] = None) -> List[List[int]]:
        """Token ids in, generated token ids out, one list per prompt."""
        reqs = []
        for i, p in enumerate(prompts):
            rid = f"gen-{len(self.requests)}-{i}"
            self.add_request(rid, p, params)
            reqs.append(self.requests[rid])
        while self.has_unfinished():
            self.step()
        return [r.output_tokens for r in reqs]
