"""Generation engine with continuous batching over ragged steps: requests wait in a queue, are admitted when a state slot
and enough cache blocks are free, feed their prompts in portions next to the decode tokens of the requests that are further
along, are sampled with the framework's sampler (sampling.py) and give slot and blocks back when they finish.

The engine owns no forward pass and no cache: every iteration is ONE call of :meth:`RaggedRunner.step` (executor/ragged.py),
the same step function the trace replay drives.  It serves the layered model family (model_layers.py); the llama-shaped
models keep their own drivers (executor: ``DecodeEngine`` for one-shot batches, ``SlotRunner`` / ``SlotBatch`` for slots).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

import torch

from .executor.ragged import RaggedRunner
from .sampling import Sampler


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0       # 0: greedy
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    eos_token_id: int | None = None


@dataclass
class _Request:
    rid: int
    prompt: list[int]
    params: SamplingParams
    slot: int | None = None
    fed: int = 0                                   # prompt tokens already in the cache
    generated: list[int] = field(default_factory=list)

    @property
    def in_prefill(self) -> bool:
        return self.fed < len(self.prompt)


@dataclass
class _Span:
    token_ids: torch.Tensor
    mask: torch.Tensor


class GenerationEngine:
    def __init__(self, model, max_tokens: int, max_requests: int = 4, block_size: int = 64, max_step_tokens: int = 512,
                 device="cuda", seed: int = 0, capture_decode: bool = False):
        """``max_tokens``: size of the cache pool (tokens over all live requests, block-rounded per request);
        ``max_step_tokens``: the most tokens one step carries -- decode tokens first, the rest goes to prompt portions;
        ``capture_decode``: steps that carry decode tokens only are replayed from a hipGraph per (running set, context
        partitions) cell (``RaggedRunner._decode_step_captured``)."""
        self.runner = RaggedRunner(model, max_tokens, max_requests, block_size, device, capture_decode=capture_decode)
        self.max_step_tokens = max(1, int(max_step_tokens))
        self.device = torch.device(device)
        self._waiting: deque[_Request] = deque()
        self._running: list[_Request] = []
        self._reserved: dict[int, int] = {}        # rid -> blocks its prompt + generation may need
        self._next_id = 0
        self._sampler = Sampler()
        self._rng = torch.Generator(device=self.device)
        self._rng.manual_seed(seed)
        self.steps = 0

    # ------------------------------------------------------------------ queue ------- #
    def add_request(self, prompt_ids, params: SamplingParams | None = None) -> int:
        params = params or SamplingParams()
        prompt = [int(t) for t in prompt_ids]
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        need = self.runner.blocks_for(len(prompt) + params.max_new_tokens)
        if need > self.runner.total_blocks or len(prompt) + params.max_new_tokens > self.runner.max_seq_len:
            raise ValueError(f"a request of {len(prompt)} + {params.max_new_tokens} tokens does not fit the cache pool")
        req = _Request(self._next_id, prompt, params)
        self._next_id += 1
        self._waiting.append(req)
        return req.rid

    def _admit(self) -> None:
        while self._waiting and self.runner.free_slots:
            req = self._waiting[0]
            need = self.runner.blocks_for(len(req.prompt) + req.params.max_new_tokens)
            if sum(self._reserved.values()) + need > self.runner.total_blocks:
                break  # first come, first served: nobody overtakes the head of the queue
            self._waiting.popleft()
            req.slot = self.runner.admit()
            self._reserved[req.rid] = need
            self._running.append(req)

    @property
    def idle(self) -> bool:
        return not self._waiting and not self._running

    # ------------------------------------------------------------------ one iteration #
    def step(self) -> list[tuple[int, list[int]]]:
        """Admit, run one ragged step, sample, retire.  Returns the requests that finished: ``(id, generated tokens)``."""
        self._admit()
        if not self._running:
            return []
        budget = self.max_step_tokens
        entries, riders = [], []
        for req in self._running:                   # decode tokens first: one each
            if not req.in_prefill and budget > 0:
                entries.append((req.slot, [req.generated[-1]]))
                riders.append(req)
                budget -= 1
        for req in self._running:                   # then prompt portions, in admission order
            if req.in_prefill and budget > 0:
                take = min(budget, len(req.prompt) - req.fed)
                entries.append((req.slot, req.prompt[req.fed:req.fed + take]))
                riders.append(req)
                req.fed += take
                budget -= take
        rows, samplers, at = [], [], 0
        for req, (_, toks) in zip(riders, entries):
            at += len(toks)
            if not req.in_prefill:                  # its last token's logits decide the next token
                rows.append(at - 1)
                samplers.append(req)
        logits = self.runner.step(entries, rows)
        self.steps += 1
        finished = []
        if samplers:
            for req, tok in zip(samplers, self._sample(logits, samplers)):
                req.generated.append(tok)
                p = req.params
                if len(req.generated) >= p.max_new_tokens or (p.eos_token_id is not None and tok == p.eos_token_id):
                    finished.append(req)
        for req in finished:
            self.runner.release([req.slot])
            self._running.remove(req)
            del self._reserved[req.rid]
        return [(r.rid, r.generated) for r in finished]

    def _sample(self, logits: torch.Tensor, reqs: list[_Request]) -> list[int]:
        """Rows with equal parameters go through the sampler together (greedy rows: one argmax launch)."""
        out = [0] * len(reqs)
        groups: dict[tuple, list[int]] = {}
        for i, r in enumerate(reqs):
            p = r.params
            groups.setdefault((p.temperature, p.top_p, p.repetition_penalty), []).append(i)
        for (temperature, _, penalty), idx in groups.items():
            rows = logits if len(idx) == len(reqs) else logits[torch.tensor(idx, device=logits.device)]
            span = None
            if penalty != 1.0:
                width = max(1, max(len(reqs[i].generated) for i in idx))
                ids = torch.zeros(len(idx), width, dtype=torch.long)
                mask = torch.zeros(len(idx), width, dtype=torch.bool)
                for j, i in enumerate(idx):
                    g = reqs[i].generated
                    ids[j, :len(g)] = torch.tensor(g, dtype=torch.long)
                    mask[j, :len(g)] = True
                span = _Span(ids.to(logits.device), mask.to(logits.device))
            uniform = torch.rand(len(idx), device=logits.device, generator=self._rng) if temperature != 0.0 else None
            toks = self._sampler.sample(rows.contiguous(), reqs[idx[0]].params, span, uniform=uniform).view(-1).tolist()
            for i, t in zip(idx, toks):
                out[i] = int(t)
        return out

    # ------------------------------------------------------------------ drivers ----- #
    def run(self) -> dict[int, list[int]]:
        done: dict[int, list[int]] = {}
        while not self.idle:
            for rid, toks in self.step():
                done[rid] = toks
        self.runner.check_errors()
        return done

    def generate(self, prompts, params: SamplingParams | None = None) -> list[list[int]]:
        """Generated tokens per prompt, in the order given."""
        ids = [self.add_request(p, params) for p in prompts]
        done = self.run()
        return [done[i] for i in ids]
