"""Teacher-forced replay: feed given token ids through the engine step by step and read
logits instead of sampling.

A replay step names, per request, its next tokens and the rows whose logits are wanted.
It runs through the same pieces as generation: the block manager hands out KV pages and
the sequence's slot (block-table row and recurrent-state slot), ``ModelRunner.build_plan``
packs the step (several tokens of a request: a prefill chunk; one token of a request that
already has context: a decode row, so decode-only steps replay the captured graphs), and
``ModelRunner.run_logits`` executes it.  Nothing is sampled, so a request's "prompt"
simply grows by the tokens of each step.  Used by ``bin/trace_run`` and by scoring.
"""
from __future__ import annotations

from typing import Optional

import torch

from .llm_engine import LLMEngine
from .sequence import SamplingParams, Sequence


class ReplayError(RuntimeError):
    pass


class TraceReplayer:
    def __init__(self, engine: LLMEngine):
        if engine.pp_depth > 1:
            raise ValueError("replay drives a single-stage engine")
        self.engine = engine
        self.bm = engine.bm
        self.runner = engine.executor.runner
        self.seqs: dict[str, Sequence] = {}
        self._params = SamplingParams(temperature=0.0, max_tokens=None)

    @property
    def live(self) -> int:
        return len(self.seqs)

    def step(self, entries: list[dict], end: Optional[list] = None) -> Optional[torch.Tensor]:
        """entries: [{"id", "tokens": [...], "want": [indices into tokens]}].  Returns fp32
        logits [wanted rows, vocab] in the order of the entries and their ``want`` (None
        when nothing is wanted), after freeing the requests named in ``end``."""
        cfg = self.engine.cfg
        prefills, decodes, order = [], [], []
        total = 0
        for e in entries:
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                continue
            seq = self.seqs.get(e["id"])
            if seq is None:
                if len(self.seqs) >= cfg.max_num_seqs:
                    raise ReplayError(f"more than {cfg.max_num_seqs} live requests")
                seq = self.seqs[e["id"]] = Sequence(str(e["id"]), [], self._params,
                                                    max_model_len=self.engine.max_model_len)
            n = len(toks)
            total += n
            if seq.num_tokens + n > self.engine.max_model_len:
                raise ReplayError(f"request {e['id']} exceeds max_model_len")
            if max(toks) >= self.engine.mcfg.vocab_size or min(toks) < 0:
                raise ReplayError("token id out of vocabulary range")
            seq.prompt_token_ids.extend(toks)
            if not self.bm.can_allocate(seq, seq.num_computed + n):
                raise ReplayError("KV pool exhausted")
            self.bm.allocate(seq, seq.num_computed + n)
            decode = n == 1 and seq.num_computed > 0
            (decodes if decode else prefills).append((seq, n))
            order.append((seq, n, decode, [int(w) for w in e.get("want", [])]))
        if total > cfg.token_budget():
            raise ReplayError(f"step of {total} tokens exceeds the token budget")
        logits = None
        if order:
            # rows of the packed step: prefill chunks first (in entry order), then decodes
            first, off = {}, 0
            for seq, n in prefills:
                first[seq.seq_id] = off
                off += n
            for seq, _ in decodes:
                first[seq.seq_id] = off
                off += 1
            rows = [first[seq.seq_id] + w for seq, n, _, want in order for w in want]
            plan, _ = self.runner.build_plan(prefills, [s for s, _ in decodes], self.bm.table)
            if rows:
                logits = self.engine.executor.execute_logits(plan, rows)
            else:
                self.engine.executor.execute(plan)
            for seq, n, _, _ in order:
                seq.num_computed += n
        for rid in end or []:
            seq = self.seqs.pop(rid, None)
            if seq is not None:
                self.bm.free_seq(seq)
        if self.engine._debug:
            self.bm.check_invariants(list(self.seqs.values()))
        return logits
