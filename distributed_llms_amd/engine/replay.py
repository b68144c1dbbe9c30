"""Trace replay: feed GIVEN token ids through the engine step by step and return logits.

A serving trace fixes what a scheduler would otherwise decide -- which requests run in a step and how
many of their next tokens each brings (a prompt portion of any length, or one decoded token) -- so a
recorded schedule can be replayed exactly, e.g. to compare logits between builds or against another
implementation.  Nothing is sampled: every token comes from the trace.

The replayer owns no model code: a step is built by the engine's batch builders
(:func:`~.batch.build_decode_batch` for the one-token rows, :func:`~.batch.build_host_batch` for the
prompt portions, :func:`~.batch.merge_mixed` for both in one batch), gets its K/V blocks and state
slots from the engine's BlockManager and runs through ``engine.runner.execute`` -- the same
``StageRunner`` -> ``stage.forward`` path generation takes.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence as Seq, Tuple

import numpy as np
import torch

from .batch import HostBatch, build_decode_batch, build_host_batch, merge_mixed
from .llm_engine import LLMEngine
from .scheduler import Step
from .sequence import SamplingParams, Sequence, SeqStatus


class TraceReplayer:
    def __init__(self, engine: LLMEngine):
        self.engine = engine
        self.live: Dict[str, Sequence] = {}

    def step(self, entries: Seq[Tuple[str, List[int], List[int]]], end: Seq[str] = ()) -> Optional[torch.Tensor]:
        """``entries``: (request id, its next tokens, places among them whose logits are wanted).
        Runs them as ONE batch; returns float32 logits [wanted, vocab] in the order of the entries and
        of their wanted places (None when nothing is wanted).  ``end``: requests whose blocks and
        state slot go back to the pool after the step."""
        eng = self.engine
        bm, bs = eng.bm, eng.ecfg.kv_block_size
        dec, pre = [], []          # (entry index, seq, n)
        for k, (rid, toks, _want) in enumerate(entries):
            if not toks:
                continue
            seq = self.live.get(rid)
            if seq is None:
                seq = self.live[rid] = Sequence(list(toks), SamplingParams(max_new_tokens=1), request_id=rid)
                seq.status, seq.slot = SeqStatus.RUNNING, 0
            else:
                seq.prompt.extend(int(t) for t in toks)
            n = len(toks)
            if not bm.ensure_capacity(seq.seq_id, seq.num_cached + n):
                raise RuntimeError(f"no K/V blocks or state slot left for request {rid!r}")
            (dec if n == 1 and seq.num_cached > 0 else pre).append((k, seq, n))
        logits = None
        if dec or pre:
            hb_d = hb_p = None
            if dec:
                ids = np.array([s.seq_id for _, s, _ in dec], dtype=np.int64)
                lens = np.array([s.num_cached + 1 for _, s, _ in dec], dtype=np.int32)
                hb_d = build_decode_batch(ids, lens, bm, bs, int(-(-int(lens.max()) // bs)), eng.step_id)
                hb_d.ids = np.array([s.prompt[s.num_cached] for _, s, _ in dec], dtype=np.int32)
            if pre:
                for _, s, n in pre:
                    s.chunk = n
                hb_p = build_host_batch(Step(True, [s for _, s, _ in pre], 0), bm, bs, None, eng.step_id)
            hb = merge_mixed(hb_d, hb_p, 0, eng.step_id) if (dec and pre) else (hb_d or hb_p)
            if dec and pre and hb_d.state_slots is not None:
                hb.state_slots = np.concatenate([hb_d.state_slots, hb_p.state_slots])
            # rows whose logits are wanted, in the order of the entries
            order = dec + pre
            first = {}
            row = 0
            for k, _s, n in order:
                first[k] = row
                row += n
            wanted = [first[k] + int(w) for k, (_r, toks, want) in enumerate(entries) if toks for w in want]
            hb.logits_idx = np.asarray(wanted if wanted else [0], dtype=np.int32)
            if not hb.is_prefill:
                # a decode-only step returns every row's logits; keep the wanted ones below
                hb.logits_idx = np.arange(hb.num_seqs, dtype=np.int32)
            eng.step_id += 1
            out = eng.runner.execute(hb, slot=0)
            if wanted:
                logits = out.float() if hb.is_prefill else out.float().index_select(
                    0, torch.as_tensor(wanted, dtype=torch.int64, device=out.device))
            for _, s, n in order:
                s.num_cached += n
                s.chunk = 0
        for rid in end:
            seq = self.live.pop(rid, None)
            if seq is not None:
                bm.free_sequence(seq.seq_id)
                seq.finish("length")
        return logits
