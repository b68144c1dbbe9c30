"""HIP-graph capture/replay of the per-stage decode step (N5 in SURVEY §2.2).

A decode step of an 8B model is ~300 kernel launches; eager launch costs ~3-4 us
each on the host, so the step is captured once per (batch bucket, context bucket) and
replayed.  Inputs are copied into persistent device buffers; padded rows of a bucket
write their K/V into the reserved scratch block 0 (slot 0) and attend to one token,
so they never touch a live sequence.
"""
from __future__ import annotations

import threading
from typing import Dict, Optional, Tuple

import torch

from ..models.stage import BatchMeta, ModelStage
from .batch import HostBatch, next_pow2

SCRATCH_SEQ_ID = -1      # owns block 0 (and state slot 0) in the BlockManager
NROWS = 5                # per-row int32 inputs: ids, positions, slots, seq_lens, state slots
_CAPTURE_LOCK = threading.Lock()   # one graph capture at a time per process


class DecodeGraphRunner:
    def __init__(self, stage: ModelStage, max_batch: int, max_blocks: int, batch_sizes,
                 min_ctx_bucket: int = 256):
        self.stage = stage
        self.dev = stage.device
        self.max_batch = max(batch_sizes) if batch_sizes else max_batch
        self.max_batch = max(self.max_batch, 1)
        self.max_blocks = max_blocks
        self.block_size = stage.kv.block_size
        self.batch_sizes = sorted(set(b for b in batch_sizes if b <= self.max_batch)) or [self.max_batch]
        self.min_ctx_bucket = min_ctx_bucket
        cfg = stage.cfg
        mb, dev = self.max_batch, self.dev
        # every int32 graph input lives in ONE device buffer laid out like the pinned staging
        # buffer -- [ids | positions | slots | seq_lens | state slots] x max_batch, then the block
        # table rows -- so a step's inputs go up in a single H2D copy (the first
        # 5 * max_batch + bb * max_blocks ints) instead of six
        self.dev_in = torch.zeros(NROWS * mb + mb * max_blocks, dtype=torch.int32, device=dev)
        self.ids = self.dev_in[0:mb]
        self.positions = self.dev_in[mb:2 * mb]
        self.slots = self.dev_in[2 * mb:3 * mb]
        self.seq_lens = self.dev_in[3 * mb:4 * mb]
        self.seq_lens.fill_(1)
        self.state_slots = self.dev_in[4 * mb:5 * mb]
        self.block_tables = self.dev_in[NROWS * mb:].view(mb, max_blocks)
        # models with per-sequence state: a decode step is one token per sequence, so the token ->
        # sequence map and the chunk offsets are constants
        self.with_state = bool(getattr(cfg, "needs_state_slots", False))
        self.with_seq_index = self.with_state or bool(getattr(cfg, "needs_seq_index", False))
        self.row_ids = torch.arange(mb + 1, dtype=torch.int32, device=dev) if self.with_seq_index else None
        self.hidden = None if stage.is_first else torch.zeros(mb, stage.in_width, dtype=stage.dtype, device=dev)
        max_splits = 64
        self.ws = (torch.empty(mb * cfg.num_heads * max_splits * cfg.head_dim, dtype=torch.float32, device=dev),
                   torch.empty(mb * cfg.num_heads * max_splits * 2, dtype=torch.float32, device=dev))
        self.pinned = torch.empty(NROWS * mb + mb * max_blocks, dtype=torch.int32).pin_memory()
        self.pinned_np = self.pinned.numpy()
        self.graphs: Dict[Tuple[int, int], Tuple[torch.cuda.CUDAGraph, torch.Tensor]] = {}
        self.pool = None
        self.copy_done: Optional[torch.cuda.Event] = None
        self.capture_stream: Optional[torch.cuda.Stream] = None

    def bucket(self, b: int, max_ctx: int) -> Tuple[int, int]:
        bb = next(x for x in self.batch_sizes if x >= b)
        cb = min(next_pow2(max_ctx, self.min_ctx_bucket), self.max_blocks * self.block_size)
        return bb, cb

    def can_run(self, b: int, max_ctx: int) -> bool:
        return b <= self.max_batch and max_ctx <= self.max_blocks * self.block_size

    def _meta(self, bb: int, cb: int) -> BatchMeta:
        meta = BatchMeta(is_prefill=False, positions=self.positions[:bb], slot_mapping=self.slots[:bb],
                         block_tables=self.block_tables[:bb], seq_lens=self.seq_lens[:bb], max_q_len=1,
                         max_ctx=cb, num_seqs=bb, num_tokens=bb, attn_workspace=self.ws)
        if self.with_state:
            meta.state_slots = self.state_slots[:bb]
        if self.with_seq_index:
            meta.tok_seq = self.row_ids[:bb]
            meta.cu_seqlens_q = self.row_ids[:bb + 1]
        return meta

    def _inp(self, bb: int) -> torch.Tensor:
        return self.ids[:bb] if self.stage.is_first else self.hidden[:bb]

    def capture(self, bb: int, cb: int):
        with _CAPTURE_LOCK:
            return self._capture(bb, cb)

    def _capture(self, bb: int, cb: int):
        # the warm-up forwards below really run: every row is made a scratch row first (block 0,
        # state slot 0, position 0), so they cannot advance a live sequence's recurrent state or
        # convolution tail; run() loads the step's inputs after the capture
        self.dev_in.zero_()
        self.seq_lens.fill_(1)
        meta = self._meta(bb, cb)
        # warm up outside capture (allocator, lazy module init)
        if self.capture_stream is None:
            self.capture_stream = torch.cuda.Stream(self.dev)
        s = self.capture_stream
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):
                self.stage.forward(self._inp(bb), meta)
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        # own capture stream: per-stream GEMM workspaces stay private to this runner's graphs;
        # thread_local mode: RCCL/gloo threads of this process may keep calling HIP meanwhile
        with torch.cuda.graph(g, pool=self.pool, stream=s, capture_error_mode="thread_local"):
            out = self.stage.forward(self._inp(bb), meta)
        self.graphs[(bb, cb)] = (g, out)
        return g, out

    def load_inputs(self, hb: HostBatch, bb: int, hidden: Optional[torch.Tensor] = None):
        b = hb.num_seqs
        mbk = hb.block_tables.shape[1]
        if mbk > self.max_blocks:
            raise ValueError("block table wider than graph buffers")
        if self.copy_done is not None:
            self.copy_done.synchronize()   # previous step's H2D may still read the pinned buffer
        # numpy views of the pinned staging buffer: a handful of memcpy-sized writes per step
        # instead of one torch op (~5-10 us of host time each) per field
        n, mb, w = bb, self.max_batch, self.max_blocks
        p = self.pinned_np
        pv = p[: NROWS * mb].reshape(NROWS, mb)
        pv[0, :b] = hb.ids
        pv[1, :b] = hb.positions
        pv[2, :b] = hb.slots
        pv[3, :b] = hb.seq_lens
        pv[4, :b] = hb.state_slots if hb.state_slots is not None else 0
        if n > b:                                       # padded rows: scratch slot 0, one token
            pv[:3, b:n] = 0
            pv[3, b:n] = 1
            pv[4, b:n] = 0
        bt = p[NROWS * mb: NROWS * mb + n * w].reshape(n, w)
        bt[:b, :mbk] = hb.block_tables
        bt[:b, mbk:] = 0
        bt[b:] = 0
        cnt = NROWS * mb + n * w
        self.dev_in[:cnt].copy_(self.pinned[:cnt], non_blocking=True)
        if self.copy_done is None:
            self.copy_done = torch.cuda.Event()
        self.copy_done.record()
        if hidden is not None:
            self.hidden[:b].copy_(hidden[:b])
            if bb > b:
                self.hidden[b:bb].zero_()

    def run(self, hb: HostBatch, hidden: Optional[torch.Tensor] = None,
            ids_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Replay the bucket's graph; returns the (static) output truncated to the real batch.
        ``ids_dev``: device-resident input ids overriding ``hb.ids`` (lookahead decode)."""
        b = hb.num_seqs
        bb, cb = self.bucket(b, hb.max_ctx)
        entry = self.graphs.get((bb, cb))
        if entry is None:
            entry = self.capture(bb, cb)       # clears the input buffers: before this step's inputs go up
        self.load_inputs(hb, bb, hidden)
        if ids_dev is not None:
            self.ids[:b].copy_(ids_dev, non_blocking=True)
        g, out = entry
        g.replay()
        return out[:b]
