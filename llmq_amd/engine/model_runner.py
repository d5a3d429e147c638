"""Model runner: batch tensor prep, forward execution, sampling, hipGraphs.

Decode steps are captured as hipGraphs per batch-size bucket (the vLLM
capability the reference relies on, SURVEY §2.9 "CUDA graph capture of
decode" → hipGraph here): all decode inputs live in static device buffers;
a step copies the small int tensors in, replays the graph, and samples from
the static logits buffer. Python/launch overhead per decode step drops to
one replay + one sampler call regardless of model depth.
"""

from __future__ import annotations

import logging
import time
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from llmq_amd import ops
from llmq_amd.engine.config import EngineConfig
from llmq_amd.engine.forward_meta import (
    ChunkGather, DecodeMeta, MixedMeta, PrefillMeta, RecurrentMeta,
)
from llmq_amd.engine.kv_cache import KVCache
from llmq_amd.engine.models.llama import CausalLM
from llmq_amd.engine.scheduler import ScheduledBatch, Sequence

logger = logging.getLogger(__name__)


def _buckets(max_bs: int) -> List[int]:
    sizes = [1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512]
    out = [b for b in sizes if b < max_bs]
    out.append(max_bs)
    return out


class ModelRunner:
    def __init__(
        self,
        model: CausalLM,
        kv_cache: KVCache,
        config: EngineConfig,
        device: torch.device,
        max_model_len: int,
    ):
        self.model = model
        self.kv_cache = kv_cache
        self.config = config
        self.device = device
        self.max_model_len = max_model_len
        self.block_size = kv_cache.block_size
        self.max_blocks_per_seq = (max_model_len + self.block_size - 1) // self.block_size
        self.use_graphs = (
            config.enable_hipgraph
            and not config.enforce_eager
            and device.type == "cuda"
        )
        self._graphs: Dict[int, torch.cuda.CUDAGraph] = {}
        self._graph_pool = None
        self.sampling_generator = torch.Generator(device=device if device.type == "cuda" else "cpu")
        self.sampling_generator.manual_seed(config.seed)
        self._sample_step = 0
        # Persistent sampler buffers, keyed by caller ("main" for the
        # decode path, "prefill" for the prefill segment of an OVERLAPPED
        # split mixed step — two concurrent streams must not share them).
        self._sample_bufs: Dict[str, Dict[str, torch.Tensor]] = {}
        self._staging_done = None  # event: last step's pinned→device copies landed
        # Models whose prompt-portion attention reads the paged cache through
        # the block table (no gathered K/V copy), and models with recurrent
        # layers (per-sequence state slots), get the extra step metadata.
        self.paged_prefill = bool(getattr(model, "paged_prefill", False))
        self.recurrent = kv_cache.recurrent if (
            kv_cache.recurrent is not None and kv_cache.recurrent.active) else None
        if self.use_graphs:
            self._alloc_static_buffers()

    # -- static buffers / graph capture ---------------------------------

    def _alloc_static_buffers(self) -> None:
        B = min(self.config.max_num_seqs, self.config.hipgraph_max_batch)
        dev = self.device
        self.graph_max_bs = B
        self.in_ids = torch.zeros(B, dtype=torch.long, device=dev)
        self.in_pos = torch.zeros(B, dtype=torch.long, device=dev)
        self.in_slots = torch.zeros(B, dtype=torch.long, device=dev)
        self.in_block_tables = torch.zeros(
            B, self.max_blocks_per_seq, dtype=torch.int32, device=dev
        )
        self.in_context_lens = torch.ones(B, dtype=torch.int32, device=dev)
        self.in_rec = None
        if self.recurrent is not None:
            # one row per sequence; slots are staged per step, rows never
            # start a sequence (decode rows sit on cached context)
            self.in_rec = RecurrentMeta(
                cu=torch.arange(B + 1, dtype=torch.int32, device=dev),
                slots=torch.full((B,), self.recurrent.pad_slot, dtype=torch.int32, device=dev),
                fresh=torch.zeros(B, dtype=torch.int32, device=dev),
            )
            self.h_rec_slots = torch.zeros(B, dtype=torch.int32, pin_memory=True)
            self.h_rec_fresh = torch.zeros(B, dtype=torch.int32, pin_memory=True)
        self.out_hidden = torch.zeros(
            B, self.model.spec.hidden_size, dtype=self.model.dtype, device=dev
        )
        # pinned host staging for fast H2D of the per-step metadata
        self.h_ids = torch.zeros(B, dtype=torch.long, pin_memory=True)
        self.h_pos = torch.zeros(B, dtype=torch.long, pin_memory=True)
        self.h_slots = torch.zeros(B, dtype=torch.long, pin_memory=True)
        self.h_block_tables = torch.zeros(
            B, self.max_blocks_per_seq, dtype=torch.int32, pin_memory=True
        )
        self.h_context_lens = torch.ones(B, dtype=torch.int32, pin_memory=True)
        # (seq uid, preemption count, staged_len) per row — incremental
        # block-table staging. Keyed on Sequence.uid (monotonic, never
        # reused), NOT request_id: callers may reuse request ids across
        # sequence lifetimes, and a reused id at the same row with an equal
        # table length but different blocks would leave the hipGraph reading
        # the old sequence's block ids. num_preemptions guards the same-life
        # case where preemption-by-recompute reassigns the whole table.
        self._staged_rows: List[Tuple[int, int, int]] = [(-1, -1, 0)] * B

    def capture_graphs(self) -> None:
        """Capture the decode forward for each batch-size bucket."""
        if not self.use_graphs:
            return
        t0 = time.perf_counter()
        torch.cuda.synchronize()
        for bs in reversed(_buckets(self.graph_max_bs)):  # large→small shares pool
            meta = DecodeMeta(
                block_tables=self.in_block_tables[:bs],
                context_lens=self.in_context_lens[:bs],
                slot_mapping=self.in_slots[:bs],
            )
            if self.in_rec is not None:
                meta.recurrent = RecurrentMeta(
                    cu=self.in_rec.cu[: bs + 1], slots=self.in_rec.slots[:bs],
                    fresh=self.in_rec.fresh[:bs],
                )
                # capture and warmup rows write the scratch slot only
                self.in_rec.slots.fill_(self.recurrent.pad_slot)
                self.in_rec.fresh.fill_(1)
            if self.paged_prefill:
                self.in_slots.fill_(-1)  # capture/warmup rows enter no cache slot
            # warmup (also materialises workspace allocations)
            out = self.model.forward(self.in_ids[:bs], self.in_pos[:bs], self.kv_cache, meta)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                out = self.model.forward(
                    self.in_ids[:bs], self.in_pos[:bs], self.kv_cache, meta
                )
                self.out_hidden[:bs].copy_(out)
            if self._graph_pool is None:
                self._graph_pool = graph.pool()
            self._graphs[bs] = graph
        torch.cuda.synchronize()
        logger.info(
            "captured %d decode hipGraphs (max_bs=%d) in %.1fs",
            len(self._graphs), self.graph_max_bs, time.perf_counter() - t0,
        )

    def _bucket_for(self, bs: int) -> Optional[int]:
        for b in _buckets(self.graph_max_bs):
            if b >= bs:
                return b
        return None

    # -- prefill / mixed (chunk-aware, eager) ----------------------------

    def _build_prefill_meta(self, pseqs, chunks, dev) -> tuple:
        """Packed ids/pos/slots for the prefill segment + optional gather
        plan for chunk continuations. Returns (ids, pos, slots, meta,
        rel_last_idx) where rel_last_idx are within-segment row indices of
        FINAL chunks (the rows that sample)."""
        bs = self.block_size
        ids: List[int] = []
        pos: List[int] = []
        slots: List[int] = []
        cu = [0]
        cu_k = [0]
        rel_last: List[int] = []
        any_chunk = (not self.paged_prefill) and any(start > 0 for (start, _e) in chunks)
        g_blocks: List[int] = []
        g_offs: List[int] = []
        past_dst: List[int] = []
        fresh_dst: List[int] = []
        krow = 0
        for seq, (start, end) in zip(pseqs, chunks):
            n = end - start
            ids.extend(seq.token_ids[start:end])
            pos.extend(range(start, end))
            bt = seq.block_table
            slots.extend(bt[p // bs] * bs + (p % bs) for p in range(start, end))
            if end == seq.num_tokens:
                rel_last.append(cu[-1] + n - 1)
            cu.append(cu[-1] + n)
            if any_chunk:
                for p in range(start):  # past rows gathered from the cache
                    g_blocks.append(bt[p // bs])
                    g_offs.append(p % bs)
                    past_dst.append(krow)
                    krow += 1
                for i in range(cu[-2], cu[-1]):
                    fresh_dst.append(krow)
                    krow += 1
            cu_k.append(cu_k[-1] + end)  # keys = full context so far
        slot_mapping = torch.tensor(slots, dtype=torch.long, device=dev)
        gather = None
        if any_chunk:
            gather = ChunkGather(
                cu_seqlens_k=torch.tensor(cu_k, dtype=torch.int32, device=dev),
                blocks=torch.tensor(g_blocks, dtype=torch.long, device=dev),
                offs=torch.tensor(g_offs, dtype=torch.long, device=dev),
                past_dst=torch.tensor(past_dst, dtype=torch.long, device=dev),
                fresh_dst=torch.tensor(fresh_dst, dtype=torch.long, device=dev),
                total_k=krow,
            )
        meta = PrefillMeta(
            cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=dev),
            max_seqlen=max(e - st for (st, e) in chunks),
            slot_mapping=slot_mapping,
            gather=gather,
        )
        if self.paged_prefill:
            meta.block_tables = self._block_table_tensor(pseqs, dev)
            meta.q_start = torch.tensor([st for (st, _e) in chunks], dtype=torch.int32, device=dev)
        if self.recurrent is not None:
            meta.recurrent = RecurrentMeta(
                cu=meta.cu_seqlens,
                slots=torch.tensor([s.state_slot for s in pseqs], dtype=torch.int32, device=dev),
                fresh=torch.tensor([int(st == 0) for (st, _e) in chunks], dtype=torch.int32,
                                   device=dev),
            )
        return ids, pos, slot_mapping, meta, rel_last

    def _block_table_tensor(self, seqs, dev) -> torch.Tensor:
        width = max(1, max(len(s.block_table) for s in seqs))
        bt_np = np.zeros((len(seqs), width), dtype=np.int32)
        for i, s in enumerate(seqs):
            bt_np[i, : len(s.block_table)] = s.block_table
        return torch.from_numpy(bt_np).to(dev)

    def _decode_recurrent_meta(self, seqs, dev):
        if self.recurrent is None:
            return None
        n = len(seqs)
        return RecurrentMeta(
            cu=torch.arange(n + 1, dtype=torch.int32, device=dev),
            slots=torch.tensor([s.state_slot for s in seqs], dtype=torch.int32, device=dev),
            fresh=torch.zeros(n, dtype=torch.int32, device=dev),
        )

    def _logits_at(self, hidden: torch.Tensor, rows: List[int]) -> torch.Tensor:
        """Logits of the given rows of a step (teacher-forced replay: the
        caller asks for positions instead of sampling)."""
        if not rows:
            return torch.empty(0, self.model.spec.vocab_size, dtype=torch.float32,
                               device=hidden.device)
        idx = torch.tensor(rows, dtype=torch.long, device=hidden.device)
        return self.model.compute_logits(hidden[idx]).float()

    @torch.no_grad()
    def execute_prefill(self, seqs: List[Sequence], chunks=None, buf_name: str = "main",
                        want=None) -> torch.Tensor:
        """Run a packed prefill segment; returns sampled next tokens for the
        rows whose context completed this step (all rows when no chunking).
        With ``want`` (per sequence, portion-relative positions) nothing is
        sampled: the logits of those rows are returned, in that order."""
        if chunks is None:
            chunks = [(0, s.num_tokens) for s in seqs]
        dev = self.device
        ids, pos, slot_mapping, meta, rel_last = self._build_prefill_meta(
            seqs, chunks, dev
        )
        input_ids = torch.tensor(ids, dtype=torch.long, device=dev)
        positions = torch.tensor(pos, dtype=torch.long, device=dev)
        hidden = self.model.forward(input_ids, positions, self.kv_cache, meta)
        if want is not None:
            cu = [0]
            for st, e in chunks:
                cu.append(cu[-1] + e - st)
            return self._logits_at(hidden, [cu[b] + w for b, ws in enumerate(want) for w in ws])
        if not rel_last:
            return torch.empty(0, dtype=torch.long, device=dev)
        last_hidden = hidden[torch.tensor(rel_last, dtype=torch.long, device=dev)]
        logits = self.model.compute_logits(last_hidden)
        sample_seqs = [s for s, (st, e) in zip(seqs, chunks) if e == s.num_tokens]
        return self._sample(logits, sample_seqs, buf_name)

    # -- mixed (decode rows + ride-along prefill rows, eager) ------------

    @torch.no_grad()
    def execute_mixed(self, batch: "ScheduledBatch", want=None) -> torch.Tensor:
        """Decode seqs[:n_decode] and prefill seqs[n_decode:] in ONE forward:
        shared GEMMs/norms over the packed rows, per-segment attention.
        Runs eager (prefill shapes vary); pure-decode steps keep hipGraphs.
        Returns tokens for [decode rows] + [final-chunk prefill rows]."""
        dev = self.device
        dseqs = batch.seqs[: batch.n_decode]
        pseqs = batch.seqs[batch.n_decode :]
        chunks = batch.chunks or [(0, s.num_tokens) for s in pseqs]
        bs = self.block_size
        nd = len(dseqs)

        ids = [s.token_ids[-1] for s in dseqs]
        pos = [s.num_tokens - 1 for s in dseqs]
        slots = [s.block_table[p // bs] * bs + (p % bs) for s, p in zip(dseqs, pos)]
        ctx = [s.num_tokens for s in dseqs]
        p_ids, p_pos, p_slots, pmeta, rel_last = self._build_prefill_meta(
            pseqs, chunks, dev
        )
        ids.extend(p_ids)
        pos.extend(p_pos)

        block_tables = torch.zeros(
            nd, max(len(s.block_table) for s in dseqs), dtype=torch.int32, device=dev
        )
        bt_np = np.zeros(tuple(block_tables.shape), dtype=np.int32)
        for i, s in enumerate(dseqs):
            bt_np[i, : len(s.block_table)] = s.block_table
        block_tables.copy_(torch.from_numpy(bt_np))
        d_slots = torch.tensor(slots, dtype=torch.long, device=dev)
        slot_mapping = torch.cat([d_slots, p_slots])
        meta = MixedMeta(
            n_decode=nd,
            decode=DecodeMeta(
                block_tables=block_tables,
                context_lens=torch.tensor(ctx, dtype=torch.int32, device=dev),
                slot_mapping=d_slots,
            ),
            prefill=pmeta,
            slot_mapping=slot_mapping,
        )
        if self.recurrent is not None:
            dr, pr = self._decode_recurrent_meta(dseqs, dev), pmeta.recurrent
            meta.decode.recurrent = dr
            meta.recurrent = RecurrentMeta(
                cu=torch.cat([dr.cu[:-1], pr.cu + nd]),
                slots=torch.cat([dr.slots, pr.slots]),
                fresh=torch.cat([dr.fresh, pr.fresh]),
            )
        input_ids = torch.tensor(ids, dtype=torch.long, device=dev)
        positions = torch.tensor(pos, dtype=torch.long, device=dev)
        hidden = self.model.forward(input_ids, positions, self.kv_cache, meta)
        if want is not None:
            cu = [nd]
            for st, e in chunks:
                cu.append(cu[-1] + e - st)
            rows = [b for b, ws in enumerate(want[:nd]) if ws]
            rows += [cu[b] + w for b, ws in enumerate(want[nd:]) for w in ws]
            return self._logits_at(hidden, rows)
        last_idx = list(range(nd)) + [nd + r for r in rel_last]
        last_hidden = hidden[torch.tensor(last_idx, dtype=torch.long, device=dev)]
        logits = self.model.compute_logits(last_hidden)
        sample_seqs = list(dseqs) + [
            s for s, (st, e) in zip(pseqs, chunks) if e == s.num_tokens
        ]
        return self._sample(logits, sample_seqs)

    # -- decode ----------------------------------------------------------

    @torch.no_grad()
    def execute_decode(self, seqs: List[Sequence], force_eager: bool = False,
                       want=None) -> torch.Tensor:
        dev = self.device
        B = len(seqs)
        bs = self.block_size
        ids = [s.token_ids[-1] for s in seqs]
        pos = [s.num_tokens - 1 for s in seqs]
        slots = [s.block_table[p // bs] * bs + (p % bs) for s, p in zip(seqs, pos)]
        ctx = [s.num_tokens for s in seqs]

        bucket = self._bucket_for(B) if (self.use_graphs and not force_eager) else None
        if bucket is not None and bucket in self._graphs:
            return self._decode_with_graph(seqs, bucket, ids, pos, slots, ctx, want)

        block_tables = torch.zeros(
            B, max(len(s.block_table) for s in seqs), dtype=torch.int32, device=dev
        )
        bt_np = np.zeros(tuple(block_tables.shape), dtype=np.int32)
        for i, s in enumerate(seqs):
            bt_np[i, : len(s.block_table)] = s.block_table
        block_tables.copy_(torch.from_numpy(bt_np))
        meta = DecodeMeta(
            block_tables=block_tables,
            context_lens=torch.tensor(ctx, dtype=torch.int32, device=dev),
            slot_mapping=torch.tensor(slots, dtype=torch.long, device=dev),
            recurrent=self._decode_recurrent_meta(seqs, dev),
        )
        input_ids = torch.tensor(ids, dtype=torch.long, device=dev)
        positions = torch.tensor(pos, dtype=torch.long, device=dev)
        hidden = self.model.forward(input_ids, positions, self.kv_cache, meta)
        if want is not None:
            return self._logits_at(hidden, [b for b, ws in enumerate(want) if ws])
        logits = self.model.compute_logits(hidden)
        return self._sample(logits, seqs)

    def _decode_with_graph(
        self, seqs: List[Sequence], bucket: int, ids, pos, slots, ctx, want=None
    ) -> torch.Tensor:
        B = len(seqs)
        # The pinned staging buffers are rewritten every step: the previous
        # step's async copies out of them must have landed first. Sampling
        # steps synchronise anyway (tokens go to the host); a replay step
        # that wants no logits does not.
        if self._staging_done is not None:
            self._staging_done.synchronize()
        # Stage metadata through pinned host buffers, one async copy each.
        self.h_ids[:B] = torch.tensor(ids, dtype=torch.long)
        self.h_pos[:B] = torch.tensor(pos, dtype=torch.long)
        self.h_slots[:B] = torch.tensor(slots, dtype=torch.long)
        self.h_context_lens[:B] = torch.tensor(ctx, dtype=torch.int32)
        self.h_context_lens[B:bucket] = 1
        # Block tables are staged INCREMENTALLY: a row is rewritten only when
        # its (request, table length) changed since the last stage. With
        # max_model_len in the 100k class the table is thousands of columns
        # wide — rewriting every row every step cost more host time than the
        # whole decode step (measured on llama-3.2-3b, max_blocks=8192).
        bt_np = self.h_block_tables.numpy()
        max_w = 1
        for i, s in enumerate(seqs):
            n = len(s.block_table)
            if n > max_w:
                max_w = n
            if self._staged_rows[i] != (s.uid, s.num_preemptions, n):
                bt_np[i, :n] = s.block_table
                self._staged_rows[i] = (s.uid, s.num_preemptions, n)
        if B < bucket:
            # pad rows: context_len 1 pointing at block 0 (defined garbage,
            # their logits are never read)
            # padding rows of a paged-prefill model enter no cache slot at all
            self.h_slots[B:bucket] = -1 if self.paged_prefill else 0
            self.h_ids[B:bucket] = 0
            self.h_pos[B:bucket] = 0
            for i in range(B, bucket):
                if self._staged_rows[i] != (-1, -1, 0):
                    bt_np[i, :1] = 0
                    self._staged_rows[i] = (-1, -1, 0)
        self.in_ids[:bucket].copy_(self.h_ids[:bucket], non_blocking=True)
        self.in_pos[:bucket].copy_(self.h_pos[:bucket], non_blocking=True)
        self.in_slots[:bucket].copy_(self.h_slots[:bucket], non_blocking=True)
        self.in_context_lens[:bucket].copy_(self.h_context_lens[:bucket], non_blocking=True)
        self.in_block_tables[:bucket, :max_w].copy_(
            self.h_block_tables[:bucket, :max_w], non_blocking=True
        )
        if self.in_rec is not None:
            # padding rows advance the scratch slot from zero, never a live one
            self.h_rec_slots[:B] = torch.tensor([s.state_slot for s in seqs], dtype=torch.int32)
            self.h_rec_slots[B:bucket] = self.recurrent.pad_slot
            self.h_rec_fresh[:B] = 0
            self.h_rec_fresh[B:bucket] = 1
            self.in_rec.slots[:bucket].copy_(self.h_rec_slots[:bucket], non_blocking=True)
            self.in_rec.fresh[:bucket].copy_(self.h_rec_fresh[:bucket], non_blocking=True)
        if self._staging_done is None:
            self._staging_done = torch.cuda.Event()
        self._staging_done.record()
        self._graphs[bucket].replay()
        if want is not None:
            return self._logits_at(self.out_hidden[:B], [b for b, ws in enumerate(want) if ws])
        logits = self.model.compute_logits(self.out_hidden[:B])
        return self._sample(logits, seqs)

    # -- sampling --------------------------------------------------------

    def _sample_buf(self, name: str, B: int, dev) -> Dict[str, torch.Tensor]:
        buf = self._sample_bufs.get(name)
        if buf is None or buf["out"].numel() < B:
            cap = max(B, self.config.max_num_seqs)
            buf = {
                "out": torch.empty(cap, dtype=torch.int64, device=dev),
                "keys": torch.empty(cap, dtype=torch.int64, device=dev),
                "temps": torch.empty(cap, dtype=torch.float32, device=dev),
                "temps_h": torch.empty(cap, dtype=torch.float32, pin_memory=True),
                "seeds": torch.empty(cap, dtype=torch.int32, device=dev),
                "seeds_h": torch.empty(cap, dtype=torch.int32, pin_memory=True),
                "pos": torch.empty(cap, dtype=torch.int32, device=dev),
                "pos_h": torch.empty(cap, dtype=torch.int32, pin_memory=True),
            }
            self._sample_bufs[name] = buf
        return buf

    def _sample(self, logits: torch.Tensor, seqs: List[Sequence],
                buf_name: str = "main") -> torch.Tensor:
        dev = logits.device
        self._sample_step += 1
        simple = all(
            s.params.top_k == 0 and s.params.top_p >= 1.0 for s in seqs
        )
        if dev.type == "cuda":
            # Fused one-pass HIP sampler (gumbel-max / greedy argmax).
            # Top-k/top-p rows reduce to a per-row logit keep-bound via
            # histogram select — no full-vocab sort, no CPU round trips,
            # seeded rows stay on-device (ADVICE r1 low #4 / weakness 6).
            B = len(seqs)
            buf = self._sample_buf(buf_name, B, dev)
            th = buf["temps_h"]
            sh = buf["seeds_h"]
            ph = buf["pos_h"]
            for i, s in enumerate(seqs):
                th[i] = s.params.temperature
                rs = s.params.seed
                if rs is None:
                    sh[i] = 0  # unseeded sentinel
                else:
                    v = rs & 0x7FFFFFFF
                    sh[i] = v if v else 0x1E3779B9  # remap literal seed 0
                ph[i] = s.output_len
            buf["temps"][:B].copy_(th[:B], non_blocking=True)
            buf["seeds"][:B].copy_(sh[:B], non_blocking=True)
            buf["pos"][:B].copy_(ph[:B], non_blocking=True)
            logits_f = logits.float()
            bounds = None
            if not simple:
                tps = torch.tensor([s.params.top_p for s in seqs],
                                   dtype=torch.float32, device=dev)
                tks = torch.tensor([s.params.top_k for s in seqs],
                                   dtype=torch.int64, device=dev)
                bounds = ops.topk_topp_bound(
                    logits_f, buf["temps"][:B], tps, tks)
            ops.sample_gumbel_argmax(
                buf["out"][:B], buf["keys"][:B], logits_f,
                buf["temps"][:B], buf["seeds"][:B],
                buf["pos"][:B], self.config.seed, self._sample_step, bounds,
            )
            return buf["out"][:B]
        temps = torch.tensor([s.params.temperature for s in seqs], dtype=torch.float32, device=dev)
        tps = torch.tensor([s.params.top_p for s in seqs], dtype=torch.float32, device=dev)
        tks = torch.tensor([s.params.top_k for s in seqs], dtype=torch.int64, device=dev)
        out = ops.sample_tokens(logits, temps, tps, tks, self.sampling_generator)
        # Per-request seeds (reproducible sampling): re-draw those rows with
        # a generator keyed on (seed, output position) — batch-independent.
        # Gathered in ONE device→host transfer (a per-row .cpu() would sync
        # the stream once per seeded row per step).
        seeded = [
            i for i, s in enumerate(seqs)
            if s.params.seed is not None and s.params.temperature > 0
        ]
        if seeded:
            idx = torch.tensor(seeded, dtype=torch.long, device=dev)
            rows = logits[idx].float().cpu()
            temps_c, tps_c, tks_c = temps[idx].cpu(), tps[idx].cpu(), tks[idx].cpu()
            redraw = torch.empty(len(seeded), dtype=out.dtype)
            for j, i in enumerate(seeded):
                s = seqs[i]
                g = torch.Generator(device="cpu")
                g.manual_seed((s.params.seed << 20) ^ s.output_len)
                redraw[j] = ops.sample_tokens(
                    rows[j : j + 1], temps_c[j : j + 1], tps_c[j : j + 1],
                    tks_c[j : j + 1], g,
                )[0]
            out[idx] = redraw.to(out.device)
        return out
