"""The step function of hybrid models (sequences that own recurrent-state slots beside their K/V pages).

A step is a list of ROW RUNS, one per sequence: `count` tokens that continue the sequence at position `start` - a whole
prompt, a portion of one, or a single decoded token; the kernels make no difference between them (layers/seqmix.py), so
portions of prompts and decoded tokens of other sequences share a batch.  ModelRunner mixes this class in: `run()` turns
the scheduler's prefill / decode steps into row runs, a trace replay (bin/trace_run) calls `run_rows` with the cut it was
given.

Metadata reaches the device as in ModelRunner.prepare_prefill: every array of the step packed into one pinned staging
buffer (two, alternating) and uploaded with one copy.
"""
from __future__ import annotations

import numpy as np
import torch

from nanovllm.utils.context import reset_context, set_context


class RowSteps:
    # ------------------------------------------------------------------ cache and state
    def allocate_hybrid_cache(self):
        """Pages for the attention layers and state slots for the recurrent ones.  num_kvcache_blocks counts the reserved
        last block as in the paged-attention models' cache (the scheduler hands out the others)."""
        cfg = self.config
        item = 4 if self.dtype == torch.float32 else 2
        per_block = max(1, self.model.cache_bytes_per_block(self.block_size, item))
        n_slots = cfg.num_state_slots or cfg.max_num_seqs
        if cfg.num_kvcache_blocks <= 0:
            free, total = torch.cuda.mem_get_info(self.device)
            budget = total * cfg.gpu_memory_utilization - (total - free) - n_slots * self.model.state_bytes_per_slot()
            cfg.num_kvcache_blocks = int(budget) // per_block
        assert cfg.num_kvcache_blocks > 1, "no memory left for the K/V pages"
        self.n_state_slots = n_slots
        # (one slot more than the scheduler hands out: the padded rows of a captured step write their state there)
        self.model.bind_cache(cfg.num_kvcache_blocks, self.block_size, n_slots + 1, self.dtype, self.device)

    def _alloc_row_staging(self):
        nbytes = 1 << 16
        self._row_hosts = [torch.empty(nbytes, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self._row_dev = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self._row_flip = 0
        self._row_events = [None, None]

    # ------------------------------------------------------------------ metadata
    def prepare_rows(self, runs, want):
        """runs: [(sequence, start, count)], want: step rows whose logits are asked for.  Installs the step's context and
        returns (input ids, wanted rows) on the device."""
        bs = self.block_size
        n = len(runs)
        counts = np.fromiter((c for _, _, c in runs), dtype=np.int64, count=n)
        cu = np.zeros(n + 1, dtype=np.int32)
        np.cumsum(counts, out=cu[1:])
        total = int(cu[-1])
        ids = np.empty(total, dtype=np.int64)
        slots = np.empty(total, dtype=np.int32)
        kv_lens = np.empty(n, dtype=np.int32)
        state_slots = np.empty(n, dtype=np.int32)
        width = max(1, max(-(-(s0 + c) // bs) for _, s0, c in runs))
        tables = np.full((n, width), -1, dtype=np.int32)
        for i, (seq, start, count) in enumerate(runs):
            a = int(cu[i])
            assert count >= 1 and start + count <= len(seq) and len(seq.block_table) * bs >= start + count, \
                (start, count, len(seq), len(seq.block_table))
            ids[a:a + count] = seq.token_ids[start:start + count]
            pos = np.arange(start, start + count)
            table = np.asarray(seq.block_table, dtype=np.int32)
            slots[a:a + count] = table[pos // bs] * bs + pos % bs
            kv_lens[i] = start + count
            assert seq.state_slot >= 0
            state_slots[i] = seq.state_slot
            nb = -(-(start + count) // bs)
            tables[i, :nb] = table[:nb]
        want = np.asarray(want, dtype=np.int64)
        arrays = (ids, slots, cu, kv_lens, state_slots, tables, want)
        offs, off = [], 0
        for a in arrays:
            offs.append(off)
            off += (a.nbytes + 15) // 16 * 16
        self._row_flip ^= 1
        b = self._row_flip
        if self._row_events[b] is not None:
            self._row_events[b].synchronize()  # the upload that last read this pinned buffer has run
        if off > self._row_hosts[b].numel():
            self._row_hosts[b] = torch.empty(off * 2, dtype=torch.uint8, pin_memory=True)
        if off > self._row_dev.numel():
            self._row_dev = torch.empty(off * 2, dtype=torch.uint8, device=self.device)
        host = self._row_hosts[b].numpy()
        for a, o in zip(arrays, offs):
            host[o:o + a.nbytes] = np.ascontiguousarray(a).reshape(-1).view(np.uint8)
        self._row_dev[:off].copy_(self._row_hosts[b][:off], non_blocking=True)
        ev = self._row_events[b] or torch.cuda.Event()
        ev.record()
        self._row_events[b] = ev

        def dev(i, dtype, shape=None):
            t = self._row_dev[offs[i]:offs[i] + arrays[i].nbytes].view(dtype)
            return t if shape is None else t.view(shape)

        set_context(True, cu_seqlens_q=dev(2, torch.int32), kv_lens=dev(3, torch.int32), slot_mapping=dev(1, torch.int32),
                    block_tables=dev(5, torch.int32, tables.shape), block_size=bs, state_slots=dev(4, torch.int32),
                    max_seqlen_q=int(counts.max()), max_seqlen_k=int(kv_lens.max()))
        return dev(0, torch.int64), dev(6, torch.int64)

    # ------------------------------------------------------------------ one step
    @torch.inference_mode()
    def run_rows(self, runs, want=None) -> torch.Tensor:
        """One step over the row runs; returns fp32 logits [len(want), vocab] on the device (default: each run's last row).
        The sequences' pages and state slots must be in place (Scheduler.admit_portion / schedule())."""
        if want is None:
            ends = np.cumsum([c for _, _, c in runs])
            want = (ends - 1).tolist()
        input_ids, rows = self.prepare_rows(runs, want)
        hidden = self.model(input_ids)
        logits = self.model.compute_logits(hidden, rows) if len(want) else None
        for seq, start, count in runs:
            seq.num_computed_tokens = start + count
        self._steps_run += 1
        reset_context()
        return logits

    # ------------------------------------------------------------------ captured decode steps
    def _row_graph_layout(self):
        cfg = self.config
        B = cfg.max_num_seqs
        cols = -(-cfg.max_model_len // self.block_size)
        off, spans = 0, {}
        for name, nbytes in (("ids", 8 * B), ("want", 8 * B), ("slots", 4 * B), ("cu", 4 * (B + 1)), ("kv", 4 * B),
                             ("state", 4 * B), ("tables", 4 * B * cols)):
            spans[name] = (off, nbytes)
            off += (nbytes + 15) // 16 * 16

        def views(buf):
            def v(name, dtype, shape):
                o, n = spans[name]
                return buf[o:o + n].view(dtype).view(shape)
            return {"ids": v("ids", torch.int64, (B,)), "want": v("want", torch.int64, (B,)),
                    "slots": v("slots", torch.int32, (B,)), "cu": v("cu", torch.int32, (B + 1,)),
                    "kv": v("kv", torch.int32, (B,)), "state": v("state", torch.int32, (B,)),
                    "tables": v("tables", torch.int32, (B, cols))}
        return off, cols, views

    @torch.inference_mode()
    def capture_row_graphs(self):
        """Decode steps - one row per sequence - of the batch buckets 1, 2, 4, ..., max_num_seqs as hipGraphs (the
        counterpart of ModelRunner.capture_decode_graphs for the row-step path).  The step's metadata sits at fixed
        addresses of one static device buffer; padded rows are token 0 of a one-token sequence that stores no K/V row
        (slot -1), reads the reserved last page and keeps its state in the spare slot.  The graph ends in the fp32
        logits of every row; sampling stays outside."""
        from nanovllm.engine.model_runner import CAPTURE_MODE, graph_buckets

        cfg = self.config
        nbytes, cols, views = self._row_graph_layout()
        self._rg_cols = cols
        self._rg_dev_buf = torch.zeros(nbytes, dtype=torch.uint8, device=self.device)
        self._rg_dev = views(self._rg_dev_buf)
        self._rg_host_bufs = [torch.zeros(nbytes, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self._rg_hosts = [{k: t.numpy() for k, t in views(b).items()} for b in self._rg_host_bufs]
        self._rg_events = [None, None]
        self._rg_flip = 0
        d, pool = self._rg_dev, None
        for bs in reversed(graph_buckets(cfg.max_num_seqs)):
            self._stage_row_graph([], bs)
            set_context(True, cu_seqlens_q=d["cu"][:bs + 1], kv_lens=d["kv"][:bs], slot_mapping=d["slots"][:bs],
                        block_tables=d["tables"][:bs], block_size=self.block_size, state_slots=d["state"][:bs],
                        max_seqlen_q=1, max_seqlen_k=cfg.max_model_len)

            def body(bs=bs):
                return self.model.compute_logits(self.model(d["ids"][:bs]))

            side = torch.cuda.Stream(device=self.device)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):  # warm-up run outside capture
                body()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=pool, capture_error_mode=CAPTURE_MODE):
                logits = body()
            pool = pool or graph.pool()
            self.row_graphs[bs] = graph
            self.row_graph_logits[bs] = logits
        reset_context()
        torch.cuda.synchronize()

    def _stage_row_graph(self, seqs, bucket: int) -> None:
        """Metadata of a decode step (every sequence's last token) at the static buffer's addresses, padded to the bucket."""
        self._rg_flip ^= 1
        b = self._rg_flip
        if self._rg_events[b] is not None:
            self._rg_events[b].synchronize()
        h, bs, real = self._rg_hosts[b], self.block_size, len(seqs)
        h["cu"][:] = np.arange(h["cu"].shape[0], dtype=np.int32)
        h["want"][:] = np.arange(h["want"].shape[0], dtype=np.int64)
        for i, s in enumerate(seqs):
            n = len(s)
            assert s.state_slot >= 0 and len(s.block_table) * bs >= n and len(s.block_table) <= self._rg_cols
            h["ids"][i] = s.last_token
            h["slots"][i] = s.block_table[(n - 1) // bs] * bs + (n - 1) % bs
            h["kv"][i] = n
            h["state"][i] = s.state_slot
            h["tables"][i, :len(s.block_table)] = s.block_table
        h["ids"][real:bucket] = 0
        h["slots"][real:bucket] = -1
        h["kv"][real:bucket] = 1
        h["state"][real:bucket] = self.n_state_slots          # the spare slot
        h["tables"][real:bucket, 0] = self.config.num_kvcache_blocks - 1   # the reserved page
        self._rg_dev_buf.copy_(self._rg_host_bufs[b], non_blocking=True)
        ev = self._rg_events[b] or torch.cuda.Event()
        ev.record()
        self._rg_events[b] = ev

    @torch.inference_mode()
    def run_row_step(self, runs) -> list[int]:
        """One scheduler step of row runs (Scheduler.schedule_rows): portions and decoded tokens together; the runs that
        reach their sequence's end get a token from the framework's sampler, in run order.  A step of single completing
        rows is a decode step and replays its captured graph."""
        done = [s for s, start, count in runs if start + count == len(s)]
        if len(done) == len(runs) and all(count == 1 for _, _, count in runs):
            return self.run_hybrid(done, False)
        ends = np.cumsum([c for _, _, c in runs])
        want = [int(e) - 1 for e, (s, start, count) in zip(ends, runs) if start + count == len(s)]
        logits = self.run_rows(runs, want)
        if not done:
            torch.cuda.current_stream().synchronize()
            return []
        self.last_logits = logits
        return self._sample_rows(logits, done)

    def _sample_rows(self, logits, seqs) -> list[int]:
        real = len(seqs)
        temps = torch.tensor([0.0 if s.greedy else s.temperature for s in seqs], dtype=torch.float32).to(self.device)
        # the sampler reads bf16 logits in rows of a multiple of 8 elements (layers/sampler.py)
        vocab = logits.shape[1]
        rounded = torch.empty((real, -(-vocab // 8) * 8), dtype=torch.bfloat16, device=self.device)[:, :vocab]
        rounded.copy_(logits)
        self.sampler(rounded, temps, out=self.tokens_dev[:real])
        return self.tokens_dev[:real].tolist()

    @torch.inference_mode()
    def run_hybrid(self, seqs, is_prefill: bool) -> list[int]:
        """ModelRunner.run for a hybrid model: the scheduler's prefill step (whole prompts; a preempted sequence comes back
        with its completion tokens and is recomputed from position 0, its state from zero) or decode step as row runs,
        then the framework's sampler on the last rows."""
        real = len(seqs)
        bucket = None if is_prefill else next((b for b in sorted(self.row_graphs) if b >= real), None)
        if bucket is not None:
            self._stage_row_graph(seqs, bucket)
            self.row_graphs[bucket].replay()
            logits = self.row_graph_logits[bucket][:real]
            for s in seqs:
                s.num_computed_tokens = len(s)
            self._steps_run += 1
        else:
            runs = [(s, 0, len(s)) if is_prefill else (s, len(s) - 1, 1) for s in seqs]
            logits = self.run_rows(runs)
        self.last_logits = logits
        return self._sample_rows(logits, seqs)
