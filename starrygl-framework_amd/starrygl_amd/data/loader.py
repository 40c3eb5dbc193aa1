"""Mini-batch loader over an event stream: the caller of the hot path.

The reference drives its sampler from `AsyncPipelineLoader(dataset, graph_engine=g, collator, sampling_config,
..., mode='CTDG', prefetch_factor, negative_sampler)` (call sites test/test.py:212-221,
test/test_dataloader.py:119-149; the class itself is not part of the reference tree).  `EventBatchLoader` plays
that part for one GPU: it walks the events in order, `batch_size` at a time, draws the negatives
(`NegSamplingSet.sample`, starrygl/graph/graph.py:15-26), and keeps `prefetch` batches in flight on a
`MiniBatchPipelinePool`.  The roots of a batch are the endpoints of its events at the events' times, a stream
that is known before the first batch: the loader looks up where each of those windows ends once, at
construction, and every batch then carries its values, so the sampler searches for the negatives only.
"""
import torch

from .pipeline import MiniBatchGroupPool, MiniBatchPipelinePool


class EventBatchLoader:
    def __init__(self, graph, src, dst, ts, batch_size, num_neg, layers, fanout, sample_type="recent",
                 node_tables=None, edge_tables=None, time_encoder=None, prefetch=4, negative_sampler=None,
                 drop_last=True, sample_ahead=1, **pipeline_kwargs):
        """graph: `pyGraph.g` / `CUDAGraph`.  src/dst/ts: the events in training order (int64, any device).
        num_neg: negatives per batch (their times repeat the batch's event times).  negative_sampler: an
        object with `sample(num_samples, num_groups)` (NegSamplingSet); default: uniform over all nodes.
        prefetch: batches in flight (pipelines of the pool; a process has four hardware queues, and
        pipelines that share one take turns).  sample_ahead: mini-batches per pass of the library calls; above 1
        the loader runs groups of that many consecutive batches through MiniBatchGroupPipeline objects (the
        batched sampler and unique: a batch of a group costs a fraction of a batch sampled alone), `prefetch`
        then counts groups in flight (three keep the GPU busy while the host reads a finished group's counts; with two
        the passes wait for the host), and a yielded batch stays valid until all batches of its
        group and of the `prefetch - 2` following groups have been yielded.  Remaining keywords go to the pipelines.
        Only full batches are produced (every buffer of a pipeline is planned for one batch shape)."""
        if not drop_last:
            raise ValueError("EventBatchLoader produces full batches only (drop_last=True)")
        dev = graph._hp.be.device
        as_dev = lambda t: torch.as_tensor(t).to(device=dev, dtype=torch.int64).contiguous()
        self.src, self.dst, self.ts = as_dev(src), as_dev(dst), as_dev(ts)
        self.B, self.num_neg = int(batch_size), int(num_neg)
        self.graph = graph
        self.negative_sampler = negative_sampler
        # one lookup per event endpoint for the whole stream (sgl_window_end)
        end_src = graph.window_end(self.src, self.ts)
        end_dst = graph.window_end(self.dst, self.ts)
        # the inputs of every full batch, laid out once as rows: [sources; destinations] and their times and
        # window ends, and the negatives' times (the batch's event times, repeated)
        nb, B, n_neg = int(self.src.numel()) // self.B, self.B, self.num_neg
        rows = lambda a, b_: torch.cat([a[: nb * B].view(nb, B), b_[: nb * B].view(nb, B)], dim=1).contiguous()
        self._roots, self._root_ts, self._hint = rows(self.src, self.dst), rows(self.ts, self.ts), rows(end_src, end_dst)
        t_rows = self.ts[: nb * B].view(nb, B)
        self._neg_ts = t_rows.repeat(1, (n_neg + B - 1) // B)[:, :n_neg].contiguous() if n_neg else t_rows[:, :0]
        self._neg_block, self._neg_at = None, 0
        self.sample_ahead = max(1, int(sample_ahead))
        if self.sample_ahead > 1:
            self.pool = MiniBatchGroupPool(max(1, int(prefetch)), graph, self.sample_ahead, 2 * self.B, self.num_neg, layers,
                                           fanout, sample_type, node_tables=node_tables, edge_tables=edge_tables,
                                           time_encoder=time_encoder, root_hints=True, **pipeline_kwargs)
        else:
            self.pool = MiniBatchPipelinePool(max(1, int(prefetch)), graph, 2 * self.B, self.num_neg, layers, fanout,
                                              sample_type, node_tables=node_tables, edge_tables=edge_tables,
                                              time_encoder=time_encoder, root_hints=True, **pipeline_kwargs)

    def __len__(self):
        return int(self.src.numel()) // self.B

    NEG_BLOCK = 64      # negatives are drawn for this many batches at a time (one launch instead of 64)

    def _negatives(self):
        n = self.num_neg
        if n == 0:
            return self.src.new_empty(0)
        if self._neg_block is None or self._neg_at == self.NEG_BLOCK:
            if self.negative_sampler is not None:
                blk = self.negative_sampler.sample(self.NEG_BLOCK * n, 1).reshape(self.NEG_BLOCK, n)
            else:
                blk = torch.randint(0, self.graph._n, (self.NEG_BLOCK, n), device=self.src.device)
            self._neg_block, self._neg_at = blk.to(self.src.device), 0
        self._neg_at += 1
        return self._neg_block[self._neg_at - 1]

    def _submit(self, i):
        return self.pool.run(self._roots[i], self._root_ts[i], self._negatives(), self._neg_ts[i], root_hint=self._hint[i])

    def _submit_group(self, i0, live):
        neg = torch.stack([self._negatives() for _ in range(live)]) if self.num_neg else self._neg_ts[i0: i0 + live]
        return self.pool.run(self._roots[i0: i0 + live], self._root_ts[i0: i0 + live], neg, self._neg_ts[i0: i0 + live],
                             root_hint=self._hint[i0: i0 + live])

    def _iter_groups(self):
        depth, total, A = len(self.pool.pipes), len(self), self.sample_ahead
        ahead = max(1, depth - 1)
        queue, nxt = [], 0
        while nxt < total and len(queue) < ahead:
            live = min(A, total - nxt)
            queue.append(self._submit_group(nxt, live)); nxt += live
        while queue:
            for mb in queue.pop(0).finalize():
                yield mb
            if nxt < total:
                live = min(A, total - nxt)
                queue.append(self._submit_group(nxt, live)); nxt += live

    def __iter__(self):
        """Yields the finalized MiniBatch of every full batch, in order.  A MiniBatch is valid until
        `prefetch` further batches have been submitted, i.e. until the next one is yielded."""
        if self.sample_ahead > 1:
            yield from self._iter_groups()
            return
        depth, total = len(self.pool.pipes), len(self)
        # a yielded batch's pipeline is reused by the submission that follows `depth - 1` yields later, so one
        # pipeline is always kept free for the batch the consumer is looking at
        ahead = max(1, depth - 1)
        queue, nxt = [], 0
        while nxt < total and len(queue) < ahead:
            queue.append(self._submit(nxt)); nxt += 1
        while queue:
            mb = queue.pop(0).finalize()
            yield mb
            if nxt < total:
                queue.append(self._submit(nxt)); nxt += 1
