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

from .pipeline import MiniBatchPipelinePool


class EventBatchLoader:
    def __init__(self, graph, src, dst, ts, batch_size, num_neg, layers, fanout, sample_type="recent",
                 node_tables=None, edge_tables=None, time_encoder=None, prefetch=3, negative_sampler=None,
                 drop_last=True, **pipeline_kwargs):
        """graph: `pyGraph.g` / `CUDAGraph`.  src/dst/ts: the events in training order (int64, any device).
        num_neg: negatives per batch (their times repeat the batch's event times).  negative_sampler: an
        object with `sample(num_samples, num_groups)` (NegSamplingSet); default: uniform over all nodes.
        prefetch: batches in flight (pipelines of the pool).  Remaining keywords go to MiniBatchPipeline.
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
        self.end_src = graph.window_end(self.src, self.ts)
        self.end_dst = graph.window_end(self.dst, self.ts)
        self.pool = MiniBatchPipelinePool(max(1, int(prefetch)), graph, 2 * self.B, self.num_neg, layers, fanout,
                                          sample_type, node_tables=node_tables, edge_tables=edge_tables,
                                          time_encoder=time_encoder, root_hints=True, **pipeline_kwargs)

    def __len__(self):
        return int(self.src.numel()) // self.B

    def _negatives(self, lo):
        n = self.num_neg
        if n == 0:
            e = self.src.new_empty(0)
            return e, e
        if self.negative_sampler is not None:
            neg = self.negative_sampler.sample(n, 1).reshape(-1).to(self.src.device)
        else:
            neg = torch.randint(0, self.graph._n, (n,), device=self.src.device)
        t = self.ts[lo: lo + self.B]
        return neg, t.repeat((n + self.B - 1) // self.B)[:n].contiguous()

    def _submit(self, i):
        lo, hi = i * self.B, (i + 1) * self.B
        roots = torch.cat([self.src[lo:hi], self.dst[lo:hi]])
        root_ts = torch.cat([self.ts[lo:hi], self.ts[lo:hi]])
        hint = torch.cat([self.end_src[lo:hi], self.end_dst[lo:hi]])
        neg, neg_ts = self._negatives(lo)
        return self.pool.run(roots, root_ts, neg, neg_ts, root_hint=hint)

    def __iter__(self):
        """Yields the finalized MiniBatch of every full batch, in order.  A MiniBatch is valid until
        `prefetch` further batches have been submitted, i.e. until the next one is yielded."""
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
