"""Inference runner: the batch as sub-batches that run side by side, one captured HIP graph per sub-batch.

A forward of the backbone is about 190 kernels, many of them too small to fill 256 compute units (the 14x14 and 7x7
stages) and each with a tail of half-empty workgroups.  The samples of a batch are independent, so sub-batches can run
concurrently: every sub-batch forward is captured once into a graph of its own (a plain single-stream graph with its own
memory pool) and a step launches the graphs together -- the first on the caller's stream, the others each on a stream
of its own -- so their kernels overlap wherever one leaves compute units idle.  Results are those of the eager forward
of each sub-batch (``max_replay_error`` checks replays against them); default-priority streams only.

Which hardware queue a new stream lands on matters: the runtime deals its few hardware queues (four here) to streams in
turn, and a worker stream that shares its queue with the caller's stream queues up behind the joins the caller's stream
carries -- its next launch then waits for the other sub-batches (measured: 6.7-7.0 ms per step instead of 5.4).  The
mapping cannot be queried, so the runner times a few sets of freshly created streams and keeps the fastest.

What a graph bakes in, and how the runner keeps it valid:
  * library scratch.  PyTorch hands rocBLAS / hipBLASLt one workspace per (handle, stream); a GEMM captured on a stream
    records that workspace's address.  Every sub-batch is therefore warmed up and captured on a stream of its own, kept
    for the runner's lifetime and used for nothing else: graphs that replay side by side never share a workspace, and no
    eager work ever touches one.
  * per-module constants.  The SS2D blocks cache small tensors derived from their parameters; a capture pins the ones it
    reads (``SS2D._inference_constants``) so that cache eviction cannot free them under a live graph.
  * parameter values.  Those pinned constants are copies, and the graphs hold the addresses of the parameters' storage:
    after an in-place update, a ``.half()`` / ``.to()`` or a ``param.data = ...`` a replay would read stale copies or
    freed memory, so ``replay()`` compares storage address, dtype and version counter of every parameter and buffer
    with what they were at capture time and refuses on any difference.
"""
import time

import torch


class ConcurrentGraphRunner:
    """``runner = ConcurrentGraphRunner(model, x, sub_batches)``; ``runner.replay()`` runs one forward of the whole batch
    ``x`` (the captured tensor: refill it in place for new inputs) and ``runner.output()`` returns the concatenated
    result.  ``sub_batches`` must divide the batch."""

    def __init__(self, model, x, sub_batches, warmup=2, stream_sets=4):
        if not x.is_cuda:
            raise NotImplementedError("ConcurrentGraphRunner: vmamba_amd runs on the GPU only")
        if sub_batches < 1 or x.shape[0] % sub_batches != 0:
            raise ValueError(f"sub_batches = {sub_batches} must divide the batch of {x.shape[0]}")
        self.model, self.x = model, x
        self.chunks = x.chunk(sub_batches)
        self.graphs, self.outs = [], []
        dev = x.device
        cur = torch.cuda.current_stream(dev)
        self.capture_streams = [torch.cuda.Stream(device=dev) for _ in self.chunks]     # one per graph, never reused
        with torch.no_grad():
            for c, capture_stream in zip(self.chunks, self.capture_streams):
                capture_stream.wait_stream(cur)
                with torch.cuda.stream(capture_stream):
                    for _ in range(warmup):
                        model(c)
                cur.wait_stream(capture_stream)
                torch.cuda.synchronize(dev)
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=capture_stream):
                    out = model(c)
                self.graphs.append(g)
                self.outs.append(out)
        torch.cuda.synchronize(dev)
        self._tensors = list(model.parameters()) + list(model.buffers())
        self._signature = self._tensor_signature()
        self.streams = self._pick_streams(sub_batches - 1, stream_sets)
        self.step_ms = self._time_step(self.streams) if sub_batches > 1 else None

    def _new_streams(self, n):
        return [torch.cuda.Stream(device=self.x.device) for _ in range(n)]

    def _replay_on(self, streams):
        cur = torch.cuda.current_stream(self.x.device)
        for s, g in zip(streams, self.graphs[1:]):
            s.wait_stream(cur)
            with torch.cuda.stream(s):
                g.replay()
        self.graphs[0].replay()
        for s in streams:
            cur.wait_stream(s)

    def _time_step(self, streams, steps=6, warm=3):
        dev = self.x.device
        for _ in range(warm):
            self._replay_on(streams)
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for _ in range(steps):
            self._replay_on(streams)
        torch.cuda.synchronize(dev)
        return (time.perf_counter() - t0) / steps * 1e3

    def _pick_streams(self, n, sets):
        """The fastest of ``sets`` sets of n new streams.  Every set (and one spare stream where n is even) stays alive
        until the choice is made, so that each set starts on the next hardware queue."""
        if n == 0:
            return []
        tried, best = [], None
        for _ in range(max(1, sets)):
            streams = self._new_streams(n)
            tried.append(streams)
            if n % 2 == 0:
                tried.append(self._new_streams(1))
            ms = self._time_step(streams)
            if best is None or ms < best[0]:
                best = (ms, streams)
        return best[1]

    def _tensor_signature(self):
        # storage address, dtype and version counter of every parameter and buffer: an in-place update bumps the
        # version; model.half() / .to() / `param.data = ...` keep it but move or retype the storage
        return [(t.data_ptr(), t.dtype, t._version) for t in self._tensors]

    def parameters_unchanged(self):
        """False once any parameter or buffer of the model was updated in place, moved or retyped after the capture (the
        graphs hold the old storage's addresses and copies derived from the old values)."""
        return self._tensor_signature() == self._signature

    def replay(self):
        if not self.parameters_unchanged():
            raise RuntimeError("ConcurrentGraphRunner: a parameter of the model changed after the graphs were captured; "
                               "they hold copies derived from the old values -- build a new runner")
        self._replay_on(self.streams)

    def output(self):
        return torch.cat(self.outs)

    def max_replay_error(self, replays=3):
        """Largest absolute difference between the eager sub-batch forwards and each of ``replays`` concurrent replays
        (interleaved with eager work and synchronisations).  0.0 = bit for bit.  Library kernels that accumulate with
        atomics (some small-batch convolutions and split GEMMs) differ from run to run in the last place, eager or
        not; anything larger means a graph node whose result depends on what runs beside it."""
        dev = self.x.device
        worst = 0.0
        with torch.no_grad():
            eager = torch.cat([self.model(c) for c in self.chunks]).float()
            torch.cuda.synchronize(dev)
            for _ in range(replays):
                self.replay()
                torch.cuda.synchronize(dev)
                err = (self.output().float() - eager).abs().max().item()
                worst = max(worst, err) if err == err else float("inf")
                self.model(self.chunks[0])            # eager work between replays
                torch.cuda.synchronize(dev)
        return worst

    def validate(self, replays=3, atol=0.0):
        """True when every replay reproduces the eager result to within ``atol`` (0.0: bit for bit)."""
        return self.max_replay_error(replays) <= atol
