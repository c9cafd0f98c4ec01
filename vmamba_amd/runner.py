"""Inference runner: the batch as sub-batches on separate HIP streams, one captured HIP graph per sub-batch.

A forward of the backbone is about 190 kernels, many of them too small to fill 256 compute units (the 14x14 and 7x7
stages) and each with a tail of half-empty workgroups.  The samples of a batch are independent, so sub-batches can run
side by side: every sub-batch forward is captured once into a graph of its own (a plain single-stream graph, on its own
stream, with its own memory pool) and a step launches the graphs together, each on its stream; their kernels overlap
wherever one leaves compute units idle.  Results are those of the eager forward of each sub-batch (``validate`` checks
replays against them); default-priority streams only.
"""
import torch


class ConcurrentGraphRunner:
    """``runner = ConcurrentGraphRunner(model, x, sub_batches)``; ``runner.replay()`` runs one forward of the whole batch
    ``x`` (the captured tensor: refill it in place for new inputs) and ``runner.output()`` returns the concatenated
    result.  ``sub_batches`` must divide the batch (equal sub-batches share the model's per-batch-size constants)."""

    def __init__(self, model, x, sub_batches, warmup=2):
        if not x.is_cuda:
            raise NotImplementedError("ConcurrentGraphRunner: vmamba_amd runs on the GPU only")
        if sub_batches < 1 or x.shape[0] % sub_batches != 0:
            raise ValueError(f"sub_batches = {sub_batches} must divide the batch of {x.shape[0]}")
        self.model, self.x = model, x
        self.chunks = x.chunk(sub_batches)
        self.streams = [torch.cuda.Stream(device=x.device) for _ in range(sub_batches)]
        self.graphs, self.outs = [], []
        cur = torch.cuda.current_stream(x.device)
        with torch.no_grad():
            for s, c in zip(self.streams, self.chunks):
                s.wait_stream(cur)
                with torch.cuda.stream(s):
                    for _ in range(warmup):
                        model(c)
                cur.wait_stream(s)
                torch.cuda.synchronize(x.device)
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=s):
                    out = model(c)
                self.graphs.append(g)
                self.outs.append(out)
        torch.cuda.synchronize(x.device)

    def replay(self):
        cur = torch.cuda.current_stream(self.x.device)
        for s, g in zip(self.streams, self.graphs):
            s.wait_stream(cur)
            with torch.cuda.stream(s):
                g.replay()
        for s in self.streams:
            cur.wait_stream(s)

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
