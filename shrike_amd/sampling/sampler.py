"""Choosing next tokens from the logits of a step: greedy, temperature, top-p,
mixed per row, on the device.

Reference: shrike/engine/sampler.py:10-31.  Rows with temperature 0 take the
argmax of the raw logits (lowest index among equal maxima); other rows draw
from softmax(logits / T) restricted to the top-p nucleus.  The reference draws
with torch's global generator; here every draw is a pure function of
(seed, number of the draw), so a generation can be repeated whatever else ran.
"""

from __future__ import annotations

import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed: int, draw: int) -> float:
    """The draw-th number in [0, 1) of the stream `seed` (24 bits, exact in float32)."""
    return (splitmix64(splitmix64(seed & _MASK) ^ (draw & _MASK)) >> 40) / float(1 << 24)


class ChosenTokens:
    """The tokens of a step, on the device (`device`, int32) and on their way to
    the host: the copy into page-locked memory is queued right behind the
    kernel that chose them, ahead of whatever is launched next, and tolist()
    waits for that copy alone."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, copied: torch.cuda.Event):
        self.device, self._host, self._copied = device, host, copied

    def tolist(self) -> list[int]:
        self._copied.synchronize()
        return self._host.tolist()


class Sampler:
    def __init__(self, device, engine_seed: int = 0):
        self.device = device
        self.engine_seed = engine_seed
        self._scratch = None
        self._staging = None  # two page-locked buffers for the rows' parameters, used by turns
        self._params = None

    def request_seed(self, req) -> int:
        if req.sampling.seed is not None:
            return req.sampling.seed
        return splitmix64((self.engine_seed << 20) ^ req.req_id)

    def launch(self, logits: torch.Tensor, reqs: list) -> ChosenTokens | None:
        """Starts the choice of one token per row of logits (float32 [R, vocab]
        on the device, one row per request) and their copy to the host; returns
        the handle that holds them.  Nothing here waits for the device."""
        if not reqs:
            return None
        rows = logits.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        self._choose(logits, out, reqs)
        host = torch.empty(rows, dtype=torch.int32, pin_memory=True)
        ops.copy_words(out, host)
        copied = torch.cuda.Event()
        copied.record()
        return ChosenTokens(out, host, copied)

    def _choose(self, logits: torch.Tensor, out: torch.Tensor, reqs: list) -> None:
        rows, vocab = logits.shape
        if all(r.sampling.temperature == 0.0 for r in reqs):
            ops.argmax(logits, out)
            return
        params = self._upload(
            [[r.sampling.temperature for r in reqs],
             [r.sampling.top_p for r in reqs],
             [uniform(self.request_seed(r), r.num_generated) for r in reqs]],
            logits.device,
        )
        need = ops.sample_scratch_floats(rows, vocab)
        if self._scratch is None or self._scratch.numel() < need:
            self._scratch = torch.empty(need, dtype=torch.float32, device=logits.device)
        nucleus = any(r.sampling.temperature > 0.0 and r.sampling.top_p < 1.0 for r in reqs)
        ops.sample(logits, out, params[0], params[1], params[2], self._scratch, nucleus=nucleus)

    def _upload(self, rows_of_floats: list, device) -> torch.Tensor:
        """float32 [3, R] on the device without a wait: through one of two page-locked
        buffers by turns and a copy kernel in stream order (a copy from ordinary memory
        would hold the host until the step before it has finished on the device)."""
        n = len(rows_of_floats[0])
        turn = self._turn = 1 - getattr(self, "_turn", 0)
        if self._staging is None or self._staging[0][0].shape[1] < n:
            if self._staging is not None:
                # A copy kernel that is still queued reads the old buffers when it runs, and
                # the host allocator may hand their memory to the next page-locked tensor
                # as soon as they are dropped: they go only after their last readers.
                for _, read in self._staging:
                    read.synchronize()
            width = max(64, 2 * n)
            self._staging = [(torch.empty(3, width, dtype=torch.float32, pin_memory=True), torch.cuda.Event())
                             for _ in range(2)]
            self._params = torch.empty(3, width, dtype=torch.float32, device=device)
        host, read = self._staging[turn]
        read.synchronize()  # the copy that last read this buffer has run
        host[:, :n] = torch.tensor(rows_of_floats, dtype=torch.float32)
        ops.copy_words(host.view(torch.int32), self._params.view(torch.int32))
        read.record()
        return self._params[:, :n]

    def sample(self, logits: torch.Tensor, reqs: list) -> list[int]:
        """The tokens themselves: launch(), then the wait for the device."""
        out = self.launch(logits, reqs)
        return [] if out is None else out.tolist()
