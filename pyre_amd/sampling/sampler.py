"""Next tokens from logits on the device: argmax, or inverse-CDF sampling."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops


class Sampler:
    """One call per step: all rows at once, one small upload, one small download."""

    def __init__(self, device: torch.device, max_rows: int):
        self.device = device
        self.max_rows = max_rows
        self._host = torch.empty(2 * max_rows, dtype=torch.float32, pin_memory=True)
        self._dev = torch.empty(2 * max_rows, dtype=torch.float32, device=device)
        self._ids = torch.empty(max_rows, dtype=torch.int32, device=device)
        self._ids_host = torch.empty(max_rows, dtype=torch.int32, pin_memory=True)
        self._scratch = torch.empty(max_rows * ops.ARGMAX_SCRATCH_PER_ROW, dtype=torch.int32, device=device)
        self._done = torch.cuda.Event()

    def launch(self, logits: torch.Tensor, temperatures: list[float], uniforms: list[float]) -> int:
        """Put the choice of one token per row of ``logits`` (float32 [M, V] on the
        device) on the stream, and the copy of the ids to the host behind it.
        Row i: argmax if temperatures[i] is 0, else the first token whose cumulative
        probability under softmax(logits / T) exceeds uniforms[i]. Returns M;
        :meth:`collect` waits for the ids. Until the next launch, :attr:`ids` holds
        them on the device."""
        m = logits.shape[0]
        if m > self.max_rows or len(temperatures) != m or len(uniforms) != m:
            raise ValueError("sampler: row counts do not fit")
        with torch.cuda.device(self.device):
            ids = self._ids[:m]
            ops.argmax(logits, ids, self._scratch)
            if any(t > 0 for t in temperatures):
                self._host[:m] = torch.tensor(temperatures, dtype=torch.float32)
                self._host[m:2 * m] = torch.tensor(uniforms, dtype=torch.float32)
                self._dev[:2 * m].copy_(self._host[:2 * m], non_blocking=True)
                ops.sample(logits, self._dev[:m], self._dev[m:2 * m], ids)
            self._ids_host[:m].copy_(ids, non_blocking=True)
            self._done.record()
        return m

    def collect(self, m: int) -> list[int]:
        """The ids of the last launch, once they are on the host. Work put on the
        stream after the launch is not waited for."""
        self._done.synchronize()
        return self._ids_host[:m].tolist()

    @property
    def ids(self) -> torch.Tensor:
        """int32 ids of the last launch, on the device."""
        return self._ids

    def sample(self, logits: torch.Tensor, temperatures: list[float], uniforms: list[float]) -> list[int]:
        return self.collect(self.launch(logits, temperatures, uniforms))
