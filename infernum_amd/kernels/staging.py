"""Small host arrays on their way to the device, and a step's chosen tokens on their way back, without the host
waiting for the GPU and without the DMA engines.

A copy from ordinary (pageable) host memory is carried out in the stream's order and the host waits for it, so
a step's int32 arrays would hold the host until everything queued before them has run.  A queued copy from
pinned memory does not, but it runs on a DMA engine, and the signals between that queue and the compute queue
cost a step of single tokens a tenth of a millisecond.  Here the arrays are laid into pinned memory and a small
kernel of the compute stream reads them from there (``kernels.api.words_from_host``); the tokens go back the same
way (``words_to_host``) with an event behind them.  ``PinnedUpload`` keeps a few pinned buffers in turn; a
buffer is written again only after the kernel that read it last has run.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from . import api as K


class PinnedUpload:
    def __init__(self, device: torch.device, buffers: int = 4):
        self.device = device
        self._bufs: List[Optional[torch.Tensor]] = [None] * buffers
        self._events: List[Optional["torch.cuda.Event"]] = [None] * buffers
        self._next = 0

    def upload(self, host: np.ndarray, out: Optional[torch.Tensor] = None, token_off: int = 0,
               token_rows: Optional[np.ndarray] = None, source: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``host``: a contiguous numpy array of 4-byte elements.  Returns the device tensor that will hold it
        (``out`` when given, of the array's dtype and at least its size), in the current stream's order.
        ``token_rows`` (int32, one per row) and ``source`` (int32 tokens on the device): the elements
        token_off + r of the result whose token_rows[r] is j >= 0 are source[j] instead."""
        src = torch.from_numpy(host).reshape(-1)
        if src.element_size() != 4:
            raise K.KernelError("PinnedUpload: arrays of 4-byte elements only")
        n = src.numel()
        nd = 0 if token_rows is None else int(token_rows.shape[0])
        i = self._next
        self._next = (i + 1) % len(self._bufs)
        if self._events[i] is not None:
            self._events[i].synchronize()
        buf = self._bufs[i]
        if buf is None or buf.numel() < n + nd:
            buf = self._bufs[i] = torch.empty(max(n + nd, 1 << 14), dtype=torch.int32, pin_memory=True)
        buf[:n].view(src.dtype).copy_(src)
        if nd:
            buf[n:n + nd].copy_(torch.from_numpy(token_rows))
        if out is None:
            out = torch.empty(host.shape, dtype=src.dtype, device=self.device)
        K.words_from_host(out.view(-1), buf, n, token_off, nd, source, n)
        ev = self._events[i] = torch.cuda.Event()
        ev.record()
        return out


class TokenDownload:
    """``start(tokens)`` queues a kernel that writes an int32 device tensor into pinned host memory, and an event
    behind it; ``wait(handle)`` gives the list once it is there."""

    def __init__(self, device: torch.device, buffers: int = 4):
        self.device = device
        self._bufs: List[Optional[torch.Tensor]] = [None] * buffers
        self._next = 0

    def start(self, tokens: torch.Tensor):
        n = tokens.numel()
        i = self._next
        self._next = (i + 1) % len(self._bufs)
        buf = self._bufs[i]
        if buf is None or buf.numel() < n:
            buf = self._bufs[i] = torch.empty(max(n, 1024), dtype=torch.int32, pin_memory=True)
        if n:
            K.words_to_host(buf, tokens)
        done = torch.cuda.Event()
        done.record()
        return buf, done, n

    @staticmethod
    def wait(handle) -> List[int]:
        buf, done, n = handle
        done.synchronize()
        return buf[:n].tolist()
