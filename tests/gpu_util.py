"""Device-memory plumbing for the GPU tests: torch owns the allocations, the
library under test only sees raw addresses."""
import numpy as np
import torch

import horovod_amd
from horovod_amd import host as H


class Arena:
    """One device allocation (and its host mirror) carved into tensors at chosen
    alignments, so that a test uploads and downloads everything in one copy."""

    def __init__(self, capacity, fill=0):
        self.host = np.full(capacity, fill, np.uint8)
        self.dev = None
        self.cursor = 0
        self.capacity = capacity

    def alloc(self, nbytes, misalign=0, align=256):
        start = (self.cursor + align - 1) // align * align + misalign
        if start + nbytes > self.capacity:
            raise MemoryError("arena too small")
        self.cursor = start + nbytes
        return start

    def upload(self):
        self.dev = torch.from_numpy(self.host).cuda()
        torch.cuda.synchronize()
        assert self.dev.data_ptr() % 256 == 0
        return self.dev.data_ptr()

    def download(self):
        torch.cuda.synchronize()
        return self.dev.cpu().numpy()

    def ptr(self, off):
        return self.dev.data_ptr() + off


class Gpu:
    def __init__(self):
        self.lib = horovod_amd.lib()
        self.stream = horovod_amd.Stream()
        self.H = H

    def upload(self, arr):
        t = torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1)).cuda()
        torch.cuda.synchronize()
        return t

    def empty(self, nbytes, fill=None):
        t = torch.empty(max(nbytes, 1), dtype=torch.uint8, device="cuda")
        if fill is not None:
            t.fill_(fill)
        torch.cuda.synchronize()
        return t

    def download(self, t, dtype=np.uint8):
        self.stream.synchronize()
        torch.cuda.synchronize()
        return t.cpu().numpy().view(dtype)

    def sync(self):
        self.stream.synchronize()
