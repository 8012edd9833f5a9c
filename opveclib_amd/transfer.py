"""
Host arrays to the GPU and back for ``evaluate`` on numpy inputs.

The reference's harness copies every host buffer to the device before the launches and every result back after them
with blocking ``cudaMemcpy`` calls on pageable memory (opveclib/testcudaop.cc:188-269, 330-380).  Pageable copies go
through a staging buffer inside the runtime, one thread, one chunk at a time.  Here large arrays travel through two
page-locked staging buffers owned by this module (allocated page-locked from the start, never registered afterwards):
a few host threads fill one buffer (numpy's copy releases the interpreter lock) while the DMA engine drains the other,
and the other way round for results.  Small arrays take PyTorch's own path.  All device work is enqueued on the
caller's current HIP stream; a transfer returns when its last host-side copy is done.
"""

import threading

import numpy as np

#: bytes per staging buffer (two of them per device, allocated on first use)
CHUNK_BYTES = 32 << 20
#: arrays smaller than this are handed to PyTorch directly
MIN_STAGED_BYTES = 8 << 20
#: host threads that copy between pageable memory and the staging buffers
COPY_THREADS = 4

_lock = threading.Lock()
_stagers = {}


class _Stager(object):
    """The two staging buffers of one device, their events and the copy threads."""

    def __init__(self, torch, device):
        from concurrent.futures import ThreadPoolExecutor
        self.buffers = [torch.empty(CHUNK_BYTES, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self.views = [b.numpy() for b in self.buffers]
        with torch.cuda.device(device):
            self.events = [torch.cuda.Event() for _ in range(2)]
        self.recorded = [False, False]
        self.pool = ThreadPoolExecutor(max_workers=COPY_THREADS)
        self.busy = threading.Lock()

    def wait(self, k):
        """Until the device has finished with staging buffer k."""
        if self.recorded[k]:
            self.events[k].synchronize()
            self.recorded[k] = False

    def copy(self, dst, src):
        """dst[:] = src for two one-dimensional byte arrays of equal length, split over the copy threads."""
        n = dst.shape[0]
        if n < (1 << 20) or COPY_THREADS < 2:
            np.copyto(dst, src)
            return
        step = -(-n // COPY_THREADS)
        step += -step % 4096
        jobs = [self.pool.submit(np.copyto, dst[o:o + step], src[o:o + step]) for o in range(0, n, step)]
        for job in jobs:
            job.result()


def _stager(torch, device):
    key = (device.type, device.index)
    with _lock:
        stager = _stagers.get(key)
        if stager is None:
            stager = _stagers[key] = _Stager(torch, device)
        return stager


def shutdown():
    """End the copy threads and drop the staging buffers (they are created again on the next large transfer)."""
    with _lock:
        stagers = list(_stagers.values())
        _stagers.clear()
    for stager in stagers:
        stager.pool.shutdown(wait=True)


def _torch_dtype(torch, dtype):
    return torch.from_numpy(np.empty(0, dtype=dtype)).dtype


def to_device(array, torch, device):
    """A contiguous device tensor with the contents of the numpy array ``array``."""
    array = np.ascontiguousarray(array)
    nbytes = array.nbytes
    if nbytes < MIN_STAGED_BYTES:
        return torch.from_numpy(array).to(device)
    stager = _stager(torch, device)
    src = array.reshape(-1).view(np.uint8)
    with torch.cuda.device(device):
        raw = torch.empty(nbytes, dtype=torch.uint8, device=device)
        stream = torch.cuda.current_stream(device)
        with stager.busy:
            for k, offset in enumerate(range(0, nbytes, CHUNK_BYTES)):
                n = min(CHUNK_BYTES, nbytes - offset)
                slot = k % 2
                stager.wait(slot)
                stager.copy(stager.views[slot][:n], src[offset:offset + n])
                raw[offset:offset + n].copy_(stager.buffers[slot][:n], non_blocking=True)
                stager.events[slot].record(stream)
                stager.recorded[slot] = True
    return raw.view(_torch_dtype(torch, array.dtype)).reshape(array.shape)


def to_host(tensor, torch):
    """A numpy array with the contents of the device tensor ``tensor`` (synchronises with the current stream)."""
    nbytes = tensor.numel() * tensor.element_size()
    if nbytes < MIN_STAGED_BYTES:
        return tensor.cpu().numpy()
    device = tensor.device
    stager = _stager(torch, device)
    shape = tuple(tensor.shape)
    raw = tensor.contiguous().reshape(-1).view(torch.uint8)
    out = np.empty(shape, dtype=torch.empty(0, dtype=tensor.dtype).numpy().dtype)
    dst = out.reshape(-1).view(np.uint8)
    chunks = [(offset, min(CHUNK_BYTES, nbytes - offset)) for offset in range(0, nbytes, CHUNK_BYTES)]
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device)
        with stager.busy:
            def request(k):
                offset, n = chunks[k]
                slot = k % 2
                stager.wait(slot)
                stager.buffers[slot][:n].copy_(raw[offset:offset + n], non_blocking=True)
                stager.events[slot].record(stream)
                stager.recorded[slot] = True

            request(0)
            for k, (offset, n) in enumerate(chunks):
                if k + 1 < len(chunks):
                    request(k + 1)          # the other buffer fills while this one is copied out
                slot = k % 2
                stager.wait(slot)
                stager.copy(dst[offset:offset + n], stager.views[slot][:n])
    return out
