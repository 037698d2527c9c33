"""Host-side steering of the decay rule's backward call by what its forward call saw.

The matrix-core backward has two forms (include/t2fw_hip.h): the chunk-parallel kernels, which decline
rows whose gate products over half a chunk fall below 2^-80 and hand them to one more launch of the
block-wise kernel, and the block-wise kernel alone.  That extra launch costs a few microseconds even
when it finds nothing to do, and when most rows are declined the chunk-parallel launches were wasted.
The forward call already looks at every gate; it leaves one hint per batch row in its workspace
("the backward may decline this row").  Given a workspace in pinned host memory, the host can read the
hints as soon as the forward call has completed on the GPU, which in a training step is long before
the backward call is issued, and pick the backward's flags without any synchronisation:

  * no row hinted          -> T2FW_FLAG_NO_FIXUP (the extra launch is skipped; no row can be flagged)
  * enough rows hinted     -> T2FW_FLAG_BLOCKWISE (see ``choose_backward_flags``)
  * hints not there yet, or the stream is being captured into a graph -> the default call, which
    decides everything on the device.

The reference has a single path (t2fw/csrc/lfw.cpp:50-96); this module has no counterpart there.
"""
import ctypes
import threading

import numpy as np
import torch

from . import _lib

# Cost model behind the choice, microseconds per 1024 tokens of a row, measured on MI355X at
# B=96 / T=1024 and B=128 / T=8192: the chunk-parallel kernels take about 0.625 per row; the block-wise
# kernel walks a row as one chain of about 85 whatever the batch, 128 rows (two workgroups each) at a time.
PAR_US_PER_ROW = 0.625
BLOCKWISE_US_PER_ROUND = 85.0
BLOCKWISE_ROWS_PER_ROUND = 128


def _rounds(rows):
    return -(-rows // BLOCKWISE_ROWS_PER_ROUND)


def choose_backward_flags(flags, hinted_rows, rows):
    """Flags for the backward call, given the caller's ``flags``, the number of rows the forward call
    hinted (None: unknown) and the number of batch rows.  Pure function of its arguments."""
    if hinted_rows is None or rows <= 0:
        return flags
    if flags & (_lib.FLAG_FORCE_SCAN | _lib.FLAG_FP16_OPERANDS | _lib.FLAG_BLOCKWISE | _lib.FLAG_NO_FIXUP):
        return flags                                   # the caller chose a path
    if hinted_rows == 0:
        return flags | _lib.FLAG_NO_FIXUP
    chunk_parallel = PAR_US_PER_ROW * rows + BLOCKWISE_US_PER_ROUND * _rounds(hinted_rows)
    blockwise = BLOCKWISE_US_PER_ROUND * _rounds(rows)
    return flags | _lib.FLAG_BLOCKWISE if blockwise <= chunk_parallel else flags


def count_hinted_rows(hints, rows):
    """``hints``: int32 array of two slots per row, [2, rows rounded up to 8] flattened (a forward launch
    that splits a row over two workgroups reports per workgroup)."""
    h = np.asarray(hints).reshape(2, -1)[:, :rows]
    return int(np.count_nonzero(h[0] | h[1]))


class _Slot:
    """One pinned workspace: the tensor that owns it, the address the GPU sees it under, a view of its
    hint region and the event recorded after the last launch that writes it."""
    __slots__ = ("buf", "dptr", "view", "event")


class _PinnedPool:
    """Pinned host workspaces, handed out for one forward call each and taken back once the GPU work that
    writes them has completed.  Grows to the number of forward calls in flight."""

    def __init__(self):
        self.lock = threading.Lock()
        self.free = {}          # (device index, nbytes, hint offset, hint count) -> list of _Slot

    def acquire(self, key):
        with self.lock:
            lst = self.free.get(key)
            if lst:
                for i in range(len(lst)):
                    if lst[i].event.query():
                        return lst.pop(i)
        _, nbytes, hint_offset, hint_count = key
        slot = _Slot()
        slot.buf = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
        slot.dptr = ctypes.c_void_p()
        _lib.check(_lib.load().t2fw_host_workspace_device_pointer(ctypes.c_void_p(slot.buf.data_ptr()),
                                                                  ctypes.byref(slot.dptr)))
        slot.view = slot.buf.numpy()[hint_offset:hint_offset + 4 * hint_count].view(np.int32)
        slot.event = torch.cuda.Event()
        return slot

    def release(self, key, slot):
        with self.lock:
            self.free.setdefault(key, []).append(slot)


_POOL = _PinnedPool()


class ForwardHints:
    """The pinned workspace of one forward call and the event that says when its hints can be read."""

    def __init__(self, device, nbytes, hint_offset, hint_count, rows):
        self.device = device
        self.rows = rows
        self.nbytes = nbytes
        self.key = (device.index if device.index is not None else torch.cuda.current_device(), nbytes, hint_offset,
                    hint_count)
        self.slot = _POOL.acquire(self.key)
        self.launched_ = False
        self.count = None

    @staticmethod
    def usable(device):
        """Not while the stream is captured into a graph: a replay would read hints of the capture."""
        return not torch.cuda.is_current_stream_capturing()

    def workspace(self):
        return self.slot.dptr, self.nbytes

    def launched(self):
        """Call right after the forward launch, on the launch stream."""
        self.slot.event.record(torch.cuda.current_stream(self.device))
        self.launched_ = True

    def hinted_rows(self):
        """Rows hinted, or None while the forward call has not completed on the GPU.  The first answer is
        kept (a backward may be asked for twice) and the buffer goes back to the pool."""
        slot = self.slot
        if self.count is None and slot is not None and self.launched_ and slot.event.query():
            self.count = count_hinted_rows(slot.view, self.rows) if slot.view.any() else 0
            self.close()
        return self.count

    def close(self):
        slot, self.slot = self.slot, None
        if slot is not None:
            if not self.launched_:
                slot.event.record(torch.cuda.current_stream(self.device))     # nothing pending: reusable at once
            _POOL.release(self.key, slot)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
