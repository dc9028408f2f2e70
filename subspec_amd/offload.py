"""Layer streaming: target decoder layers kept in pinned host memory and copied into a small ring of
device slabs ahead of the compute stream.

Replaces the reference's hook-chain offloaders (``PrefetchOffloader``,
specdecodes/helpers/offloaders/prefetch_offloader_postspec.py:54-241; placement by
``LayerOffloadRecipe(keep_first_n_layers_on_gpu)``, recipes/offload/layer_offload.py:9-56) with an
explicit schedule:

* every offloaded layer is ONE contiguous pinned slab (all seven projections + norms), so a layer
  is one ``hipMemcpyAsync`` instead of seven hooked ``copy_`` calls;
* a ring of device slabs; a copy into a slab waits on an event recorded after the last kernel that
  read the slab (the write-after-read edge the reference leaves to timing), and a layer's compute
  waits on its copy event;
* the ring does not stop at the end of a forward: the next forward's first layers are prefetched
  while the cycle verifies and speculates;
* the copy stream runs at default priority.
"""
from __future__ import annotations

from typing import Optional, Callable, Dict, List, Sequence, Tuple

import torch

from . import _lib as L


class LayerSlabLayout:
    """Names, shapes and byte offsets of one layer's tensors inside a slab (256-byte aligned)."""

    def __init__(self, shapes: Dict[str, Tuple[int, ...]], dtype: torch.dtype):
        self.dtype = dtype
        self.entries: List[Tuple[str, Tuple[int, ...], int, int]] = []
        off = 0
        esize = torch.empty((), dtype=dtype).element_size()
        for name, shape in shapes.items():
            numel = 1
            for s in shape:
                numel *= int(s)
            self.entries.append((name, tuple(shape), off, numel))
            off += (numel * esize + 255) // 256 * 256
        self.nbytes = off
        self.esize = esize

    def views(self, slab: torch.Tensor) -> Dict[str, torch.Tensor]:
        """Typed views into a uint8 slab."""
        out = {}
        for name, shape, off, numel in self.entries:
            out[name] = slab[off:off + numel * self.esize].view(self.dtype).view(shape)
        return out


class LayerStreamer:
    """``n_slabs`` device slabs form a ring indexed by the running count of layer visits (not by the
    layer number), so the ring keeps turning across forwards: when a forward ends, the copies of the
    NEXT forward's first ``n_slabs - 1`` layers are already on their way and overlap whatever runs in
    between (verification, the draft's speculation)."""

    def __init__(self, layout: LayerSlabLayout, host_layers: Sequence[Dict[str, torch.Tensor]], device,
                 n_slabs: int = 4):
        self.layout = layout
        self.device = torch.device(device)
        self.n = len(host_layers)
        self.n_slabs = max(2, min(int(n_slabs), max(2, self.n)))
        # pinned host arena: one slab per offloaded layer (allocated pinned, never registered afterwards)
        self.host = torch.empty((self.n, layout.nbytes), dtype=torch.uint8, pin_memory=True)
        for i, tensors in enumerate(host_layers):
            views = layout.views(self.host[i])
            for name, t in tensors.items():
                views[name].copy_(t)
        self.slabs = [torch.empty(layout.nbytes, dtype=torch.uint8, device=self.device) for _ in range(self.n_slabs)]
        self.slab_views = [layout.views(s) for s in self.slabs]
        self.copy_stream = torch.cuda.Stream(device=self.device)          # default priority
        self.copied = [torch.cuda.Event() for _ in range(self.n_slabs)]
        self.released = [torch.cuda.Event() for _ in range(self.n_slabs)]
        self._released_valid = [False] * self.n_slabs
        self._visit = 0                 # visits computed so far (visit v = layer v % n, slab v % n_slabs)
        self._issued = 0                # visits whose copy has been issued
        self.bytes_streamed = 0
        # Called as idle_hook(copy_done_event) right before the compute stream has to wait for a slab whose copy is
        # still running: work queued by the hook runs in the gap (post-speculation of the draft, as the reference's
        # wait hook does, prefetch_offloader_postspec.py:193-232).
        self.idle_hook: Optional[Callable[[torch.cuda.Event], None]] = None

    def _issue_until(self, visit: int) -> None:
        """Issue the copies of all visits up to and including ``visit``."""
        while self._issued <= visit:
            v = self._issued
            slot, layer = v % self.n_slabs, v % self.n
            if self._released_valid[slot]:
                self.copy_stream.wait_event(self.released[slot])          # last reader of this slab is done
            code = L.lib().subspec_stream_copy_h2d(self.slabs[slot].data_ptr(), self.host[layer].data_ptr(),
                                                   self.layout.nbytes, self.copy_stream.cuda_stream)
            L.check(code, "subspec_stream_copy_h2d")
            self.copied[slot].record(self.copy_stream)
            self.bytes_streamed += self.layout.nbytes
            self._issued += 1

    def run(self, fn: Callable[[int, Dict[str, torch.Tensor]], None]) -> None:
        """Calls ``fn(i, weights_of_layer_i)`` for every offloaded layer in order on the current
        stream, with the copies of the following ``n_slabs - 1`` visits in flight while layer i computes."""
        compute = torch.cuda.current_stream(self.device)
        if self.n == 0:
            return
        assert self._visit % self.n == 0, "a previous forward stopped half way"
        for i in range(self.n):
            v = self._visit
            slot = v % self.n_slabs
            self._issue_until(v + self.n_slabs - 1)
            if self.idle_hook is not None and not self.copied[slot].query():
                self.idle_hook(self.copied[slot])
            compute.wait_event(self.copied[slot])
            fn(i, self.slab_views[slot])
            self.released[slot].record(compute)
            self._released_valid[slot] = True
            self._visit += 1
