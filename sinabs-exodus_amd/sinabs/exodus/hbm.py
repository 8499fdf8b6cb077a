"""Where tensors live in HBM: region-aware allocation for MI355X.

The 288 GiB of HBM3E of an MI355X behave as three regions of 96 GiB.  A kernel that streams from one
region into another moves its data 8-12 % faster than one that reads and writes inside one region:
a flat copy between 4 GiB buffers runs at 5.7-6.1 TB/s inside a region and at 6.3-6.5 TB/s across, and the
time-strided layer kernels go from 5.2-5.4 TB/s to 5.6-5.9 TB/s.  Reads alone and writes alone do not care
where they go; it is the mix of both in one region that costs.

A process cannot ask the driver for memory of a region, and the order in which the driver hands memory out
follows the regions only on a machine that has run nothing yet.  So the library sorts: it takes the free
device memory in chunks of 4 GiB, measures with timed copies which chunks disturb each other, maps chunks of
one kind behind each other into three address ranges and gives the rest back
(``exodus_hbm_regions_create``, csrc/exodus_hbm.hip).  ``HbmRegions`` hands out tensors from these ranges.

``empty(shape, region=k)`` allocates in range k; ``empty_like(x, away_from=[...])`` in a range that none of
the given tensors lies in.  Tensors of the ranges are recognised by their addresses; for a tensor from
elsewhere (the ordinary allocator) the range it copies to slowest is looked up once per storage with three
short timed copies.  After ``enable()`` the layer-layout wrappers (``_hip.layerLifForward`` and friends)
allocate their outputs this way; without it nothing changes.  The reference has no counterpart (its CUDA
extension allocates outputs with ``torch.empty_like``, reference cuda/bindings.cu:98,144,183).

Memory of a released tensor is handed out again at once, without regard to streams: a tensor from here is for
work on one stream, or has to outlive (``torch.cuda.synchronize``) what other streams do with it.
"""
from __future__ import annotations

import ctypes
import threading
import warnings
from typing import Dict, Iterable, List, Optional, Sequence

import torch

GIB = 2 ** 30
CHUNK = 4 * GIB                 # physical memory is sorted in pieces of this size: shorter copies tell less
ALIGN = 2 * 2 ** 20             # every tensor of a range starts on a 2 MiB boundary
PROBES = 15                     # EXODUS_HBM_PROBES of include/exodus_hip.h
SMALLEST_PLACED = 2 ** 20       # smaller requests are left to the ordinary allocator
PROBE_BYTES = GIB               # the slice of a foreign tensor that is timed against the ranges
SMALLEST_PROBE = 256 * 2 ** 20  # foreign tensors below this are not classified (too short to time, too small to matter)


class _Report(ctypes.Structure):
    """exodus_hbm_report of include/exodus_hip.h"""
    _fields_ = [("base", ctypes.c_void_p * 3), ("bytes", ctypes.c_uint64 * 3), ("chunk_bytes", ctypes.c_uint64),
                ("chunks_examined", ctypes.c_int32), ("kinds_found", ctypes.c_int32),
                ("chunks_ambiguous", ctypes.c_int32), ("chunks_of_region", ctypes.c_int32 * 3),
                ("threshold_GBs", ctypes.c_float), ("probe_same_kind_GBs", ctypes.c_float),
                ("probe_other_kind_GBs", ctypes.c_float), ("copy_inside_GBs", ctypes.c_float * 3),
                ("copy_across_GBs", ctypes.c_float * 6), ("probe_chunk", ctypes.c_int32 * PROBES),
                ("probe_kind", ctypes.c_int32 * PROBES), ("probe_pair_GBs", (ctypes.c_float * PROBES) * PROBES)]


class _Block:
    """What torch keeps alive for as long as a tensor of a range has storage; gives the bytes back after."""

    def __init__(self, owner: "HbmRegions", k: int, offset: int, nbytes: int, rounded: int):
        self.owner, self.k, self.offset, self.rounded = owner, k, offset, rounded
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "version": 2,
                                         "data": (owner.bases[k] + offset, False)}

    def __del__(self):
        try:
            self.owner._give_back(self.k, self.offset, self.rounded)
        except Exception:                                  # interpreter shutdown: nothing left to give back to
            pass


def _copy_rate(dst: torch.Tensor, src: torch.Tensor, reps: int = 5) -> float:
    """bytes moved per millisecond by dst.copy_(src), median of `reps` (events on the current stream)"""
    dst.copy_(src)
    dst.copy_(src)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record()
        dst.copy_(src)
        b.record()
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in ev)[reps // 2]
    return 2 * src.numel() * src.element_size() / ms


class HbmRegions:
    """Three ranges of device memory, each made of physical memory of one region of HBM.

    ``gib_per_region`` is what each range holds for good (until ``close()``); a request that a range cannot
    serve is passed to the ordinary allocator, which is harmless but loses the placement.  Creating the ranges
    takes nearly all free device memory for a second or two and gives back what it does not keep, so do it
    early, before the program's big allocations.  ``report`` holds what the sorting measured, ``verified``
    whether copies between the finished ranges beat copies inside them.
    Raises RuntimeError when the device's memory shows no three regions or too little of it is free.
    """

    def __init__(self, gib_per_region: float = 24.0, device: Optional[torch.device] = None):
        from . import _hip
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("HbmRegions needs a HIP device")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        if not 1 <= gib_per_region <= 80:
            raise ValueError("gib_per_region must be between 1 and 80 (rounded up to whole chunks of 4 GiB): a range "
                             "has to fit inside one region")
        self._lib = _hip.lib
        rep = _Report()
        with torch.cuda.device(self.device):
            torch.zeros(1, device=self.device)             # the device's context exists
            torch.cuda.empty_cache()                       # what torch has cached cannot be sorted
            torch.cuda.synchronize()
            rc = self._lib.exodus_hbm_regions_create(self.device.index, int(gib_per_region * GIB), CHUNK,
                                                     ctypes.byref(rep))
        self.report: Dict[str, object] = {
            "chunks_examined": rep.chunks_examined, "kinds_found": rep.kinds_found,
            "chunks_ambiguous": rep.chunks_ambiguous, "chunks_of_region": list(rep.chunks_of_region),
            "threshold_GBs": rep.threshold_GBs, "probe_chunks_same_region_GBs": rep.probe_same_kind_GBs,
            "probe_chunks_other_region_GBs": rep.probe_other_kind_GBs,
            "inside_one_range_GBs": list(rep.copy_inside_GBs), "across_ranges_GBs": list(rep.copy_across_GBs)}
        # the probe chunks: position, group, and the copy rate between every two (what the groups were read from)
        self.probes = {"chunk": list(rep.probe_chunk), "kind": list(rep.probe_kind),
                       "pair_GBs": [[rep.probe_pair_GBs[a][b] for b in range(PROBES)] for a in range(PROBES)]}
        if rc != 0:
            text = self._lib.exodus_hip_error_string(rc)
            raise RuntimeError(f"exodus_hbm_regions_create: {text.decode() if isinstance(text, bytes) else text} "
                               f"(status {rc}; measured: {self.report}; "
                               f"probe chunks {self.probes['chunk']} in groups {self.probes['kind']})")
        self.bases: List[int] = [int(rep.base[k]) for k in range(3)]
        self.sizes: List[int] = [int(rep.bytes[k]) for k in range(3)]
        self._free: List[List[List[int]]] = [[[0, n]] for n in self.sizes]   # per range: [offset, bytes], by offset
        self._lock = threading.Lock()
        self._live, self._closing, self._closed = 0, False, False
        self._foreign: Dict[int, int] = {}
        self._anchors: Optional[List[torch.Tensor]] = None
        inside = [r for r in rep.copy_inside_GBs if r > 0] or [rep.probe_same_kind_GBs]
        across = list(rep.copy_across_GBs)
        # single pairs of chunks scatter by a few percent around 6.0 (same region) and 6.35 TB/s (two regions);
        # the copies over whole ranges average over many pairs
        self.verified = bool(sum(across) / len(across) > 1.025 * sum(inside) / len(inside))
        if not self.verified:
            warnings.warn(f"HbmRegions: copies between the finished ranges are not clearly faster than copies "
                          f"inside them ({self.report}); allocation works, the gain may not be there")

    # ------------------------------------------------------------------ the ranges' free lists
    def _take(self, k: int, nbytes: int) -> Optional[int]:
        rounded = -(-nbytes // ALIGN) * ALIGN
        with self._lock:
            if self._closing:
                return None
            for slot, (off, n) in enumerate(self._free[k]):
                if n >= rounded:
                    if n == rounded:
                        del self._free[k][slot]
                    else:
                        self._free[k][slot] = [off + rounded, n - rounded]
                    self._live += 1
                    return off
        return None

    def _give_back(self, k: int, offset: int, rounded: int) -> None:
        with self._lock:
            free = self._free[k]
            slot = 0
            while slot < len(free) and free[slot][0] < offset:
                slot += 1
            free.insert(slot, [offset, rounded])
            if slot + 1 < len(free) and free[slot][0] + free[slot][1] == free[slot + 1][0]:
                free[slot][1] += free.pop(slot + 1)[1]
            if slot > 0 and free[slot - 1][0] + free[slot - 1][1] == free[slot][0]:
                free[slot - 1][1] += free.pop(slot)[1]
            self._live -= 1
            last = self._closing and self._live == 0
        if last:
            self._destroy()

    def _destroy(self) -> None:
        if not self._closed:
            self._closed = True
            self._lib.exodus_hbm_regions_destroy(self.device.index)     # waits for the device first

    def bytes_free(self, k: int) -> int:
        with self._lock:
            return sum(n for _, n in self._free[k])

    # ------------------------------------------------------------------ queries
    def pool_of(self, t: torch.Tensor) -> Optional[int]:
        """Index of the range whose memory holds ``t``, or None."""
        p = t.data_ptr()
        for k in range(3):
            if self.bases[k] <= p < self.bases[k] + self.sizes[k]:
                return k
        return None

    def region_of(self, t: torch.Tensor) -> Optional[int]:
        """The range (0, 1, 2) made of the same kind of memory as ``t``: by address for tensors of the ranges,
        by three timed copies (once per storage) for others; None for tensors too small to tell or to matter."""
        k = self.pool_of(t)
        if k is not None:
            return k
        nbytes = t.numel() * t.element_size()
        if nbytes < SMALLEST_PROBE or not t.is_contiguous() or t.device != self.device:
            return None
        key = t.untyped_storage().data_ptr()
        if key not in self._foreign:
            if torch.cuda.is_current_stream_capturing():
                return None                                # timing needs to wait for the device
            with torch.cuda.device(self.device), torch.no_grad():
                if self._anchors is None:
                    n = min(PROBE_BYTES, min(self.sizes) // 4)
                    self._anchors = [self.empty((n,), torch.uint8, region=j) for j in range(3)]
                n = min(self._anchors[0].numel(), nbytes)
                src = t.detach().reshape(-1).view(torch.uint8)[:n]
                rates = [_copy_rate(a[:n], src) for a in self._anchors]
            self._foreign[key] = min(range(3), key=lambda j: rates[j])   # slowest copy = same kind of memory
            if len(self._foreign) > 4096:
                self._foreign.pop(next(iter(self._foreign)))
        return self._foreign[key]

    def _pick(self, away_from: Iterable[Optional[torch.Tensor]]) -> int:
        taken = [0, 0, 0]
        for t in away_from:
            if isinstance(t, torch.Tensor) and t.is_cuda and t.numel():
                k = self.region_of(t)
                if k is not None:
                    taken[k] += t.numel() * t.element_size()
        return min(range(3), key=lambda k: (taken[k], k))

    # ------------------------------------------------------------------ allocation
    def empty(self, shape: Sequence[int], dtype=torch.float32, region: Optional[int] = None,
              away_from: Iterable[Optional[torch.Tensor]] = ()) -> torch.Tensor:
        """An uninitialised tensor in range ``region``, or in the range that holds none (or the least) of
        ``away_from``; from the ordinary allocator if it is tiny or the range is full."""
        shape = tuple(int(s) for s in shape)
        count = 1
        for s in shape:
            count *= s
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        if nbytes >= SMALLEST_PLACED:
            k = self._pick(away_from) if region is None else int(region)
            offset = self._take(k, nbytes)
            if offset is not None:
                block = _Block(self, k, offset, nbytes, -(-nbytes // ALIGN) * ALIGN)
                return torch.as_tensor(block, device=self.device).view(dtype).view(shape)
        return torch.empty(shape, dtype=dtype, device=self.device)

    def empty_like(self, like: torch.Tensor, away_from: Optional[Iterable[Optional[torch.Tensor]]] = None) -> torch.Tensor:
        return self.empty(like.shape, like.dtype, away_from=[like] if away_from is None else away_from)

    def close(self) -> None:
        """Give the ranges' memory back to the driver -- at once if no tensor lives in them, else when the last
        one is released; from now on requests are served by the ordinary allocator."""
        self._anchors = None
        with self._lock:
            self._closing = True
            last = self._live == 0
        if last:
            self._destroy()


_active: Optional[HbmRegions] = None


def enable(gib_per_region: float = 24.0, device: Optional[torch.device] = None) -> HbmRegions:
    """Create the ranges and make the layer-layout kernels' wrappers allocate their outputs through them."""
    global _active
    if _active is not None:
        disable()
    _active = HbmRegions(gib_per_region, device)
    return _active


def disable() -> None:
    """Undo ``enable()``.  Tensors that live in the ranges stay valid; the memory goes back with the last one."""
    global _active
    if _active is not None:
        _active.close()
    _active = None


def active() -> Optional[HbmRegions]:
    return _active


def empty_like(like: torch.Tensor, away_from: Optional[Iterable[Optional[torch.Tensor]]] = None) -> torch.Tensor:
    """``torch.empty_like(like)``, or -- after ``enable()`` -- a tensor of that shape in a region of HBM that
    none of ``away_from`` (default: ``like`` itself) lies in."""
    if _active is None or like.device != _active.device:
        return torch.empty_like(like)
    return _active.empty_like(like, away_from)


def empty(shape, like: torch.Tensor, away_from: Optional[Iterable[Optional[torch.Tensor]]] = None) -> torch.Tensor:
    """``torch.empty(shape)`` with dtype and device of ``like``, placed as ``empty_like`` places its result."""
    if _active is None or like.device != _active.device:
        return torch.empty(tuple(shape), dtype=like.dtype, device=like.device)
    return _active.empty(shape, like.dtype, away_from=[like] if away_from is None else away_from)
