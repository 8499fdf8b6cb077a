"""Where tensors live in HBM: region-aware allocation for MI355X.

The 288 GiB of HBM3E of an MI355X behave as three regions of 96 GiB, and what a kernel *writes* is held back by
the region it goes to.  Into a tensor that lies in one region the time-strided layer kernels write at 5.5-5.7 TB/s
and the (rows, time) kernels (single 128-byte lines) at 4.4-4.9 TB/s; into a tensor whose memory alternates between
the regions every 64 MiB the same kernels reach 6.0-6.3 and 5.6-5.8 TB/s.  Where the data they *read* lies matters
less: inputs in one region and outputs striped over the others is the best case, everything striped is 3-4 % behind
it, outputs in a single region 9-25 % (reads alone and writes alone in flat copies do not care).

A process cannot ask the driver for memory of a region, and the order in which the driver hands memory out
follows the regions only on a machine that has run nothing yet.  So the library sorts: it takes the free
device memory in pages of 64 MiB, judges every 4 GiB of consecutively created pages with timed copies (which chunks
disturb each other), and maps pages into four address ranges: one per region, and a *striped* one whose consecutive
pages come from regions 0, 1, 2, 0, 1, 2, ... (``exodus_hbm_regions_create``, csrc/exodus_hbm.hip).  The rest goes
back to the driver.  ``HbmRegions`` hands out tensors from these ranges.

``empty(shape)`` allocates in the striped range, ``empty(shape, region=k)`` in the range of region k (0, 1, 2).
After ``enable()`` the kernels' wrappers (``_hip.layerLifForward`` and friends, the (rows, time) wrappers, the
``IntegrateAndFire`` Function) allocate their big outputs through ``empty_like`` / ``empty`` of this module -- striped when there is a striped range; with region ranges only, in a
range that none of the tensors the kernel reads lies in (tensors of the ranges are recognised by their addresses;
for a tensor from the ordinary allocator the range it copies to slowest is looked up once per storage with three
short timed copies).  Without ``enable()`` nothing changes.  The reference has no counterpart (its CUDA
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
FINER_CHUNK = 256 * 2 ** 20     # ... and in pieces of this size when the big ones show no regions (memory that earlier
                                # processes left mixed below 4 GiB is mostly still in order at this scale)
REGIONS_NOT_FOUND = -3          # EXODUS_ERROR_REGIONS_NOT_FOUND of include/exodus_hip.h
ALIGN = 2 * 2 ** 20             # every tensor of a range starts on a 2 MiB boundary
PROBES = 15                     # EXODUS_HBM_PROBES of include/exodus_hip.h
ARENAS = 4                      # EXODUS_HBM_ARENAS: one range per region and the striped one
STRIPED = 3                     # index of the striped range
SMALLEST_PLACED = 2 ** 20       # smaller requests are left to the ordinary allocator
PROBE_BYTES = GIB               # the slice of a foreign tensor that is timed against the ranges
SMALLEST_PROBE = 256 * 2 ** 20  # foreign tensors below this are not classified (too short to time, too small to matter)


class _Report(ctypes.Structure):
    """exodus_hbm_report of include/exodus_hip.h"""
    _fields_ = [("base", ctypes.c_void_p * ARENAS), ("bytes", ctypes.c_uint64 * ARENAS),
                ("chunk_bytes", ctypes.c_uint64), ("page_bytes", ctypes.c_uint64),
                ("chunks_examined", ctypes.c_int32), ("kinds_found", ctypes.c_int32),
                ("chunks_ambiguous", ctypes.c_int32), ("chunks_of_region", ctypes.c_int32 * 3),
                ("threshold_GBs", ctypes.c_float), ("probe_same_kind_GBs", ctypes.c_float),
                ("probe_other_kind_GBs", ctypes.c_float), ("copy_inside_GBs", ctypes.c_float * 3),
                ("copy_across_GBs", ctypes.c_float * 6), ("copy_striped_GBs", ctypes.c_float),
                ("probe_chunk", ctypes.c_int32 * PROBES),
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


def _create(lib, device_index: int, bytes_per_region: int, bytes_striped: int, chunk_sizes: Sequence[int], sort: bool):
    """``exodus_hbm_regions_create`` with each of ``chunk_sizes`` in turn until one shows the regions (or none is
    left); returns (status, report, chunk size used).  A striped range that came out unsorted is given back before
    the next try."""
    for attempt, size in enumerate(chunk_sizes):
        rep = _Report()
        rc = lib.exodus_hbm_regions_create(device_index, bytes_per_region, bytes_striped, int(size), int(sort),
                                           ctypes.byref(rep))
        no_regions = rc == REGIONS_NOT_FOUND or (rc == 0 and sort and rep.kinds_found != 3)
        if not no_regions or attempt + 1 == len(chunk_sizes):
            break
        if rc == 0:
            lib.exodus_hbm_regions_destroy(device_index)
    return rc, rep, int(size)


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
    """Address ranges of device memory sorted by region of HBM: one per region (``gib_per_region`` each, may be 0)
    and a striped one (``gib_striped``, may be 0) whose 64 MiB pages alternate between the regions.

    The sizes are what the ranges hold for good (until ``close()``); a request that a range cannot
    serve is passed to the ordinary allocator, which is harmless but loses the placement.  Creating the ranges
    takes nearly all free device memory for a second or two and gives back what it does not keep, so do it
    early, before the program's big allocations.  ``chunk_bytes`` is the amount of memory judged as one piece
    (4 GiB; smaller pieces copy too quickly to tell the regions apart as reliably); when pieces of that size show no
    regions -- memory that earlier processes left mixed -- the sorting is repeated once with ``finer_chunk_bytes``.  ``report`` holds what the sorting
    measured; ``sort=False`` skips the timed copies and makes the striped range from chunks spread evenly over the
    free memory (what is done anyway when the memory shows no regions); ``verified`` says
    whether copies between regions beat copies inside them on the finished ranges (on the probe chunks when there
    are no region ranges).
    Raises RuntimeError when too little memory is free, or when ranges of single regions are asked for and the
    device's memory shows no three regions (a striped range alone is then still made, ``sorted`` False).
    """

    def __init__(self, gib_per_region: float = 0.0, gib_striped: float = 48.0,
                 device: Optional[torch.device] = None, chunk_bytes: int = CHUNK, sort: bool = True,
                 finer_chunk_bytes: Optional[int] = FINER_CHUNK):
        from . import _hip
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("HbmRegions needs a HIP device")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        if gib_per_region < 0 or gib_striped < 0 or (gib_per_region == 0 and gib_striped == 0):
            raise ValueError("gib_per_region and gib_striped must not be negative, and one of them positive")
        if not sort and gib_per_region:
            raise ValueError("ranges of single regions (gib_per_region) need the sorting")
        if chunk_bytes <= 0 or chunk_bytes % (64 * 2 ** 20):
            raise ValueError("chunk_bytes must be a multiple of the 64 MiB page")
        if gib_per_region + gib_striped / 3 > 80:
            raise ValueError("gib_per_region + gib_striped / 3 must not exceed 80 (rounded up to whole chunks of "
                             "4 GiB): that much is taken from each region, and a region has 96 GiB")
        self._lib = _hip.lib
        sizes = [int(chunk_bytes)]
        if sort and finer_chunk_bytes and finer_chunk_bytes < chunk_bytes:
            sizes.append(int(finer_chunk_bytes))
        with torch.cuda.device(self.device):
            torch.zeros(1, device=self.device)             # the device's context exists
            torch.cuda.empty_cache()                       # what torch has cached cannot be sorted
            torch.cuda.synchronize()
            rc, rep, size = _create(self._lib, self.device.index, int(gib_per_region * GIB), int(gib_striped * GIB),
                                    sizes, bool(sort))
        self.chunk_bytes = size                            # the size the ranges were sorted in
        self.report: Dict[str, object] = {
            "chunks_examined": rep.chunks_examined, "kinds_found": rep.kinds_found,
            "chunks_ambiguous": rep.chunks_ambiguous, "chunks_of_region": list(rep.chunks_of_region),
            "threshold_GBs": rep.threshold_GBs, "probe_chunks_same_region_GBs": rep.probe_same_kind_GBs,
            "probe_chunks_other_region_GBs": rep.probe_other_kind_GBs,
            "inside_one_range_GBs": list(rep.copy_inside_GBs), "across_ranges_GBs": list(rep.copy_across_GBs),
            "inside_striped_range_GBs": rep.copy_striped_GBs}
        # the probe chunks: position, group, and the copy rate between every two (what the groups were read from)
        self.probes = {"chunk": list(rep.probe_chunk), "kind": list(rep.probe_kind),
                       "pair_GBs": [[rep.probe_pair_GBs[a][b] for b in range(PROBES)] for a in range(PROBES)]}
        if rc != 0:
            text = self._lib.exodus_hip_error_string(rc)
            raise RuntimeError(f"exodus_hbm_regions_create: {text.decode() if isinstance(text, bytes) else text} "
                               f"(status {rc}; measured: {self.report}; "
                               f"probe chunks {self.probes['chunk']} in groups {self.probes['kind']})")
        self.bases: List[int] = [int(rep.base[k] or 0) for k in range(ARENAS)]
        self.sizes: List[int] = [int(rep.bytes[k]) for k in range(ARENAS)]
        self.page_bytes = int(rep.page_bytes)
        # False: the copies showed no three regions (memory that came back from earlier processes as a mixture of
        # them); the striped range is then made of chunks spread over the memory, as they are
        self.sorted = rep.kinds_found == 3
        self._free: List[List[List[int]]] = [[[0, n]] for n in self.sizes]   # per range: [offset, bytes], by offset
        self._lock = threading.Lock()
        self._live, self._closing, self._closed = 0, False, False
        self._foreign: Dict[int, int] = {}
        self._anchors: Optional[List[torch.Tensor]] = None
        inside = [r for r in rep.copy_inside_GBs if r > 0] or [rep.probe_same_kind_GBs]
        across = [r for r in rep.copy_across_GBs if r > 0] or [rep.probe_other_kind_GBs]
        # single pairs of chunks scatter by a few percent around 6.0 (same region) and 6.35 TB/s (two regions);
        # the copies over whole ranges average over many pairs
        self.verified = bool(self.sorted and sum(across) / len(across) > 1.025 * sum(inside) / len(inside))
        if self.sorted and not self.verified:
            warnings.warn(f"HbmRegions: copies between the regions are not clearly faster than copies "
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
        """Index of the range whose memory holds ``t`` (0, 1, 2: a region's; 3: the striped one), or None."""
        p = t.data_ptr()
        for k in range(ARENAS):
            if self.sizes[k] and self.bases[k] <= p < self.bases[k] + self.sizes[k]:
                return k
        return None

    def region_of(self, t: torch.Tensor) -> Optional[int]:
        """The region (0, 1, 2) that holds ``t``: by address for tensors of the regions' ranges, by three timed
        copies (once per storage) for others; None for tensors of the striped range, tensors too small to tell or
        to matter, and when there are no region ranges to time against."""
        k = self.pool_of(t)
        if k is not None:
            return k if k < STRIPED else None
        nbytes = t.numel() * t.element_size()
        if nbytes < SMALLEST_PROBE or not t.is_contiguous() or t.device != self.device or not self.sizes[0]:
            return None
        key = t.untyped_storage().data_ptr()
        if key not in self._foreign:
            if torch.cuda.is_current_stream_capturing():
                return None                                # timing needs to wait for the device
            with torch.cuda.device(self.device), torch.no_grad():
                if self._anchors is None:
                    n = min(PROBE_BYTES, min(self.sizes[:3]) // 4)
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
        """An uninitialised tensor in range ``region`` (0, 1, 2: that region; ``STRIPED``); without ``region`` in
        the striped range, or -- when there is none -- in the region that holds none (or the least) of
        ``away_from``.  From the ordinary allocator if it is tiny or the range is full or absent."""
        shape = tuple(int(s) for s in shape)
        count = 1
        for s in shape:
            count *= s
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        if nbytes >= SMALLEST_PLACED:
            k = int(region) if region is not None else (STRIPED if self.sizes[STRIPED] else self._pick(away_from))
            offset = self._take(k, nbytes) if self.sizes[k] else None
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


def enable(gib_per_region: float = 0.0, gib_striped: float = 48.0,
           device: Optional[torch.device] = None, **how) -> HbmRegions:
    """Create the ranges (``HbmRegions(gib_per_region, gib_striped, device, **how)``) and make the kernels' wrappers
    allocate their outputs through them."""
    global _active
    if _active is not None:
        disable()
    _active = HbmRegions(gib_per_region, gib_striped, device, **how)
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
    """``torch.empty_like(like)``, or -- after ``enable()`` -- a tensor of that shape in the striped range, or
    (region ranges only) in a region of HBM that none of ``away_from`` (default: ``like`` itself) lies in."""
    if _active is None or like.device != _active.device:
        return torch.empty_like(like)
    return _active.empty_like(like, away_from)


def empty(shape, like: torch.Tensor, away_from: Optional[Iterable[Optional[torch.Tensor]]] = None) -> torch.Tensor:
    """``torch.empty(shape)`` with dtype and device of ``like``, placed as ``empty_like`` places its result."""
    if _active is None or like.device != _active.device:
        return torch.empty(tuple(shape), dtype=like.dtype, device=like.device)
    return _active.empty(shape, like.dtype, away_from=[like] if away_from is None else away_from)
