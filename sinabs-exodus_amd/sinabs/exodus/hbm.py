"""Where tensors live in HBM: region-aware allocation for MI355X.

The 288 GiB of HBM3E of an MI355X behave as three regions of 96 GiB, and what a kernel *writes* is held back by
the region it goes to.  Into a tensor that lies in one region the time-strided layer kernels write at 5.5-5.7 TB/s
and the (rows, time) kernels (single 128-byte lines) at 4.4-4.9 TB/s; into a tensor whose memory alternates between
the regions every 64 MiB the same kernels reach 6.0-6.3 and 5.6-5.8 TB/s.  Where the data they *read* lies matters
less: inputs in one region and outputs striped over the others is the best case, everything striped is 3-4 % behind
it, outputs in a single region 9-25 % (reads alone and writes alone in flat copies do not care).

A process cannot ask the driver for memory of a region, and the order in which the driver hands memory out
follows the regions only on a machine that has run nothing yet.  So the library takes the free device memory in
chunks, optionally judges them with timed copies (which chunks disturb each other), and maps 64 MiB pages into four
address ranges: one per region, and a *striped* one whose consecutive pages come from regions 0, 1, 2, 0, 1, 2, ...
(``exodus_hbm_regions_create``, csrc/exodus_hbm.hip).  The rest goes back to the driver.

Tensors come out of a range through PyTorch's own caching allocator: every range is a ``torch.cuda.MemPool`` whose
segments the library's ``exodus_hbm_alloc_*`` / ``exodus_hbm_free`` supply (``CUDAPluggableAllocator``).  PyTorch
splits, caches and reuses the segments as it does ordinary memory, which includes keeping track of the streams a
block was used on (``Tensor.record_stream``): a tensor of a range is as safe across streams as any other tensor.

``enable()`` makes the ranges and from then on the kernels' wrappers (``_hip.layerLifForward`` and friends, the
(rows, time) wrappers, the ``IntegrateAndFire`` Function) allocate their big outputs in the striped range.
``with placement():`` sends *every* allocation of the calling thread there (what torch itself allocates in a forward
pass: activations of other layers, temporaries); ``enable(everything=True)`` does that for all threads until
``disable()``, which covers the gradients that autograd's own thread allocates in a backward pass.  Without
``enable()`` nothing changes -- unless the environment asks for it: ``SINABS_EXODUS_HBM=striped[:GiB]`` or
``everything[:GiB]`` stands for that call in a program that is to run unchanged (``_from_environment``).  The reference has no counterpart (its CUDA extension allocates outputs with
``torch.empty_like``, reference cuda/bindings.cu:98,144,183).

While a HIP graph is being captured the wrappers leave allocation to the capture's own pool (a graph's memory must
not be handed to anybody else between replays, which is what that pool guarantees); ``everything=True`` would
override that pool and must not be active during a capture.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import threading
import time
import warnings
from typing import Dict, List, Optional, Sequence

import torch

GIB = 2 ** 30
CHUNK = 4 * GIB                 # physical memory is sorted in pieces of this size: shorter copies tell less
FINER_CHUNK = 256 * 2 ** 20     # ... and in pieces of this size when the big ones show no regions (memory that earlier
                                # processes left mixed below 4 GiB is mostly still in order at this scale)
REGIONS_NOT_FOUND = -3          # EXODUS_ERROR_REGIONS_NOT_FOUND of include/exodus_hip.h
RANGE_IN_USE = -4               # EXODUS_ERROR_RANGE_IN_USE
PROBES = 15                     # EXODUS_HBM_PROBES of include/exodus_hip.h
ARENAS = 4                      # EXODUS_HBM_ARENAS: one range per region and the striped one
STRIPED = 3                     # index of the striped range
SMALLEST_PLACED = 2 ** 20       # the wrappers leave smaller outputs to the ordinary allocator
_ALLOC_NAMES = ("exodus_hbm_alloc_region0", "exodus_hbm_alloc_region1", "exodus_hbm_alloc_region2",
                "exodus_hbm_alloc_striped")


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
                ("probe_kind", ctypes.c_int32 * PROBES), ("probe_pair_GBs", (ctypes.c_float * PROBES) * PROBES),
                ("phase_s", ctypes.c_float * 4)]


def _create(lib, device_index: int, bytes_per_region: int, bytes_striped: int, chunk_sizes: Sequence[int], sort: bool,
            take_limit: int = 0):
    """``exodus_hbm_regions_create`` with each of ``chunk_sizes`` in turn until one shows the regions (or none is
    left); returns (status, report, chunk size used).  A striped range that came out unsorted is given back before
    the next try."""
    for attempt, size in enumerate(chunk_sizes):
        rep = _Report()
        rc = lib.exodus_hbm_regions_create(device_index, bytes_per_region, bytes_striped, int(size), int(sort),
                                           int(take_limit), ctypes.byref(rep))
        no_regions = rc == REGIONS_NOT_FOUND or (rc == 0 and sort and rep.kinds_found != 3)
        if not no_regions or attempt + 1 == len(chunk_sizes):
            break
        if rc == 0:
            lib.exodus_hbm_regions_destroy(device_index)
    return rc, rep, int(size)


class HbmRegions:
    """Address ranges of device memory sorted by region of HBM: one per region (``gib_per_region`` each, may be 0)
    and a striped one (``gib_striped``, may be 0) whose 64 MiB pages alternate between the regions; each range
    is the backing store of a ``torch.cuda.MemPool``.

    The sizes are what the ranges hold for good (until ``close()``); what a range cannot serve comes from the
    ordinary allocator, which is harmless but loses the placement.  Creating the ranges takes nearly all free
    device memory for a moment and gives back what it does not keep, so do it early, before the program's big
    allocations, and not while another process is starting up on the same GPU (``take_limit_gib`` bounds what is
    held, at the price stated in include/exodus_hip.h).
    ``sort=False`` (the default for a striped range alone) builds the striped range from chunks of the first,
    second and last third of the free memory in turn: on a machine that hands memory out in address order those are
    the regions, on one that does not the memory is a mixture already; nothing is timed, so nothing depends on what
    else the machine is doing.  ``sort=True`` (the default when ranges of single regions are asked for, which need
    it) judges the memory with timed copies in pieces of ``chunk_bytes`` (4 GiB; smaller pieces copy too
    quickly to tell the regions apart as reliably), and once more with ``finer_chunk_bytes`` when those show no
    regions -- memory that earlier processes left mixed; it takes several seconds.  ``report`` holds what was measured, ``setup_s`` the time
    the whole set-up took, ``verified`` whether copies between regions beat copies inside them on the finished
    ranges (on the probe chunks when there are no region ranges).
    Raises RuntimeError when too little memory is free, or when ranges of single regions are asked for and the
    device's memory shows no three regions (a striped range alone is then still made, ``sorted`` False).
    """

    def __init__(self, gib_per_region: float = 0.0, gib_striped: float = 48.0,
                 device: Optional[torch.device] = None, chunk_bytes: int = CHUNK, sort: Optional[bool] = None,
                 finer_chunk_bytes: Optional[int] = FINER_CHUNK, take_limit_gib: Optional[float] = None):
        from . import _hip
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("HbmRegions needs a HIP device")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        if gib_per_region < 0 or gib_striped < 0 or (gib_per_region == 0 and gib_striped == 0):
            raise ValueError("gib_per_region and gib_striped must not be negative, and one of them positive")
        if sort is None:
            sort = gib_per_region > 0
        if not sort and gib_per_region:
            raise ValueError("ranges of single regions (gib_per_region) need the sorting")
        if chunk_bytes <= 0 or chunk_bytes % (64 * 2 ** 20):
            raise ValueError("chunk_bytes must be a multiple of the 64 MiB page")
        if gib_per_region + gib_striped / 3 > 80:
            raise ValueError("gib_per_region + gib_striped / 3 must not exceed 80 (rounded up to whole chunks of "
                             "4 GiB): that much is taken from each region, and a region has 96 GiB")
        if take_limit_gib is not None and take_limit_gib <= 0:
            raise ValueError("take_limit_gib must be positive (None: no bound)")
        self._lib = _hip.lib
        self._lib_path = _hip.LIB_PATH
        sizes = [int(chunk_bytes)]
        if sort and finer_chunk_bytes and finer_chunk_bytes < chunk_bytes:
            sizes.append(int(finer_chunk_bytes))
        t0 = time.perf_counter()
        with torch.cuda.device(self.device):
            torch.zeros(1, device=self.device)             # the device's context exists
            torch.cuda.empty_cache()                       # what torch has cached cannot be sorted
            torch.cuda.synchronize()
            rc, rep, size = _create(self._lib, self.device.index, int(gib_per_region * GIB), int(gib_striped * GIB),
                                    sizes, bool(sort), 0 if take_limit_gib is None else int(take_limit_gib * GIB))
        self.setup_s = time.perf_counter() - t0
        self.chunk_bytes = size                            # the size the ranges were sorted in
        self.report: Dict[str, object] = {
            "chunks_examined": rep.chunks_examined, "kinds_found": rep.kinds_found,
            "chunks_ambiguous": rep.chunks_ambiguous, "chunks_of_region": list(rep.chunks_of_region),
            "threshold_GBs": rep.threshold_GBs, "probe_chunks_same_region_GBs": rep.probe_same_kind_GBs,
            "probe_chunks_other_region_GBs": rep.probe_other_kind_GBs,
            "inside_one_range_GBs": list(rep.copy_inside_GBs), "across_ranges_GBs": list(rep.copy_across_GBs),
            "inside_striped_range_GBs": rep.copy_striped_GBs,
            "seconds_taking_sorting_building_checking": [round(v, 3) for v in rep.phase_s]}
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
        # False: no timed copies were made, or they showed no three regions (memory that came back from earlier
        # processes as a mixture of them); the striped range is then made of chunks spread over the memory, as they are
        self.sorted = rep.kinds_found == 3
        self._pools: Dict[int, "torch.cuda.MemPool"] = {}
        self._allocators: Dict[int, object] = {}           # the pools' allocators have to outlive them
        self._lock = threading.Lock()
        self._closing, self._closed = False, False
        self._everything = False
        self._local = threading.local()                    # .depth: placement() contexts this thread is inside
        inside = [r for r in rep.copy_inside_GBs if r > 0] or [rep.probe_same_kind_GBs]
        across = [r for r in rep.copy_across_GBs if r > 0] or [rep.probe_other_kind_GBs]
        # single pairs of chunks scatter by a few percent around 6.0 (same region) and 6.35 TB/s (two regions);
        # the copies over whole ranges average over many pairs
        self.verified = bool(self.sorted and sum(across) / len(across) > 1.025 * sum(inside) / len(inside))
        if self.sorted and not self.verified:
            warnings.warn(f"HbmRegions: copies between the regions are not clearly faster than copies "
                          f"inside them ({self.report}); allocation works, the gain may not be there")

    # ------------------------------------------------------------------ the pools
    def pool(self, k: int = STRIPED) -> "torch.cuda.MemPool":
        """The ``torch.cuda.MemPool`` on range ``k`` (0, 1, 2: a region's; ``STRIPED``), made on first use."""
        k = int(k)
        if not 0 <= k < ARENAS or not self.sizes[k]:
            raise ValueError(f"these ranges have no range {k}")
        with self._lock:
            if self._closing:
                raise RuntimeError("these ranges were closed")
            if k not in self._pools:
                self._allocators[k] = torch.cuda.memory.CUDAPluggableAllocator(self._lib_path, _ALLOC_NAMES[k],
                                                                               "exodus_hbm_free")
                self._pools[k] = torch.cuda.MemPool(self._allocators[k].allocator())
            return self._pools[k]

    def _covered(self) -> bool:
        """True when this thread's allocations go to the striped range anyway."""
        return self._everything or getattr(self._local, "depth", 0) > 0

    @contextlib.contextmanager
    def allocating(self, k: int = STRIPED):
        """Inside the block every device allocation of the calling thread comes from range ``k``
        (``torch.cuda.use_mem_pool``).  Inside ``placement()`` or under ``enable(everything=True)`` the striped range
        is being allocated from already and the block changes nothing."""
        if self._covered() or self._closing:
            yield
            return
        with torch.cuda.use_mem_pool(self.pool(k), device=self.device):
            yield

    @contextlib.contextmanager
    def placement(self):
        """Inside the block every device allocation of the calling thread comes from the striped range: whatever
        torch allocates for the operations in it, not only the outputs of this package's kernels."""
        if self._covered() or self._closing or not self.sizes[STRIPED]:
            yield
            return
        with torch.cuda.use_mem_pool(self.pool(STRIPED), device=self.device):
            self._local.depth = getattr(self._local, "depth", 0) + 1
            try:
                yield
            finally:
                self._local.depth -= 1

    def _set_everything(self, on: bool) -> None:
        if on == self._everything:
            return
        pool = self.pool(STRIPED)
        if on:
            torch._C._cuda_beginAllocateToPool(self.device.index, pool.id)
        else:
            torch._C._cuda_endAllocateToPool(self.device.index, pool.id)
            torch._C._cuda_releasePool(self.device.index, pool.id)
        self._everything = on

    def bytes_in_use(self, k: int = STRIPED) -> int:
        """Bytes of range ``k`` that PyTorch's allocator currently holds as segments (in use or cached)."""
        used = (ctypes.c_uint64 * ARENAS)()
        self._lib.exodus_hbm_usage(self.device.index, used, None)
        return int(used[k])

    def bytes_elsewhere(self) -> int:
        """Bytes that the pools took from the ordinary device memory because their range was full."""
        used, other = (ctypes.c_uint64 * ARENAS)(), ctypes.c_uint64(0)
        self._lib.exodus_hbm_usage(self.device.index, used, ctypes.byref(other))
        return int(other.value)

    # ------------------------------------------------------------------ queries
    def pool_of(self, t: torch.Tensor) -> Optional[int]:
        """Index of the range whose memory holds ``t`` (0, 1, 2: a region's; 3: the striped one), or None."""
        p = t.data_ptr()
        for k in range(ARENAS):
            if self.sizes[k] and self.bases[k] <= p < self.bases[k] + self.sizes[k]:
                return k
        return None

    def live_blocks(self) -> List[tuple]:
        """(address, bytes, range) of every block of the ranges that a tensor still occupies, from PyTorch's own
        book-keeping (``torch.cuda.memory_snapshot``): what keeps ``close()`` from giving the memory back."""
        out = []
        for seg in torch.cuda.memory_snapshot():
            if seg.get("device") != self.device.index:
                continue
            address = seg.get("address", 0)
            for block in seg.get("blocks", []):
                size = block.get("size", 0)
                if str(block.get("state", "")).startswith("active"):
                    for k in range(ARENAS):
                        if self.sizes[k] and self.bases[k] <= address < self.bases[k] + self.sizes[k]:
                            out.append((address, size, k))
                address += size
        return out

    # ------------------------------------------------------------------ allocation
    def empty(self, shape: Sequence[int], dtype=torch.float32, region: Optional[int] = None) -> torch.Tensor:
        """An uninitialised tensor in range ``region`` (0, 1, 2: that region; ``STRIPED``, the default).  From the
        ordinary allocator when there is no such range, when the range is full, and while a HIP graph is being
        captured (the capture's own pool must keep what the graph uses)."""
        shape = tuple(int(s) for s in shape)
        k = STRIPED if region is None else int(region)
        if self.sizes[k] and not self._closing and not torch.cuda.is_current_stream_capturing():
            with self.allocating(k):
                return torch.empty(shape, dtype=dtype, device=self.device)
        return torch.empty(shape, dtype=dtype, device=self.device)

    def empty_like(self, like: torch.Tensor) -> torch.Tensor:
        return self.empty(like.shape, like.dtype)

    def close(self) -> bool:
        """Give the ranges' memory back to the driver.  True when that happened; False when tensors of the ranges
        are still alive: the ranges then stay mapped (new requests go to the ordinary allocator) and a later
        ``close()`` -- ``disable()`` and the next ``enable()`` call it -- tries again."""
        if self._closed:
            return True
        if self._everything:
            self._set_everything(False)
        with self._lock:
            self._closing = True
            self._pools.clear()                            # PyTorch may now release the pools' cached segments
        with torch.cuda.device(self.device):
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            rc = self._lib.exodus_hbm_regions_destroy(self.device.index)
        if rc == RANGE_IN_USE:
            return False
        self._closed = True
        self._allocators.clear()
        if rc != 0:
            text = self._lib.exodus_hip_error_string(rc)
            raise RuntimeError(f"exodus_hbm_regions_destroy: {text.decode() if isinstance(text, bytes) else text}")
        return True


_active: Optional[HbmRegions] = None
_lingering: List[HbmRegions] = []         # closed while tensors were alive: still mapped, to be closed again


def _close_lingering() -> bool:
    _lingering[:] = [r for r in _lingering if not r.close()]
    return not _lingering


def enable(gib_per_region: float = 0.0, gib_striped: float = 48.0, device: Optional[torch.device] = None,
           everything: bool = False, **how) -> HbmRegions:
    """Create the ranges (``HbmRegions(gib_per_region, gib_striped, device, **how)``) and make the kernels' wrappers
    allocate their big outputs in the striped range.  ``everything=True`` sends every allocation on the device
    there, from every thread (autograd's included), until ``disable()``.
    Raises RuntimeError when ranges made earlier cannot be given back because tensors in them are still alive."""
    global _active
    if _active is not None:
        disable()
    if not _close_lingering():
        blocks = [b for r in _lingering for b in r.live_blocks()]
        raise RuntimeError(f"hbm.enable(): {len(blocks)} tensors allocated in the previous ranges are still alive "
                           f"({sum(b[1] for b in blocks)} bytes); release them (and what refers to them, e.g. layer "
                           "states, .grad tensors and autograd graphs) before making new ranges")
    regions = HbmRegions(gib_per_region, gib_striped, device, **how)
    if everything:
        if not regions.sizes[STRIPED]:
            regions.close()
            raise ValueError("everything=True needs a striped range")
        regions._set_everything(True)
    _active = regions
    return regions


def disable() -> bool:
    """Undo ``enable()``.  Tensors that live in the ranges stay valid; the memory goes back to the driver once none
    is left (True: it went back now; False: tensors are alive, a later ``disable()`` or ``enable()`` tries again)."""
    global _active
    if _active is not None:
        _lingering.append(_active)
    _active = None
    return _close_lingering()


def active() -> Optional[HbmRegions]:
    return _active


@contextlib.contextmanager
def placement():
    """``with hbm.placement():`` -- every device allocation of the calling thread inside the block comes from the
    striped range (nothing changes when ``enable()`` was not called)."""
    if _active is None:
        yield
        return
    with _active.placement():
        yield


ENVIRONMENT_SWITCH = "SINABS_EXODUS_HBM"
FIRST_PLACED_UNASKED = 64 * 2 ** 20   # the environment switch makes the ranges when the first output this big is due
_switch_tried = False


def _read_switch(asked: str):
    """``striped`` / ``everything``, optionally ``:<GiB>`` -> (GiB of the striped range, everything); None for an empty
    value or one that says no; ValueError for anything else."""
    asked = asked.strip().lower()
    if not asked or asked in ("0", "off", "no", "false"):
        return None
    mode, _, size = asked.partition(":")
    if mode in ("1", "on", "yes", "true"):
        mode = "striped"
    if mode not in ("striped", "everything"):
        raise ValueError(f"unknown mode '{mode}' (striped or everything, optionally followed by :<GiB>)")
    gib = float(size) if size else 48.0
    if not gib > 0:
        raise ValueError("the size must be positive")
    return gib, mode == "everything"


def _from_environment(nbytes: int, device: torch.device) -> None:
    """``SINABS_EXODUS_HBM=striped`` (or ``striped:<GiB>``, ``everything``, ``everything:<GiB>``; default 48 GiB) in the
    environment stands for a call of ``enable(gib_striped=<GiB>, everything=...)``, for programs that are to run
    unchanged: the ranges are made on the device of the first kernel output of 64 MiB or more (a program with small
    layers never pays the set-up).  A value that cannot be read, or ranges that cannot be made, give one warning and
    the ordinary allocator."""
    global _switch_tried
    if _switch_tried or nbytes < FIRST_PLACED_UNASKED or device.type != "cuda":
        return
    asked = os.environ.get(ENVIRONMENT_SWITCH, "")
    if not asked.strip():
        return
    if torch.cuda.is_current_stream_capturing():
        return                                             # not now: try again at the next eager call
    _switch_tried = True
    try:
        how = _read_switch(asked)
        if how is not None:
            enable(gib_striped=how[0], device=device, everything=how[1])
    except (RuntimeError, ValueError) as err:
        warnings.warn(f"{ENVIRONMENT_SWITCH}={asked}: no placement, ordinary allocator used ({err})")


def _wanted(nbytes: int, device: torch.device) -> bool:
    if _active is None:
        _from_environment(nbytes, device)
    return (_active is not None and nbytes >= SMALLEST_PLACED and device == _active.device
            and bool(_active.sizes[STRIPED]))


def empty_like(like: torch.Tensor) -> torch.Tensor:
    """``torch.empty_like(like)`` (contiguous) -- after ``enable()``, and for 1 MiB or more, in the striped range."""
    if not _wanted(like.numel() * like.element_size(), like.device):
        return torch.empty_like(like, memory_format=torch.contiguous_format)
    return _active.empty(like.shape, like.dtype)


def empty(shape, like: torch.Tensor) -> torch.Tensor:
    """``torch.empty(shape)`` with dtype and device of ``like``, placed as ``empty_like`` places its result."""
    shape = tuple(int(s) for s in shape)
    count = 1
    for s in shape:
        count *= s
    if not _wanted(count * like.element_size(), like.device):
        return torch.empty(shape, dtype=like.dtype, device=like.device)
    return _active.empty(shape, like.dtype)
