"""Pinned host memory for the offload path, placed where the link is.

The reference keeps the target's layers in `pin_memory()` tensors (umbrella/models/llama.py:203-212, llama_layer.py:220-258)
and lets the allocator decide where the pages live.  On a two-socket host that decides the copy rate: a slab on the far
socket crosses the inter-socket fabric on its way to the GPU (round 4 measured 330 - 377 ms per step for the same 40
streamed layers, by what the process had allocated before).  Here the slabs of a model come out of ONE arena:

  * ONE pinned allocation (hipHostMalloc) made while the allocating thread prefers the NUMA
    node of the GPU's PCIe root (libnuma `numa_set_preferred`; the node is read from sysfs) and touched once there -- one
    allocation instead of one per layer, and no registration of existing pages (hosts may refuse it);
  * `reserve()` lets a process claim the arena EARLY (bench.py does, before the headline's allocations fragment the
    host); a model that streams takes its slabs from the reserved arena when it fits, else from a fresh one;
  * every step that is not available (no libnuma, a single-node host, no sysfs entry) degrades to the next best thing
    and `describe()` says which: the bench line reports `numa_node`, `arena` and the per-copy rates.
"""
from __future__ import annotations

import ctypes as C
import os
import weakref

import torch

ALIGN = 2 << 20


def gpu_numa_node(device) -> int:
    """NUMA node of the GPU's PCIe function (sysfs), -1 if the host does not say"""
    try:
        p = torch.cuda.get_device_properties(torch.device(device))
        dom, bus, dev = getattr(p, "pci_domain_id", 0), p.pci_bus_id, p.pci_device_id
        with open(f"/sys/bus/pci/devices/{dom:04x}:{bus:02x}:{dev:02x}.0/numa_node") as f:
            return int(f.read().strip())
    except Exception:
        return -1


def host_nodes() -> int:
    try:
        return len([d for d in os.listdir("/sys/devices/system/node") if d.startswith("node") and d[4:].isdigit()])
    except OSError:
        return 1


HOST_MALLOC_NUMA_USER = 0x20000000      # hipHostMallocNumaUser: place the pages by the calling thread's NUMA policy
_hip = None


def _hip_runtime():
    """the HIP runtime torch has already loaded, through ctypes (hipHostMalloc / hipHostFree only)"""
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so")
        _hip.hipHostMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.c_uint]
        _hip.hipHostMalloc.restype = C.c_int
        _hip.hipHostFree.argtypes = [C.c_void_p]
        _hip.hipHostFree.restype = C.c_int
        _hip.hipGetLastError.restype = C.c_int
    return _hip


class HostArena:
    def __init__(self, nbytes: int, device):
        self.size = (int(nbytes) + ALIGN - 1) // ALIGN * ALIGN
        self.device = torch.device(device)
        self.node = gpu_numa_node(device)
        if os.environ.get("UMB_HOST_ARENA_NODE"):                        # experiments: place the arena on a chosen node
            self.node = int(os.environ["UMB_HOST_ARENA_NODE"])
        self.nodes = host_nodes()
        self.notes = []
        # The arena is ALLOCATED pinned (hipHostMalloc), never registered after the fact:
        # registering existing pages (hipHostRegister) is refused on some hosts, and the error it leaves behind surfaces in
        # whatever GPU call comes next.  Placement: the allocating thread prefers the GPU's NUMA node while the pages are
        # first touched (libnuma numa_set_preferred; local allocation is restored right after).
        numa, self.bound = None, False
        if self.node >= 0 and self.nodes > 1:
            try:
                numa = C.CDLL("libnuma.so.1", use_errno=True)
                if numa.numa_available() >= 0:
                    numa.numa_node_size64.argtypes = [C.c_int, C.POINTER(C.c_longlong)]
                    numa.numa_node_size64.restype = C.c_longlong
                    free = C.c_longlong(0)
                    total = numa.numa_node_size64(self.node, C.byref(free))
                    if total > 0 and free.value >= self.size + (1 << 30):
                        numa.numa_set_preferred.argtypes = [C.c_int]
                        numa.numa_set_preferred(self.node)
                        self.bound = True
                    else:
                        self.notes.append(f"node {self.node} has {free.value >> 20} MiB free of the {self.size >> 20} MiB wanted: "
                                          "first-touch placement")
                else:
                    numa = None
            except OSError:
                numa = None
                self.notes.append("libnuma missing: first-touch placement")
        elif self.nodes <= 1:
            self.notes.append("single NUMA node")
        else:
            self.notes.append("GPU NUMA node unknown")
        # hipHostMalloc directly, not torch's caching pinned allocator: that one rounds a request up to a power of two
        # (36 GB of slabs would pin 64) and keeps the block pinned after the model is gone
        self.base = None
        hip = _hip_runtime()
        ptr = C.c_void_p()
        try:
            rc = hip.hipHostMalloc(C.byref(ptr), self.size + ALIGN, HOST_MALLOC_NUMA_USER if self.bound else 0)
            if rc != 0 and self.bound:
                hip.hipGetLastError()
                rc = hip.hipHostMalloc(C.byref(ptr), self.size + ALIGN, 0)
            if rc != 0 or not ptr.value:
                hip.hipGetLastError()                                    # leave no sticky error behind for the next GPU call
                raise MemoryError(f"hipHostMalloc of {self.size >> 20} MiB failed ({rc})")
            self.base = ptr.value
            C.memset(self.base, 0, self.size + ALIGN)                    # first touch under the preference
        finally:
            if numa is not None and self.bound:
                numa.numa_set_localalloc()
        self.skew = (-self.base) % ALIGN                                 # slabs start on 2 MiB boundaries
        self.off = 0
        self.live = 0

    def alloc(self, nbytes: int):
        """a pinned uint8 CPU tensor of nbytes inside the arena (2 MiB aligned), or None if it does not fit"""
        n = (int(nbytes) + ALIGN - 1) // ALIGN * ALIGN
        if self.base is None or self.off + n > self.size:
            return None
        buf = (C.c_uint8 * int(nbytes)).from_address(self.base + self.skew + self.off)
        t = torch.frombuffer(buf, dtype=torch.uint8)
        t._arena = self                                                  # the arena outlives its tensors
        self.off += n
        self.live += 1
        weakref.finalize(t, self._gone)
        return t

    def _gone(self):
        self.live = max(0, self.live - 1)

    def release_all(self):
        """forget every slab handed out (their tensors must be gone): the arena can be carved again"""
        self.off, self.live = 0, 0

    def describe(self) -> dict:
        return {"arena": f"{self.size >> 20} MiB in one pinned allocation" + ("; " + "; ".join(self.notes) if self.notes else ""),
                "numa_node": self.node, "host_numa_nodes": self.nodes, "bound_to_gpu_node": self.bound}

    def close(self):
        if getattr(self, "base", None):
            _hip_runtime().hipHostFree(C.c_void_p(self.base))
            self.base = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_reserved: HostArena | None = None


def reserve(nbytes: int, device) -> HostArena | None:
    """claim an arena now for a model that will stream later (None, with the reason logged by the caller, if it cannot be had)"""
    global _reserved
    if _reserved is not None and _reserved.size >= nbytes:
        return _reserved
    try:
        _reserved = HostArena(nbytes, device)
    except Exception:
        _reserved = None
    return _reserved


def take(nbytes: int, device) -> HostArena | None:
    """the reserved arena if it is idle and large enough, else a new one, else None (the caller falls back to pin_memory)"""
    if os.environ.get("UMB_HOST_ARENA", "1") == "0":
        return None
    if _reserved is not None and _reserved.live == 0 and _reserved.size >= nbytes and _reserved.device == torch.device(device):
        _reserved.release_all()
        return _reserved
    try:
        return HostArena(nbytes, device)
    except Exception:
        return None
