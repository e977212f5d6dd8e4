"""What a captured HIP graph is made of.

A step may be replayed as a graph only if every node of the graph is a kernel launch. A library
product can bring other nodes into a capture (a kernel that needs a cleared workspace records a
memset node before itself), and memset nodes in a replayed graph have given wrong results on the
second and later replays. So the runner looks at each graph it has captured and throws away any
that holds something else than kernels; that step's shape then runs eagerly.
"""

from __future__ import annotations

import ctypes
from collections import Counter

import torch

# hipGraphNodeType (hip/hip_runtime_api.h)
NODE_KINDS = {
    0: "kernel", 1: "memcpy", 2: "memset", 3: "host", 4: "graph", 5: "empty", 6: "wait_event",
    7: "event_record", 8: "semaphore_signal", 9: "semaphore_wait", 10: "mem_alloc", 11: "mem_free",
    12: "memcpy_from_symbol", 13: "memcpy_to_symbol", 14: "batch_mem_op",
}

_hip = None


def _runtime() -> ctypes.CDLL:
    """The HIP runtime this process already runs on (the one torch loaded), not a second copy."""
    global _hip
    if _hip is None:
        path = None
        with open("/proc/self/maps", encoding="utf-8") as maps:
            for line in maps:
                if "libamdhip64" in line:
                    path = line.split()[-1]
                    break
        if path is None:
            raise RuntimeError("no HIP runtime is loaded in this process")
        lib = ctypes.CDLL(path)
        lib.hipGraphGetNodes.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t)]
        lib.hipGraphGetNodes.restype = ctypes.c_int
        lib.hipGraphNodeGetType.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        lib.hipGraphNodeGetType.restype = ctypes.c_int
        _hip = lib
    return _hip


def node_kinds(graph: "torch.cuda.CUDAGraph") -> Counter:
    """How many nodes of each kind a captured graph holds, e.g. ``{"kernel": 231}``. The graph
    must have been made with ``keep_graph=True``."""
    hip = _runtime()
    handle = ctypes.c_void_p(graph.raw_cuda_graph())
    count = ctypes.c_size_t(0)
    status = hip.hipGraphGetNodes(handle, None, ctypes.byref(count))
    if status != 0:
        raise RuntimeError(f"hipGraphGetNodes failed with status {status}")
    nodes = (ctypes.c_void_p * max(count.value, 1))()
    if count.value:
        status = hip.hipGraphGetNodes(handle, nodes, ctypes.byref(count))
        if status != 0:
            raise RuntimeError(f"hipGraphGetNodes failed with status {status}")
    kinds: Counter = Counter()
    for i in range(count.value):
        kind = ctypes.c_int(-1)
        status = hip.hipGraphNodeGetType(nodes[i], ctypes.byref(kind))
        if status != 0:
            raise RuntimeError(f"hipGraphNodeGetType failed with status {status}")
        kinds[NODE_KINDS.get(kind.value, f"kind {kind.value}")] += 1
    return kinds


def only_kernels(kinds: Counter) -> bool:
    return all(kind == "kernel" for kind in kinds)
