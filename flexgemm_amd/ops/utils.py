"""Hash-table allocation for the neighbor-map builder."""
import ctypes as C

import torch

from .. import _native as nat


def hashmap_key_dtype(spatial_size):
    """uint32 keys when the flattened index space B*W*H*D is below 2^32, else uint64
    (same rule as the reference's init_hashmap, flex_gemm/ops/utils.py:9-17)."""
    n, _, w, h, d = spatial_size
    vol = int(n) * int(w) * int(h) * int(d)
    if vol < 2 ** 32:
        return torch.uint32
    if vol < 2 ** 64:
        return torch.uint64
    raise ValueError(f"The spatial size is too large to fit in a hashmap. Get volumn {vol} > 2^64.")


def init_hashmap(spatial_size, hashmap_size, device, with_values=True):
    """Allocate an empty open-addressing table of `hashmap_size` slots on `device`.

    Keys are set to the all-ones sentinel by the library's fill kernel; values stay uninitialised.
    Mirrors flex_gemm/ops/utils.py:4-19 (signature and return convention)."""
    kdt = hashmap_key_dtype(spatial_size)
    device = torch.device(device)
    if device.type != "cuda":
        raise NotImplementedError("CPU version of hashmap is not implemented")
    keys = torch.empty((int(hashmap_size),), dtype=kdt, device=device)
    with torch.cuda.device(device):
        nat.check(nat.lib().fgx_hash_init(nat.ptr(keys), C.c_int(32 if kdt == torch.uint32 else 64),
                                          nat.sz(hashmap_size), nat.stream()))
    if with_values:
        vals = torch.empty((int(hashmap_size),), dtype=torch.uint32, device=device)
        return keys, vals
    return keys
