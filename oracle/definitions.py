"""TEST INFRASTRUCTURE ONLY -- definition-level builders, written independently of subm_ref.c.

They state WHAT each table is (the mathematical definition) rather than HOW the reference
computes it, so that a slip in the C restatement (wrong offset order, wrong mirror column, an
off-by-one in a segment table) fails the comparison in tests/test_oracle_tables.py.
"""
from __future__ import annotations

from typing import Dict, Sequence, Tuple

import numpy as np

EMPTY = 0xFFFFFFFF


def offsets(kernel_size=(3, 3, 3), dilation=(1, 1, 1)) -> np.ndarray:
    """[V, 3] offset vectors, x-major flattening: v = (i*Kh + j)*Kd + k, delta = ((i-Kw//2)*Dw, ...).

    Same flattening as weight[Co, Kw, Kh, Kd, Ci] -> [Co, V, Ci]
    (flex_gemm/ops/spconv/submanifold_conv3d.py:204; subm_neighbor_map.cu:69-71)."""
    kw, kh, kd = kernel_size
    out = []
    for i in range(kw):
        for j in range(kh):
            for k in range(kd):
                out.append(((i - kw // 2) * dilation[0], (j - kh // 2) * dilation[1], (k - kd // 2) * dilation[2]))
    return np.asarray(out, dtype=np.int64)


def neighbor_map_searchsorted(coords: np.ndarray, shape: Sequence[int], kernel_size=(3, 3, 3),
                              dilation=(1, 1, 1)) -> np.ndarray:
    """neighbor_map[n, v] = m iff coords[m] == coords[n] + delta_v (same batch, inside the grid), else all ones.

    Mirrors the idea of the reference's torch builder (submanifold_conv3d.py:109-144) with int64 keys."""
    coords = np.asarray(coords, dtype=np.int64)
    n = coords.shape[0]
    _, _, W, H, D = [int(s) for s in shape]
    off = offsets(kernel_size, dilation)
    V = off.shape[0]
    out = np.full((n, V), EMPTY, dtype=np.uint32)
    if n == 0:
        return out
    keys = ((coords[:, 0] * W + coords[:, 1]) * H + coords[:, 2]) * D + coords[:, 3]
    order = np.argsort(keys, kind="stable")
    skeys = keys[order]
    for v in range(V):
        q = coords[:, 1:] + off[v][None, :]
        inside = (q[:, 0] >= 0) & (q[:, 0] < W) & (q[:, 1] >= 0) & (q[:, 1] < H) & (q[:, 2] >= 0) & (q[:, 2] < D)
        qk = ((coords[:, 0] * W + q[:, 0]) * H + q[:, 1]) * D + q[:, 2]
        pos = np.clip(np.searchsorted(skeys, qk), 0, n - 1)
        hit = inside & (skeys[pos] == qk)
        out[hit, v] = order[pos[hit]].astype(np.uint32)
    return out


def neighbor_map_bruteforce(coords: np.ndarray, shape: Sequence[int], kernel_size=(3, 3, 3),
                            dilation=(1, 1, 1)) -> np.ndarray:
    """Python dict on coordinate tuples; small inputs only."""
    _, _, W, H, D = [int(s) for s in shape]
    table = {tuple(int(t) for t in c): i for i, c in enumerate(coords)}
    off = offsets(kernel_size, dilation)
    out = np.full((len(coords), off.shape[0]), EMPTY, dtype=np.uint32)
    for i, c in enumerate(coords):
        b, x, y, z = (int(t) for t in c)
        for v, (dx, dy, dz) in enumerate(off):
            q = (x + int(dx), y + int(dy), z + int(dz))
            if 0 <= q[0] < W and 0 <= q[1] < H and 0 <= q[2] < D:
                m = table.get((b,) + q)
                if m is not None:
                    out[i, v] = m
    return out


def gray_code(nmap: np.ndarray) -> np.ndarray:
    V = nmap.shape[1]
    bits = (nmap != EMPTY).astype(np.int64) << np.arange(V, dtype=np.int64)[None, :]
    return bits.sum(axis=1).astype(np.uint32).view(np.int32)


def gray_to_binary(gray: np.ndarray) -> np.ndarray:
    """Textbook Gray decode, bit by bit from the MSB: b_top = g_top, b_i = b_{i+1} xor g_i."""
    g = gray.view(np.uint32).astype(np.uint64)
    b = np.zeros_like(g)
    prev = np.zeros_like(g)
    for bit in range(31, -1, -1):
        cur = prev ^ ((g >> np.uint64(bit)) & np.uint64(1))
        b |= cur << np.uint64(bit)
        prev = cur
    return b.astype(np.uint32).view(np.int32)


def pair_lists(nmap: np.ndarray) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Pairs (v, n) in lexicographic order with a present neighbor."""
    V = nmap.shape[1]
    vs, ns = np.nonzero(nmap.T != EMPTY)
    sig_o = ns.astype(np.uint32)
    sig_i = nmap.T[vs, ns].astype(np.uint32)
    seg = np.zeros(V + 1, dtype=np.uint32)
    seg[1:] = np.cumsum(np.bincount(vs, minlength=V))
    return sig_i, sig_o, seg


def tile_masks(gray: np.ndarray, sorted_idx: np.ndarray, block: int) -> Tuple[np.ndarray, np.ndarray]:
    g = gray.view(np.uint32)[sorted_idx]
    n = g.shape[0]
    nb = (n + block - 1) // block
    vk = []
    seg = [0]
    for b in range(nb):
        code = int(np.bitwise_or.reduce(g[b * block:(b + 1) * block])) if n else 0
        vk.extend(v for v in range(32) if (code >> v) & 1)
        seg.append(len(vk))
    return np.asarray(vk, dtype=np.int32), np.asarray(seg, dtype=np.int32)
