"""TEST INFRASTRUCTURE ONLY -- a CPU builder and a checker for the chunk plan of the chunk-resident gather GEMM
(fgx_chunk_plan_* / fgx_conv_gather_gemm_chunk).  Nothing shipped may import this module.

The chunk plan has no counterpart in the reference: it is a private schedule of the gfx950 kernels, like the
reference's `valid_kernel` lists are a private schedule of its Triton kernels
(flex_gemm/kernels/cuda/spconv/migemm_neighmap_pp.cu:246-368).  What IS fixed by the reference is the table it must
reproduce, neighbor_map[n, v] (flex_gemm/kernels/cuda/spconv/subm_neighbor_map.cu:33-83).  `check()` therefore states
the plan's contract in terms of that map alone, so any builder -- this one or the HIP one -- is tested against the
definition, not against another builder's choices:

  * every output row appears in exactly one (chunk, position);
  * for every position p holding row n and every offset v:  chunk_src[c][chunk_idx[c][v][p]] == neighbor_map[n, v]
    (all ones, the empty marker, for a missing neighbor: local row 0 of every chunk is the empty row);
  * band masks: bit v of chunk_band[c][band] is set iff some row of the band has a neighbor at v;
  * chunk_nsrc[c] <= SMAX and every local row at or beyond it is empty.

Layout (shared with flexgemm_amd/csrc/conv_gemm_chunk.hip):
  CS = 512 rows per chunk = 8 wavefronts x 4 bands x 16 rows; position p = wave * 64 + band * 16 + row.
  chunk_src  uint32 [nchunks, SMAX]        source row of each local row (0xFFFFFFFF = empty)
  chunk_nsrc int32  [nchunks]              local rows in use (including the empty row 0)
  chunk_idx  uint16 [nchunks, V, 8, 16, 4] local row of neighbor v of position (wave, row, band)
  chunk_out  uint32 [nchunks, 512]         output row at each position (0xFFFFFFFF = none)
  chunk_band uint32 [nchunks, 32]          offset mask of band wave * 4 + band
"""
from __future__ import annotations

import numpy as np

from . import serialize

EMPTY = 0xFFFFFFFF
CS = 512
WAVES = 8
BANDS_PER_WAVE = 4
BAND = 16
SMAX = 912


def _gray_decode(g: np.ndarray) -> np.ndarray:
    b = g.astype(np.int64) & 0xFFFFFFFF
    s = 1
    while s < 32:
        b ^= b >> s
        s <<= 1
    return b


def curve_order(coords: np.ndarray, mode: str = "hilbert") -> np.ndarray:
    """Rows ranked along a space-filling curve over (b, x, y, z); ties (repeated voxels) keep their input order."""
    c = np.asarray(coords, dtype=np.int64)
    ext = int(c[:, 1:].max()) + 1 if c.shape[0] else 1
    bl = max((ext - 1).bit_length(), 1)
    code = serialize.encode(c, bl, mode).view(np.uint64)
    return np.argsort(code, kind="stable")


def build(coords: np.ndarray, nmap: np.ndarray, mode: str = "hilbert", smax: int = SMAX):
    """Reference plan: chunks of CS consecutive rows along the curve; inside a chunk rows sorted by the Gray-decoded
    offset mask, band j of that order dealt to wavefront j % 8; local rows = empty row, the chunk's own rows in curve
    order, then the other rows its neighbors name in ascending curve rank.  Returns a dict of the five arrays, or
    None when some chunk needs more than `smax` local rows."""
    nmap = np.asarray(nmap)
    n, V = nmap.shape
    nm = nmap.astype(np.int64)
    nm[nm == EMPTY] = -1
    mask = ((nm >= 0).astype(np.int64) << np.arange(V, dtype=np.int64)[None, :]).sum(1)
    key = _gray_decode(mask)
    order = curve_order(coords, mode)
    rank = np.empty(n, dtype=np.int64)
    rank[order] = np.arange(n)
    nch = (n + CS - 1) // CS
    chunk_src = np.full((nch, smax), EMPTY, dtype=np.uint32)
    chunk_nsrc = np.zeros((nch,), dtype=np.int32)
    chunk_idx = np.zeros((nch, V, WAVES, BAND, BANDS_PER_WAVE), dtype=np.uint16)
    chunk_out = np.full((nch, CS), EMPTY, dtype=np.uint32)
    chunk_band = np.zeros((nch, WAVES * BANDS_PER_WAVE), dtype=np.uint32)
    local_of = np.zeros(n, dtype=np.int64)            # scratch: local row of a source row in the current chunk
    for c in range(nch):
        rows = order[c * CS:(c + 1) * CS]                 # curve order
        m = len(rows)
        nb = nm[rows]                                     # [m, V]
        inside = (nb >= 0) & (rank[np.maximum(nb, 0)] // CS == c)
        halo = np.unique(nb[(nb >= 0) & ~inside])
        halo = halo[np.argsort(rank[halo], kind="stable")]
        nsrc = 1 + m + len(halo)
        if nsrc > smax:
            return None
        chunk_nsrc[c] = nsrc
        chunk_src[c, 1:1 + m] = rows
        chunk_src[c, 1 + m:nsrc] = halo
        local_of[rows] = 1 + np.arange(m)
        local_of[halo] = 1 + m + np.arange(len(halo))
        srt = np.argsort(key[rows], kind="stable")        # positions in mask order
        j = np.arange(m)
        band_j, r = j // BAND, j % BAND
        wave, slot = band_j % WAVES, band_j // WAVES
        chunk_out[c, wave * 64 + slot * BAND + r] = rows[srt]
        np.bitwise_or.at(chunk_band[c], wave * BANDS_PER_WAVE + slot, mask[rows[srt]].astype(np.uint32))
        nbs = nb[srt]                                     # [m, V] in mask order
        loc = np.where(nbs >= 0, local_of[np.maximum(nbs, 0)], 0)
        chunk_idx[c][:, wave, r, slot] = loc.T.astype(np.uint16)
    return dict(chunk_src=chunk_src, chunk_nsrc=chunk_nsrc, chunk_idx=chunk_idx, chunk_out=chunk_out,
                chunk_band=chunk_band)


def check(plan, nmap: np.ndarray, smax: int = SMAX) -> None:
    """Assert the contract in the module docstring; raises AssertionError naming what failed."""
    nmap = np.asarray(nmap).astype(np.int64) & 0xFFFFFFFF
    n, V = nmap.shape
    src = np.asarray(plan["chunk_src"]).astype(np.int64) & 0xFFFFFFFF
    nsrc = np.asarray(plan["chunk_nsrc"]).astype(np.int64)
    idx = np.asarray(plan["chunk_idx"]).astype(np.int64)
    out = np.asarray(plan["chunk_out"]).astype(np.int64) & 0xFFFFFFFF
    band = np.asarray(plan["chunk_band"]).astype(np.int64) & 0xFFFFFFFF
    nch = src.shape[0]
    assert src.shape == (nch, smax) and out.shape == (nch, CS) and band.shape == (nch, WAVES * BANDS_PER_WAVE)
    assert idx.shape == (nch, V, WAVES, BAND, BANDS_PER_WAVE)
    assert (nsrc >= 1).all() and (nsrc <= smax).all(), "chunk_nsrc out of range"
    assert (src[:, 0] == EMPTY).all(), "local row 0 must be the empty row"
    beyond = np.arange(smax)[None, :] >= nsrc[:, None]
    assert (src[beyond] == EMPTY).all(), "local rows beyond chunk_nsrc must be empty"
    live = out != EMPTY
    rows = out[live]
    assert rows.size == n and (np.sort(rows) == np.arange(n)).all(), "every output row exactly once"
    # position p = wave * 64 + slot * 16 + r  <->  idx[c, v, wave, r, slot]
    idx_p = idx.transpose(0, 1, 2, 4, 3).reshape(nch, V, CS)          # [c, v, p]
    assert (idx_p < nsrc[:, None, None]).all(), "local row index beyond chunk_nsrc"
    named = np.take_along_axis(src[:, None, :].repeat(V, axis=1), idx_p, axis=2)     # [c, v, p]
    want = np.full((nch, V, CS), EMPTY, dtype=np.int64)
    cc, pp = np.nonzero(live)
    want[cc, :, pp] = nmap[out[cc, pp]]
    assert (named == want).all(), "chunk_src[chunk_idx] does not reproduce neighbor_map"
    has = (want != EMPTY).reshape(nch, V, WAVES * BANDS_PER_WAVE, BAND).any(axis=3)   # [c, v, band]
    want_band = (has.astype(np.int64) << np.arange(V, dtype=np.int64)[None, :, None]).sum(axis=1)
    assert (band == want_band).all(), "band masks"
