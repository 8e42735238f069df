"""Submanifold sparse 3-D convolution on MI355X: host side of the operator.

Public surface and argument meaning follow the reference operator
(flex_gemm/ops/spconv/submanifold_conv3d.py): `sparse_submanifold_conv3d`, `SubMConv3dFunction`
with its four static helpers, and the attribute-bag `SubMConv3dNeighborCache`.  All device work
of the implicit-GEMM algorithms is done by hand-written gfx950 kernels behind the C ABI in
include/flexgemm_hip.h; torch only allocates tensors and owns the stream.
"""
from __future__ import annotations

import ctypes as C
import threading
import weakref
from typing import Optional, Tuple

import torch
from torch.autograd import Function

from ... import _native as nat
from .. import spconv, utils
from . import Algorithm

EMPTY = 0xFFFFFFFF

_IMPLICIT = (Algorithm.IMPLICIT_GEMM, Algorithm.IMPLICIT_GEMM_SPLITK,
             Algorithm.MASKED_IMPLICIT_GEMM, Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
_NO_SPLITK = (Algorithm.IMPLICIT_GEMM, Algorithm.MASKED_IMPLICIT_GEMM)
_MASKED = (Algorithm.MASKED_IMPLICIT_GEMM, Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)


def _require_cuda(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise NotImplementedError(f"{what}: the implicit-GEMM algorithms run on the GPU only (got a {t.device} tensor)")


class SubMConv3dNeighborCache:
    """Neighbor tables of one coordinate set, reusable across layers and calls.

    Fields (reference: submanifold_conv3d.py:86-104): `neighbor_map` uint32 [N, V]; for the
    implicit-GEMM algorithms also `gray_code` int32 [N] (validity mask), `sorted_idx` int64 [N];
    when gradients are needed `valid_signal_i`, `valid_signal_o` uint32 [L] and `valid_signal_seg`
    uint32 [V+1].  `valid_kernel_{B}` / `valid_kernel_seg_{B}` are computed on demand per tile
    size B.  Names starting with an underscore are private schedules of the gfx950 kernels.
    """

    def __init__(self, **kwargs):
        for k, v in kwargs.items():
            setattr(self, k, v)

    def __getitem__(self, key):
        return getattr(self, key)

    def __setitem__(self, key, value):
        setattr(self, key, value)

    def __contains__(self, key):
        return hasattr(self, key)

    # The pair lists are filled while their length L is still on its way to the host: they are allocated at their bound
    # (one entry per slot of the map) and cut to L when somebody first reads them or the host copy of the segment
    # table, which by then has long arrived.  (__getattr__ is only asked for names that are not there yet.)
    _PENDING = ("valid_signal_i", "valid_signal_o", "_valid_signal_seg_host")

    def __getattr__(self, name):
        if name in SubMConv3dNeighborCache._PENDING and "_pending_pairs" in self.__dict__:
            self._finish_pairs()
            return self.__dict__[name]
        raise AttributeError(name)

    def _attach_pairs(self, pairs):
        """Take the result of _pair_lists: finished lists, or buffers whose length is still in flight."""
        self["valid_signal_seg"] = pairs["seg"]
        if "pending" in pairs:
            self.__dict__["_pending_pairs"] = pairs["pending"]
        else:
            self["valid_signal_i"], self["valid_signal_o"] = pairs["sig_i"], pairs["sig_o"]
            self["_valid_signal_seg_host"] = pairs["seg_host"]

    def _finish_pairs(self):
        buf_i, buf_o, seg_pinned, arrived = self.__dict__.pop("_pending_pairs")
        arrived.synchronize()
        seg_host = [x & 0xFFFFFFFF for x in seg_pinned.tolist()]
        total = seg_host[-1]
        self["valid_signal_i"], self["valid_signal_o"] = buf_i[:total], buf_o[:total]
        self["_valid_signal_seg_host"] = seg_host

    # -- per-tile offset lists -------------------------------------------------------------------
    def _tile_tables(self, block_size: int, private: bool):
        """(order int64 [N], tile_code int32 [nb], seg int32 [nb+1]) for tiles of `block_size` rows; no host sync.

        private=False: tiles of the public `sorted_idx` (what `valid_kernel_{B}` describes).
        private=True : tiles of the cache-friendly row order the gfx950 kernels walk (`_tile_order` when the cache
        was built from coordinates, otherwise the public order)."""
        if private:
            self._ensure_tile_order()
        use_private = private and hasattr(self, "_tile_order")
        order = self["_tile_order"] if use_private else self["sorted_idx"]
        key = f"_tile_code_{block_size}" if use_private else f"_mask_code_{block_size}"
        seg_key = f"_tile_seg_{block_size}" if use_private else f"valid_kernel_seg_{block_size}"
        if not hasattr(self, key):
            gray = self["gray_code"]
            n = gray.shape[0]
            nb = (n + block_size - 1) // block_size
            code = torch.empty((nb,), dtype=torch.int32, device=gray.device)
            seg = torch.empty((nb + 1,), dtype=torch.int32, device=gray.device)
            with torch.cuda.device(gray.device):
                L = nat.lib()
                ws_bytes = L.fgx_tile_workspace_bytes(nat.sz(n), C.c_int(block_size))
                ws = nat.workspace(ws_bytes, gray.device)
                nat.check(L.fgx_tile_codes(nat.ptr(gray), nat.ptr(order), nat.sz(n), C.c_int(block_size),
                                           nat.ptr(code), nat.ptr(seg), nat.ptr(ws), nat.sz(ws.numel()), nat.stream()))
            setattr(self, key, code)
            setattr(self, seg_key, seg)
        return order, getattr(self, key), getattr(self, seg_key)

    def _dense_tile_tables(self, block_size: int):
        """(order, tile_code) of the non-masked schedule (reference: ..._fwd_implicit_gemm.py:18-89): rows in their
        natural order, every tile walks all V offsets."""
        key = f"_dense_code_{block_size}"
        if not hasattr(self, key):
            nmap = self["neighbor_map"]
            n, v = nmap.shape
            nb = (n + block_size - 1) // block_size
            full = (1 << v) - 1
            if full >= 1 << 31:
                full -= 1 << 32                  # V = 32: all ones as int32
            if not hasattr(self, "_dense_order"):
                self["_dense_order"] = torch.arange(n, dtype=torch.int64, device=nmap.device)
            setattr(self, key, torch.full((nb,), full, dtype=torch.int32, device=nmap.device))
        return self["_dense_order"], getattr(self, key)

    def _gather_plan(self, block_size: int, private: bool, dense: bool = False):
        """(order, tile_code int32 [nb], plan_seg int32 [nb+1], plan_idx uint32 [P, block_size], plan_band uint32 [P])
        for the streaming GEMM: per tile and offset present in it, the tile's source rows as one contiguous run and the
        mask of its 32-row bands that hold any.  Built once per tile size and kept with the cache; the lists are
        allocated at their bound (every offset present in every tile), plan_seg[-1] rows of them are used."""
        if dense:
            order, code = self._dense_tile_tables(block_size)
            key = f"_plan_d_{block_size}"
        else:
            order, code, _ = self._tile_tables(block_size, private)
            use_private = private and hasattr(self, "_tile_order")
            key = f"_plan_{'t' if use_private else 'm'}_{block_size}"
        if not hasattr(self, key):
            nmap = self["neighbor_map"]
            n, v = nmap.shape
            nb = code.shape[0]
            dev = nmap.device
            seg = torch.empty((nb + 1,), dtype=torch.int32, device=dev)
            with torch.cuda.device(dev):
                L = nat.lib()
                ws = nat.workspace(L.fgx_tile_workspace_bytes(nat.sz(nb), C.c_int(1)), dev)
                nat.check(L.fgx_gather_plan_count(nat.ptr(code), nat.sz(nb), nat.ptr(seg), nat.ptr(ws), nat.sz(ws.numel()),
                                                  nat.stream()))
                rows = nb * min(v, 32)       # the bound (every offset in every tile): no wait for the exact count
                plan_idx = torch.empty((rows, block_size), dtype=torch.uint32, device=dev)
                plan_band = torch.empty((rows,), dtype=torch.uint32, device=dev)
                nat.check(L.fgx_gather_plan_fill(nat.ptr(nmap), nat.ptr(order), nat.ptr(code), nat.ptr(seg), nat.sz(n),
                                                 C.c_int(v), C.c_int(block_size), nat.ptr(plan_idx), nat.ptr(plan_band),
                                                 nat.stream()))
            setattr(self, key, (seg, plan_idx, plan_band))
        return (order, code) + getattr(self, key) + (key,)

    def _item_order(self, plan_key: str, code: torch.Tensor, col_tiles: int, groups: int, slabs: int):
        """uint32 device tensor for fgx_conv_gather_gemm_stream's item_at (or None): the tiles dealt to the persistent
        workgroups by cost, built on the device (no read-back) once per plan and shape and kept with the cache."""
        mode = spconv.GEMM_ITEM_ORDER
        nb = code.shape[0]
        if mode == "auto":
            # the locality order of short-row layers lives on neighboring tiles sharing an XCD (dealing them by cost
            # alone: 0.32 -> 0.42 ms per launch at C = 32); with rows of 512 bytes and more balance wins whatever the
            # number of tiles (-6 % per launch at C = 256, -8 % at C = 1024); with shorter rows it wins while a workgroup
            # has few tiles (C = 128, forward: 143 616 voxels 0.120 -> 0.101 ms, 252 392 voxels 0.179 -> 0.155, 577 592
            # voxels 0.342 -> 0.320; 669 288 voxels, 10 rounds of items, and 1 026 536 voxels, 16 rounds: no change), and the ordering kernel takes
            # ~3 us per round of items and neighbor cache
            few_rounds = nb * col_tiles <= ITEM_ORDER_ANY_ROW_MAX_ROUNDS * groups
            mode = "balanced" if (slabs >= 4 or few_rounds) and not plan_key.startswith("_plan_t_") else "default"
        # with at most one item per workgroup there is nothing to even out; from there on the dealt order pays (forward at
        # 64 160 voxels: C = 256, two rounds of items, 0.158 -> 0.141 ms; C = 512, four rounds, 0.550 -> 0.512 ms;
        # 15 192 voxels C = 1024, two rounds, 0.601 -> 0.568 ms)
        if mode == "default" or nb * col_tiles <= ITEM_ORDER_MIN_ROUNDS * groups or groups > 1024:
            return None
        if mode != "balanced":
            raise ValueError(f"unknown GEMM_ITEM_ORDER {spconv.GEMM_ITEM_ORDER!r}; expected 'auto', 'balanced' or 'default'")
        key = f"_items_{plan_key}_{col_tiles}_{groups}_{slabs}"
        if not hasattr(self, key):
            dev = code.device
            item_at = torch.empty((nb * col_tiles,), dtype=torch.int32, device=dev)
            with torch.cuda.device(dev):
                L = nat.lib()
                ws = nat.workspace(L.fgx_gather_item_order_workspace_bytes(nat.sz(nb), C.c_int(col_tiles)), dev)
                nat.check(L.fgx_gather_item_order(nat.ptr(code), nat.sz(nb), C.c_int(col_tiles), C.c_int(slabs), C.c_int(groups),
                                                  nat.ptr(ws), nat.sz(ws.numel()), nat.ptr(item_at), nat.stream()))
            setattr(self, key, item_at)
        return getattr(self, key)

    def compute_kernel_idx(self, block_size: int):
        """Fill `valid_kernel_{B}` / `valid_kernel_seg_{B}` (reference: submanifold_conv3d.py:20-23,
        native side migemm_neighmap_pp.cu:330-368).  One 4-byte read-back sizes the list."""
        block_size = int(block_size)
        if block_size < 1:
            raise ValueError(f"block_size must be positive, got {block_size}")
        _, code, seg = self._tile_tables(block_size, private=False)
        nb = code.shape[0]
        total = int(seg[-1].item())
        vk = torch.empty((total,), dtype=torch.int32, device=code.device)
        if total:
            with torch.cuda.device(code.device):
                nat.check(nat.lib().fgx_tile_fill(nat.ptr(code), nat.ptr(seg), nat.sz(nb), nat.ptr(vk), nat.stream()))
        self[f"valid_kernel_{block_size}"] = vk

    def valid_kernel_callback(self, block_size: int) -> torch.Tensor:
        if not hasattr(self, f"valid_kernel_{block_size}"):
            self.compute_kernel_idx(block_size)
        return self[f"valid_kernel_{block_size}"]

    def valid_kernel_seg_callback(self, block_size: int) -> torch.Tensor:
        if not hasattr(self, f"valid_kernel_{block_size}"):
            self.compute_kernel_idx(block_size)
        return self[f"valid_kernel_seg_{block_size}"]

    # -- lazily completed fields -----------------------------------------------------------------
    def _ensure_tile_order(self):
        """Z-order-chunked, mask-sorted row order (private); needs the coordinates the cache was built from."""
        if hasattr(self, "_tile_order") or not hasattr(self, "_coords"):
            return
        self._ensure_sorted()
        if not hasattr(self, "_binary_code"):
            _, binary, _ = _codes_and_order(self["neighbor_map"], None, None)
            self["_binary_code"] = binary
        self["_tile_order"] = _locality_order(self["_coords"], self["_binary_code"], self["neighbor_map"].shape[1],
                                              getattr(self, "_grid", None))


    def _narrow_plan(self):
        """Plan of the resident-row gather GEMM for narrow layers (fgx_narrow_plan): chunks of 128 rows along a Z-order
        curve of the coordinates, per chunk the distinct source rows and the LDS slot of every (row, offset).  Needs the
        coordinates the cache was built from; made once and kept (it depends on the map and the coordinates alone)."""
        if not hasattr(self, "_narrow_plan_buf"):
            nmap = self["neighbor_map"]
            n, v = nmap.shape
            dev = nmap.device
            L = nat.lib()
            with torch.cuda.device(dev):
                order = torch.empty((n,), dtype=torch.int64, device=dev)
                ws = nat.workspace(L.fgx_locality_workspace_bytes(nat.sz(n)), dev)
                # the Z-order of the rows; the grid the cache was built for bounds the key bits that can differ
                bits, batch_bits = _grid_key_bits(self["_grid"])
                nat.check(L.fgx_zorder_rows(nat.ptr(self["_coords"]), nat.sz(n), C.c_int(bits), C.c_int(batch_bits), nat.ptr(order),
                                            nat.ptr(ws), nat.sz(ws.numel()), nat.stream()))
                plan = torch.empty((int(L.fgx_narrow_plan_bytes(nat.sz(n), C.c_int(v))),), dtype=torch.uint8, device=dev)
                nat.check(L.fgx_narrow_plan(nat.ptr(nmap), nat.ptr(order), nat.sz(n), C.c_int(v), C.c_int(1), nat.ptr(plan), nat.stream()))
            self["_narrow_plan_buf"] = plan
        return self["_narrow_plan_buf"]

    def _ensure_sorted(self):
        """gray_code / sorted_idx for a cache that only carries `neighbor_map`."""
        if hasattr(self, "gray_code") and hasattr(self, "sorted_idx"):
            return
        nmap = self["neighbor_map"]
        gray, _, order = _codes_and_order(nmap, None, None)
        self["gray_code"], self["sorted_idx"] = gray, order

    def _ensure_pairs(self):
        """valid_signal_* for a cache that was built without gradients."""
        if hasattr(self, "valid_signal_i") and hasattr(self, "valid_signal_o") and hasattr(self, "valid_signal_seg"):
            return
        self._ensure_sorted()
        self._attach_pairs(_pair_lists(self["neighbor_map"], self["gray_code"]))

    def _wgrad_bounds(self, block_rows: int):
        """First pair of every (offset, voxel block) for wgrad's blocks of `block_rows` rows: a function of the pair lists
        alone, so it is made once per block size and kept."""
        key = f"_wgrad_bounds_{block_rows}"
        if not hasattr(self, key):
            sig_o = self["valid_signal_o"]
            n, v = self["neighbor_map"].shape
            seg_host = self._seg_host()
            L = nat.lib()
            count = L.fgx_wgrad_block_bounds_count(nat.sz(n), C.c_int(v), C.c_int(block_rows))
            bounds = torch.empty((max(int(count), 1),), dtype=torch.uint32, device=sig_o.device)
            with torch.cuda.device(sig_o.device):
                nat.check(L.fgx_wgrad_block_bounds(nat.ptr(sig_o), (C.c_uint32 * (v + 1))(*seg_host), nat.sz(n), C.c_int(v),
                                                   C.c_int(block_rows), nat.ptr(bounds), nat.stream()))
            setattr(self, key, bounds)
        return getattr(self, key)

    def _wgrad_item_lists(self, block_rows: int, tile_rows: int, tile_cols: int, ci: int, co: int):
        """Balanced work lists of the streaming weight gradient (fgx_wgrad_item_lists) for one block size, tile shape and
        channel counts, made on the device from the block table and kept; None where the library has none for the shape."""
        key = f"_wgrad_lists_{block_rows}_{tile_rows}_{tile_cols}_{ci}_{co}"
        if not hasattr(self, key):
            bounds = self._wgrad_bounds(block_rows)
            n, v = self["neighbor_map"].shape
            L = nat.lib()
            lists = None
            with torch.cuda.device(bounds.device):
                words = int(L.fgx_wgrad_item_lists_count(nat.sz(n), C.c_int(v), C.c_int(ci), C.c_int(co), C.c_int(tile_rows),
                                                         C.c_int(tile_cols), C.c_int(block_rows)))
                if words > 0:
                    lists = torch.empty((words,), dtype=torch.uint32, device=bounds.device)
                    nat.check(L.fgx_wgrad_item_lists(nat.ptr(bounds), nat.sz(n), C.c_int(v), C.c_int(ci), C.c_int(co), C.c_int(tile_rows),
                                                     C.c_int(tile_cols), C.c_int(block_rows), nat.ptr(lists), nat.stream()))
            setattr(self, key, lists)
        return getattr(self, key)

    def _wgrad_sweep_plan(self, sub_rows: int):
        """Step lists of the paced wgrad sweep (fgx_wgrad_sweep_plan): a function of the pair lists and the sub-block
        size alone, made once and kept."""
        key = f"_wgrad_sweep_plan_{sub_rows}"
        if not hasattr(self, key):
            sig_o = self["valid_signal_o"]
            n, v = self["neighbor_map"].shape
            seg_host = self._seg_host()
            L = nat.lib()
            with torch.cuda.device(sig_o.device):
                nbytes = L.fgx_wgrad_sweep_plan_bytes(nat.sz(n), nat.sz(seg_host[-1]), C.c_int(v), C.c_int(sub_rows))
                plan = nat.workspace(nbytes, sig_o.device)
                nat.check(L.fgx_wgrad_sweep_plan(nat.ptr(sig_o), (C.c_uint32 * (v + 1))(*seg_host), nat.sz(n), C.c_int(v),
                                                 C.c_int(sub_rows), nat.ptr(plan), nat.sz(plan.numel()), nat.stream()))
            setattr(self, key, plan)
        return getattr(self, key)

    def _seg_host(self):
        if not hasattr(self, "_valid_signal_seg_host"):
            seg = self["valid_signal_seg"]
            self["_valid_signal_seg_host"] = [int(x) & 0xFFFFFFFF for x in seg.view(torch.int32).cpu().tolist()]
        return self["_valid_signal_seg_host"]


# ------------------------------------------------------------------------------------------------
# native helpers
# ------------------------------------------------------------------------------------------------
def _codes_and_order(nmap: torch.Tensor, gray: Optional[torch.Tensor], binary: Optional[torch.Tensor]):
    """(gray_code, binary_code, sorted_idx) from a neighbor map; gray/binary may come precomputed from the fused builder."""
    n, v = nmap.shape
    dev = nmap.device
    L = nat.lib()
    with torch.cuda.device(dev):
        if gray is None:
            gray = torch.empty((n,), dtype=torch.int32, device=dev)
            binary = torch.empty((n,), dtype=torch.int32, device=dev)
            nat.check(L.fgx_mask_codes(nat.ptr(nmap), nat.sz(n), C.c_int(v), nat.ptr(gray), nat.ptr(binary), nat.stream()))
        order = torch.empty((n,), dtype=torch.int64, device=dev)
        ws = nat.workspace(L.fgx_sort_workspace_bytes(nat.sz(n)), dev)
        nat.check(L.fgx_sort_by_code(nat.ptr(binary), nat.sz(n), C.c_int(v), nat.ptr(order), nat.ptr(ws),
                                     nat.sz(ws.numel()), nat.stream()))
    return gray, binary, order


# The kernels' private row order (Z-order chunks, mask-sorted inside a chunk) trades ~12 % more padded MFMA work for
# gathers that stay inside an XCD's L2.  It pays when rows are short, the pass is bandwidth bound and the voxels are many
# more than an L2 holds -- measured per forward pass at 32 / 64 channels: 4.1 M voxels 0.61 -> 0.54 / 1.07 -> 1.02 ms,
# 1.03 M 0.169 -> 0.143 / 0.275 -> 0.240, 578 k 0.109 -> 0.103 / 0.172 -> 0.168, 252 k 0.060 -> 0.065 / 0.092 -> 0.090,
# 64 k 0.049 -> 0.051 / 0.050 -> 0.053 -- and making it (two sorts and the tile tables of the new order) costs what seven to
# ten passes gain (0.50 ms at 4.1 M voxels, 0.24 at 1.03 M).  So a cache gets it once it has served LOCALITY_AFTER_CALLS
# short-row passes on the public order: whatever happens next, the detour then costs at most what those passes did.
LOCALITY_CHUNK_ROWS = 8192      # rows per spatial chunk
LOCALITY_MAX_ROW_BYTES = 128    # use the private order when a gathered row is at most this long
LOCALITY_MIN_ROWS = 786432      # ... and the map has this many rows or more
LOCALITY_AFTER_CALLS = 8        # ... and the cache has served this many such passes on the public order


def _locality_applies(cache, n: int, row_bytes: int) -> bool:
    """Whether a masked gather GEMM with rows of `row_bytes` walks the private row order of `cache` (see above).  An order
    that exists is used; none is made during a graph capture (the capture would hold the sorts)."""
    if row_bytes > LOCALITY_MAX_ROW_BYTES:
        return False
    if hasattr(cache, "_tile_order"):
        return True
    if n < LOCALITY_MIN_ROWS or not hasattr(cache, "_coords") or torch.cuda.is_current_stream_capturing():
        return False
    calls = getattr(cache, "_short_row_calls", 0) + 1
    cache["_short_row_calls"] = calls
    return calls > LOCALITY_AFTER_CALLS


def _grid_key_bits(grid) -> Tuple[int, int]:
    """(bits per axis, batch bits) a Z-order key needs for coordinates of `grid` = (batch size, spatial sizes); 16 and 16
    -- any coordinates -- when the grid is unknown or too large for less."""
    if grid is None:
        return 16, 16
    batch, spatial = grid
    bits = max(max(int(d) for d in spatial) - 1, 1).bit_length()
    batch_bits = max(int(batch) - 1, 0).bit_length()
    if bits > 16 or 3 * bits + batch_bits > 64:
        return 16, 16
    return bits, batch_bits


def _locality_order(coords: torch.Tensor, binary: torch.Tensor, v: int, grid=None) -> torch.Tensor:
    """Z-order chunks, mask-sorted inside each chunk (int64 permutation); `grid` = (batch size, spatial sizes) the
    coordinates lie in, when known: it bounds the key bits the sorts go over."""
    n = coords.shape[0]
    dev = coords.device
    order = torch.empty((n,), dtype=torch.int64, device=dev)
    L = nat.lib()
    bits, batch_bits = _grid_key_bits(grid)
    with torch.cuda.device(dev):
        ws = nat.workspace(L.fgx_locality_workspace_bytes(nat.sz(n)), dev)
        nat.check(L.fgx_locality_order_grid(nat.ptr(coords), nat.ptr(binary), nat.sz(n), C.c_int(v), C.c_int(LOCALITY_CHUNK_ROWS),
                                            C.c_int(bits), C.c_int(batch_bits), nat.ptr(order), nat.ptr(ws), nat.sz(ws.numel()),
                                            nat.stream()))
    return order


# pair lists up to this many bytes (both together, at their bound of one entry per slot of the map) are allocated before
# their length is known, which saves the build its wait for the host; larger ones wait and are allocated exactly
PAIR_LISTS_UNSIZED_MAX_BYTES = 1 << 30


def _pair_lists(nmap: torch.Tensor, gray: torch.Tensor, exact: bool = False):
    """The (input row, output row) lists per offset and their segment table (reference: migemm_neighmap_pp.cu:180-260).
    Returns {"seg", "sig_i", "sig_o", "seg_host"}, or {"seg", "pending"} when the lists were filled into buffers of the
    bound's size without waiting for their length (SubMConv3dNeighborCache._attach_pairs takes either); exact=True
    always waits and returns the finished lists."""
    n, v = nmap.shape
    dev = nmap.device
    L = nat.lib()
    with torch.cuda.device(dev):
        seg = torch.empty((v + 1,), dtype=torch.uint32, device=dev)
        ws = nat.workspace(L.fgx_pair_workspace_bytes(nat.sz(n), C.c_int(v)), dev)
        nat.check(L.fgx_pair_count(nat.ptr(gray), nat.sz(n), C.c_int(v), nat.ptr(seg), nat.ptr(ws), nat.sz(ws.numel()),
                                   nat.stream()))
        bound = n * v
        if not exact and 0 < bound * 8 <= PAIR_LISTS_UNSIZED_MAX_BYTES:
            seg_pinned = torch.empty((v + 1,), dtype=torch.int32, pin_memory=True)
            seg_pinned.copy_(seg.view(torch.int32), non_blocking=True)
            arrived = torch.cuda.Event()
            arrived.record()
            buf_i = torch.empty((bound,), dtype=torch.uint32, device=dev)
            buf_o = torch.empty((bound,), dtype=torch.uint32, device=dev)
            nat.check(L.fgx_pair_fill(nat.ptr(nmap), nat.ptr(gray), nat.sz(n), C.c_int(v), nat.ptr(ws), nat.ptr(buf_i),
                                      nat.ptr(buf_o), nat.stream()))
            return {"seg": seg, "pending": (buf_i, buf_o, seg_pinned, arrived)}
        seg_host = [x & 0xFFFFFFFF for x in seg.view(torch.int32).cpu().tolist()]   # a host sync: sizes L
        total = seg_host[-1]
        sig_i = torch.empty((total,), dtype=torch.uint32, device=dev)
        sig_o = torch.empty((total,), dtype=torch.uint32, device=dev)
        if total:
            nat.check(L.fgx_pair_fill(nat.ptr(nmap), nat.ptr(gray), nat.sz(n), C.c_int(v), nat.ptr(ws), nat.ptr(sig_i),
                                      nat.ptr(sig_o), nat.stream()))
    return {"seg": seg, "sig_i": sig_i, "sig_o": sig_o, "seg_host": seg_host}


SORT_DECIDED_ON_DEVICE_MAX = 1 << 21     # fgx_subm_neighbor_map_sorted honours presorted = 2 up to this many voxels

# The masked algorithms' cache through one library call (fgx_subm_cache_build) where it applies; False: step by step.
CACHE_BUILD_ONE_CALL = True
# from this many voxels on a training cache's pair lists are made on a second stream, beside the mask sort (below, the
# build waits for the host, and the second stream's events and context cost it 0.07 ms more: 42 608 voxels 0.149 -> 0.222 ms)
PAIR_LISTS_SIDE_STREAM_MIN_ROWS = 393216
_side_streams: dict = {}                 # device index -> that stream (default priority, made on first use)


def _side_stream(dev: torch.device) -> torch.cuda.Stream:
    key = dev.index if dev.index is not None else torch.cuda.current_device()
    if key not in _side_streams:
        _side_streams[key] = torch.cuda.Stream(device=dev)
    return _side_streams[key]


def _build_neighbor_map(coords: torch.Tensor, shape, kernel_size, dilation, with_codes: bool):
    n = coords.shape[0]
    B, _, W, H, D = [int(s) for s in shape]
    kw, kh, kd = [int(k) for k in kernel_size]
    v = kw * kh * kd
    dev = coords.device
    nmap = torch.empty((n, v), dtype=torch.uint32, device=dev)
    gray = binary = None
    if with_codes:
        gray = torch.empty((n,), dtype=torch.int32, device=dev)
        binary = torch.empty((n,), dtype=torch.int32, device=dev)
    builder = spconv.NEIGHBOR_MAP_BUILDER
    if builder == "auto":
        builder = "sort" if n * v >= spconv.SORT_BUILDER_MIN_PROBES else "hash"
    vol = B * W * H * D
    if builder == "sort" and kw * kh <= 128 and vol <= 2 ** 63:
        key_bits = 32 if vol <= 2 ** 32 else 64
        with torch.cuda.device(dev):
            L = nat.lib()
            # voxels that already come in scan order (a dense grid's nonzero(), a sorted voxelizer) need no key sort.  Up to
            # 2^21 voxels with 32-bit keys the library finds out on the device (presorted = 2) and nothing is read back;
            # beyond that a skipped sort is worth more than the wait: one pass over the coordinates and a 4-byte read-back
            presorted = 2
            if n > SORT_DECIDED_ON_DEVICE_MAX or key_bits != 32:
                descents = torch.zeros((1,), dtype=torch.int32, device=dev)
                nat.check(L.fgx_coords_key_order(nat.ptr(coords), nat.sz(n), C.c_int(W), C.c_int(H), C.c_int(D), nat.ptr(descents), nat.stream()))
                presorted = 1 if int(descents.item()) == 0 else 0
            ws = nat.workspace(L.fgx_subm_neighbor_map_sorted_workspace_bytes(nat.sz(n), C.c_int(key_bits), C.c_int(kw), C.c_int(kh)), dev)
            nat.check(L.fgx_subm_neighbor_map_sorted(
                nat.ptr(coords), nat.sz(n), C.c_int(B), C.c_int(W), C.c_int(H), C.c_int(D), C.c_int(kw), C.c_int(kh), C.c_int(kd),
                C.c_int(int(dilation[0])), C.c_int(int(dilation[1])), C.c_int(int(dilation[2])), C.c_int(key_bits),
                C.c_int(presorted),
                nat.ptr(ws), nat.sz(ws.numel()), nat.ptr(nmap), nat.ptr(gray), nat.ptr(binary), nat.stream()))
        return nmap, gray, binary
    table = int(spconv.HASHMAP_RATIO * n)
    if n > 0 and table < n:
        raise ValueError(f"hashmap ratio {spconv.HASHMAP_RATIO} gives a table smaller than the input")
    keys, vals = utils.init_hashmap(shape, table, dev)
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_subm_neighbor_map(
            nat.ptr(keys), C.c_int(32 if keys.dtype == torch.uint32 else 64), nat.ptr(vals), nat.sz(table),
            nat.ptr(coords), nat.sz(n), C.c_int(W), C.c_int(H), C.c_int(D), C.c_int(kw), C.c_int(kh), C.c_int(kd),
            C.c_int(int(dilation[0])), C.c_int(int(dilation[1])), C.c_int(int(dilation[2])),
            nat.ptr(nmap), nat.ptr(gray), nat.ptr(binary), nat.stream()))
    return nmap, gray, binary


def _build_cache_one_call(coords: torch.Tensor, shape, kernel_size, dilation, needs_grad: bool):
    """The masked algorithms' neighbor cache through fgx_subm_cache_build: map, codes, mask sort and (needs_grad) the pair
    lists enqueued by one library call, with every buffer allocated beforehand -- the GPU does not wait for the host
    between the steps.  Returns (nmap, gray, binary, order, pairs or None), or None where the call does not apply (the
    hash builder's range, kernels beyond what the sorted builder takes, pair lists too large to allocate at their bound)
    and the step-by-step path runs."""
    n = coords.shape[0]
    B, _, W, H, D = [int(s) for s in shape]
    kw, kh, kd = [int(k) for k in kernel_size]
    v = kw * kh * kd
    builder = spconv.NEIGHBOR_MAP_BUILDER
    if builder == "auto":
        builder = "sort" if n * v >= spconv.SORT_BUILDER_MIN_PROBES else "hash"
    vol = B * W * H * D
    bound = n * v
    if builder != "sort" or n == 0 or v > 32 or kw * kh > 128 or vol > 2 ** 63 or bound >= 0xFFFFFFFF:
        return None
    if needs_grad and bound * 8 > PAIR_LISTS_UNSIZED_MAX_BYTES:
        return None
    key_bits = 32 if vol <= 2 ** 32 else 64
    dev = coords.device
    with torch.cuda.device(dev):
        L = nat.lib()
        presorted = 2                       # (as in _build_neighbor_map)
        if n > SORT_DECIDED_ON_DEVICE_MAX or key_bits != 32:
            descents = torch.zeros((1,), dtype=torch.int32, device=dev)
            nat.check(L.fgx_coords_key_order(nat.ptr(coords), nat.sz(n), C.c_int(W), C.c_int(H), C.c_int(D), nat.ptr(descents), nat.stream()))
            presorted = 1 if int(descents.item()) == 0 else 0
        nmap = torch.empty((n, v), dtype=torch.uint32, device=dev)
        gray = torch.empty((n,), dtype=torch.int32, device=dev)
        binary = torch.empty((n,), dtype=torch.int32, device=dev)
        order = torch.empty((n,), dtype=torch.int64, device=dev)
        seg = buf_i = buf_o = None
        if needs_grad:
            seg = torch.empty((v + 1,), dtype=torch.uint32, device=dev)
            buf_i = torch.empty((bound,), dtype=torch.uint32, device=dev)
            buf_o = torch.empty((bound,), dtype=torch.uint32, device=dev)
        ws = nat.workspace(L.fgx_subm_cache_workspace_bytes(nat.sz(n), C.c_int(key_bits), C.c_int(kw), C.c_int(kh), C.c_int(kd),
                                                            C.c_int(1 if needs_grad else 0)), dev)
        nat.check(L.fgx_subm_cache_build(
            nat.ptr(coords), nat.sz(n), C.c_int(B), C.c_int(W), C.c_int(H), C.c_int(D), C.c_int(kw), C.c_int(kh), C.c_int(kd),
            C.c_int(int(dilation[0])), C.c_int(int(dilation[1])), C.c_int(int(dilation[2])), C.c_int(key_bits), C.c_int(presorted),
            C.c_int(1 if needs_grad else 0), nat.ptr(ws), nat.sz(ws.numel()), nat.ptr(nmap), nat.ptr(gray), nat.ptr(binary),
            nat.ptr(order), nat.ptr(seg), nat.ptr(buf_i), nat.ptr(buf_o), nat.stream()))
        pairs = None
        if needs_grad:
            # the lists' length travels to pinned host memory behind an event; the cache cuts them to it when first asked
            seg_pinned = torch.empty((v + 1,), dtype=torch.int32, pin_memory=True)
            seg_pinned.copy_(seg.view(torch.int32), non_blocking=True)
            arrived = torch.cuda.Event()
            arrived.record()
            pairs = {"seg": seg, "pending": (buf_i, buf_o, seg_pinned, arrived)}
    return nmap, gray, binary, order, pairs


def _pad_cols(t: torch.Tensor, mult: int) -> torch.Tensor:
    c = t.shape[-1]
    pad = (-c) % mult
    return t if pad == 0 else torch.nn.functional.pad(t, (0, pad))


_panel_bytes_kept = 0       # bytes of weight panels kept with their weights (all devices)
_pure_answers: dict = {}    # answers of the library's size / occupancy queries, which depend on their arguments alone


def _panel_nbytes(code: int, mode: int, ci: int, co: int, v: int, slab_bytes: int, tile_cols: int) -> int:
    key = ("panel", code, mode, ci, co, v, slab_bytes, tile_cols)
    if key not in _pure_answers:
        _pure_answers[key] = int(nat.lib().fgx_weight_panel_bytes(C.c_int(code), C.c_int(mode), C.c_int(ci), C.c_int(co), C.c_int(v),
                                                                   C.c_int(slab_bytes), C.c_int(tile_cols)))
    return _pure_answers[key]


def _stream_groups(code: int, cols: int, tile_rows: int, tile_cols: int, slab_bytes: int, dev: torch.device) -> int:
    key = ("groups", code, cols, tile_rows, tile_cols, slab_bytes, dev.index)
    if key not in _pure_answers:
        groups = C.c_int(0)
        nat.check(nat.lib().fgx_conv_gather_gemm_stream_groups(C.c_int(code), C.c_int(cols), C.c_int(tile_rows), C.c_int(tile_cols),
                                                               C.c_int(slab_bytes), C.byref(groups)))
        _pure_answers[key] = groups.value
    return _pure_answers[key]


def _release_panel_bytes(nbytes: int) -> None:
    global _panel_bytes_kept
    _panel_bytes_kept -= nbytes


_public_call = threading.local()


class _grad_mode_of_the_caller:
    """autograd runs Function.forward with grad mode off, so forward cannot see whether its caller stands under
    torch.no_grad() / inference_mode(); the public wrappers note it here (per thread) around apply().  Direct callers of
    apply() count as wanting gradients, like in the reference."""

    def __enter__(self):
        _public_call.grad_enabled = torch.is_grad_enabled()

    def __exit__(self, *exc):
        _public_call.grad_enabled = True
        return False


def _gradients_possible(ctx) -> bool:
    """Whether a backward pass can follow this forward: an argument wants a gradient and the caller records them."""
    return any(ctx.needs_input_grad) and getattr(_public_call, "grad_enabled", True)


def _weight_panel(owner: Optional[torch.Tensor], weight_cvk: torch.Tensor, code: int, mode: int, sched, dev) -> torch.Tensor:
    """The weight repacked for the gather GEMM of `mode` under schedule `sched`.  With spconv.WEIGHT_PANEL_CACHE and an
    `owner` (the caller's weight tensor, whose version counter and data pointer say whether it changed) the panel is
    kept on the owner from the second request at the same version and handed out without packing after that."""
    global _panel_bytes_kept
    co, v, ci = weight_cvk.shape
    L = nat.lib()
    nbytes = _panel_nbytes(code, mode, ci, co, v, int(sched.slab_bytes), int(sched.tile_cols))

    def pack(panel):
        nat.check(L.fgx_pack_weight(C.c_int(code), C.c_int(mode), nat.ptr(weight_cvk), C.c_int(ci), C.c_int(co), C.c_int(v),
                                    C.c_int(sched.slab_bytes), C.c_int(sched.tile_cols), nat.ptr(panel), nat.stream()))
        return panel

    # Under graph capture the pack kernel must be part of the graph: a kept panel read by the captured GEMMs would pin
    # the weights of the day of the capture, whatever the optimizer does to them between replays.
    if owner is None or not spconv.WEIGHT_PANEL_CACHE or torch.cuda.is_current_stream_capturing():
        return pack(nat.workspace(nbytes, dev))
    kept = owner.__dict__.setdefault("_fgx_weight_panels", {})
    key = (code, mode, ci, co, v, int(sched.slab_bytes), int(sched.tile_cols), str(dev))
    stamp = (owner._version, owner.data_ptr())
    entry = kept.get(key)
    if entry is not None and entry[0] == stamp:
        if entry[1] is not None:
            # (a panel packed on another stream is ordered like any other tensor: by the caller's stream semantics)
            return entry[1]
        if _panel_bytes_kept + nbytes <= spconv.WEIGHT_PANEL_CACHE_MAX_BYTES:
            panel = pack(nat.workspace(nbytes, dev))
            kept[key] = (stamp, panel)
            _panel_bytes_kept += panel.numel()
            weakref.finalize(panel, _release_panel_bytes, panel.numel())
            return panel
        return pack(nat.workspace(nbytes, dev))
    kept[key] = (stamp, None)           # first sight of this version (a stale panel, if any, is dropped here)
    return pack(nat.workspace(nbytes, dev))


def _gather_gemm(src: torch.Tensor, weight_cvk: torch.Tensor, bias: Optional[torch.Tensor], cache, mode: int,
                 allow_splitk: bool, masked: bool = True, weight_owner: Optional[torch.Tensor] = None,
                 activation: int = nat.ACT_NONE, relu_mask_out: Optional[list] = None) -> torch.Tensor:
    """mode 0: out = conv(src) with weight [Co, V, Ci] (+bias); mode 1: grad_input from src = grad_output through the
    same map with the offsets mirrored (submanifold); mode 2: grad_input through a map of its own, offsets as they
    are (generic sparse convolution).  The result has one row per row of cache["neighbor_map"]; src may have a
    different number of rows.  masked=False: the non-masked schedule (natural row order, all offsets per tile).
    weight_owner: the tensor the caller's weight lives in, for the optional panel cache (see _weight_panel).
    activation: nat.ACT_RELU clamps (sum + bias) at zero in the kernel's epilogue.  relu_mask_out: a list; where the kernels
    can (ReLU, 16-bit type, a multiple of 8 output columns) they also write one bit per output, "greater than zero", and
    the uint8 tensor [n * cols / 8] holding them is appended to the list."""
    co, v, ci = weight_cvk.shape
    n = cache["neighbor_map"].shape[0]
    n_src = src.shape[0]
    dt = src.dtype
    if dt not in nat.DTYPE_CODE:
        raise TypeError(f"unsupported feature dtype {dt}; expected float16, bfloat16 or float32")
    if weight_cvk.dtype != dt or (bias is not None and bias.dtype != dt):
        raise TypeError("features, weight and bias must share one dtype")
    k_true, cols = (ci, co) if mode == 0 else (co, ci)
    dev = src.device
    if n_src == 0:      # nothing to gather: the bias alone
        out = torch.zeros((n, cols), dtype=dt, device=dev)
        out = out if bias is None else out + bias
        return torch.relu(out) if activation == nat.ACT_RELU else out
    # rows must be whole 16-byte chunks: zero-pad the contraction dimension when they are not
    align = 16 // src.element_size()
    if k_true % align:
        src = _pad_cols(src, align)
        weight_owner = None             # the padded copy is made per call: nothing to key a kept panel on
        if mode == 0:
            weight_cvk = _pad_cols(weight_cvk, align)
        else:
            weight_cvk = torch.nn.functional.pad(weight_cvk, (0, 0, 0, 0, 0, (-co) % align))
        co, v, ci = weight_cvk.shape
    k = ci if mode == 0 else co
    src = src.contiguous()
    weight_cvk = weight_cvk.contiguous()
    if bias is not None:
        bias = bias.contiguous()        # the kernels read it with stride 1 (a view such as a column of a matrix has another)
    sched = nat.table_lookup(nat.PASS_FWD if mode == 0 else nat.PASS_DGRAD, dt, n, ci, co, v)
    splitk = sched.splitk if allow_splitk else 1
    if masked:
        cache._ensure_sorted()
    private = masked and _locality_applies(cache, n, k * src.element_size())
    out = torch.empty((n, cols), dtype=dt, device=dev)
    if n == 0:
        return out
    L = nat.lib()
    code = nat.DTYPE_CODE[dt]
    name = "gather_gemm_fwd" if mode == 0 else "gather_gemm_dgrad"
    mask = None
    if relu_mask_out is not None and activation == nat.ACT_RELU and src.element_size() == 2 and cols % 8 == 0:
        mask = torch.empty((n * cols // 8,), dtype=torch.uint8, device=dev)
        relu_mask_out.append(mask)
    with torch.cuda.device(dev):
        panel = _weight_panel(weight_owner, weight_cvk, code, mode, sched, dev)
        if _narrow_applies(cache, src, k, cols, v, n, n_src, sched):
            plan = cache._narrow_plan()
            nat.mark(name, "start")
            nat.check(L.fgx_conv_narrow_gemm(
                C.c_int(code), nat.ptr(src), nat.ptr(panel), nat.ptr(bias), nat.ptr(cache["neighbor_map"]), nat.ptr(plan),
                nat.sz(n), nat.sz(n_src), C.c_int(k), C.c_int(cols), C.c_int(v), C.c_int(activation), nat.ptr(out), nat.ptr(mask),
                nat.stream()))
            nat.mark(name, "stop")
            return out
        if sched.stream and _stream_fits(n, n_src, k * src.element_size()):
            order, tile_code, plan_seg, plan_idx, plan_band, plan_key = cache._gather_plan(sched.tile_rows, private,
                                                                                           dense=not masked)
            groups = _stream_groups(code, cols, int(sched.tile_rows), int(sched.tile_cols), int(sched.slab_bytes), dev)
            item_at = cache._item_order(plan_key, tile_code, -(-cols // sched.tile_cols), groups,
                                        -(-(k * src.element_size()) // sched.slab_bytes))
            nat.mark(name, "start")
            nat.check(L.fgx_conv_gather_gemm_stream_act_mask(
                C.c_int(code), nat.ptr(src), nat.ptr(panel), nat.ptr(bias), nat.ptr(order), nat.ptr(tile_code),
                nat.ptr(plan_seg), nat.ptr(plan_idx), nat.ptr(plan_band), nat.sz(plan_idx.shape[0]), nat.sz(n), nat.sz(n_src),
                C.c_int(k), C.c_int(cols), C.c_int(v),
                C.c_int(sched.tile_rows), C.c_int(sched.tile_cols), C.c_int(sched.slab_bytes), nat.ptr(item_at),
                C.c_int(groups), C.c_int(activation), nat.ptr(out), nat.ptr(mask), nat.stream()))
            nat.mark(name, "stop")
            return out
        if masked:
            order, tile_code, _ = cache._tile_tables(sched.tile_rows, private)
        else:
            order, tile_code = cache._dense_tile_tables(sched.tile_rows)
        scratch = None
        if splitk > 1:
            scratch = nat.workspace(L.fgx_conv_scratch_bytes(nat.sz(n), C.c_int(cols), C.c_int(splitk)), dev)
        nat.mark(name, "start")
        nat.check(L.fgx_conv_gather_gemm_act_mask(
            C.c_int(code), nat.ptr(src), nat.ptr(panel), nat.ptr(bias), nat.ptr(cache["neighbor_map"]),
            nat.ptr(order), nat.ptr(tile_code), nat.sz(n), C.c_int(k), C.c_int(cols), C.c_int(v),
            C.c_int(sched.tile_rows), C.c_int(sched.tile_cols), C.c_int(sched.slab_bytes), C.c_int(splitk),
            nat.ptr(scratch), C.c_int(activation), nat.ptr(out), nat.ptr(mask), nat.stream()))
        nat.mark(name, "stop")
    return out


def _relu_mask_apply(grad_output: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """grad_output where the forward pass's bit mask says the activated output was positive, zero elsewhere
    (fgx_relu_mask_apply: one pass that reads an eighth of a byte per element beside the gradient)."""
    g = grad_output.contiguous()
    out = torch.empty_like(g)
    with torch.cuda.device(g.device):
        nat.check(nat.lib().fgx_relu_mask_apply(C.c_int(nat.DTYPE_CODE[g.dtype]), nat.ptr(g), nat.ptr(mask), nat.sz(g.numel()),
                                                nat.ptr(out), nat.stream()))
    return out


def _narrow_applies(cache, src: torch.Tensor, k: int, cols: int, v: int, n: int, n_src: int, sched) -> bool:
    """Whether the resident-row kernel for narrow layers runs this gather GEMM (spconv.NARROW_RESIDENT): 16-bit rows of
    8 ... 32 channels on both sides, a panel of one 64-byte slab and 32 columns (what the schedule table picks for such
    layers), enough rows, coordinates to order the rows by, operands within its 32-bit offsets."""
    mode = spconv.NARROW_RESIDENT
    if mode == "off":
        return False
    if mode not in ("auto", "on"):
        raise ValueError(f"unknown NARROW_RESIDENT {mode!r}; expected 'auto', 'on' or 'off'")
    fits = (src.element_size() == 2 and 8 <= k <= 32 and k % 8 == 0 and 8 <= cols <= 32 and cols % 8 == 0 and v <= 27
            and int(sched.slab_bytes) == 64 and int(sched.tile_cols) == 32
            and getattr(cache, "_coords", None) is not None and cache._coords.shape[0] == n and n_src == n
            and n_src * k * 2 < 0xFF000000 and n * 82 + 10752 < 0xFF000000)
    if not fits:
        return False
    if hasattr(cache, "_narrow_plan_buf"):
        return True
    if torch.cuda.is_current_stream_capturing():
        return False                    # no plan is made inside a graph capture (it would be remade on every replay)
    if mode == "on":
        return True
    # "auto": the plan costs half of a neighbor-cache build (0.48 ms for 2.7 M voxels, 0.16 ms for 252 k) and a call
    # gains 0.2 - 0.3 ms on it at 2.7 M voxels (0.39 - 0.51 ms on the streaming kernel over the public row order, 0.195 ms
    # here) but 0.01 ms at 252 k, so a cache gets one once it has served what the plan costs in passes on the streaming
    # kernel -- NARROW_RESIDENT_AFTER_CALLS of them, NARROW_RESIDENT_AFTER_CALLS_SMALL below half a million rows:
    # whatever happens next, the detour then costs at most what the calls before it did.
    if n < NARROW_RESIDENT_MIN_ROWS:
        return False
    calls = getattr(cache, "_narrow_calls", 0) + 1
    cache["_narrow_calls"] = calls
    if n < NARROW_RESIDENT_TRAINING_MIN_ROWS:
        return calls > NARROW_RESIDENT_AFTER_CALLS_SMALL
    # A cache made for training also serves weight gradients, which gain three times what a forward pass does (0.66 ->
    # 0.26 ms at 2.67 M voxels): with half a million voxels and more its plan pays from the second layer on, so it comes
    # at the second product (a single layer never asks for one).
    eager = getattr(cache, "_needs_grad", False) and n >= NARROW_RESIDENT_TRAINING_MIN_ROWS
    return calls > (NARROW_RESIDENT_AFTER_CALLS_TRAINING if eager else NARROW_RESIDENT_AFTER_CALLS)


def _narrow_wgrad_applies(cache, f: torch.Tensor, ci: int, co: int, v: int, n: int, n_in: int) -> bool:
    """Whether the weight gradient runs on the resident-row kernel: a narrow 16-bit layer on a cache that has (mode "on":
    or can have) the plan, and no chunk of the plan has more distinct sources than slots (the plan's header says so;
    read back once per plan)."""
    mode = spconv.NARROW_RESIDENT
    if mode == "off":
        return False
    fits = (f.element_size() == 2 and 8 <= ci <= 32 and ci % 8 == 0 and 8 <= co <= 32 and co % 8 == 0 and v <= 27
            and n > 0                   # no rows, no plan: its header would be read before anything wrote it
            and getattr(cache, "_coords", None) is not None and cache._coords.shape[0] == n and n_in == n
            and n * 64 < 0xFF000000 and n * 82 + 10752 < 0xFF000000)
    if not fits or not (mode == "on" or hasattr(cache, "_narrow_plan_buf")):
        return False
    if not hasattr(cache, "_narrow_overflows"):
        if torch.cuda.is_current_stream_capturing():
            return False                # the header cannot be read back inside a graph capture
        cache["_narrow_overflows"] = int(cache._narrow_plan()[:4].view(torch.int32).item())
    return cache["_narrow_overflows"] == 0


def _stream_fits(n: int, n_src: int, row_bytes: int) -> bool:
    """The streaming kernel addresses its operands with 32-bit byte offsets."""
    return n_src * row_bytes <= 0xFF000000 and n * 8 <= 0xFF000000 and n * 27 * 4 * 2 <= 0xFF000000


def _sweep_fits(n: int, n_in: int, ci: int, co: int, elem_bytes: int, n_pairs: int) -> bool:
    """What fgx_conv_wgrad_sweep accepts: it multiplies row numbers with 24-bit multiplies and addresses both operands
    and the pair lists with 32-bit byte offsets below 0xFF000000 (the checks of the C entry point, restated)."""
    return (0 < n <= (1 << 24) and n_in <= (1 << 24) and n_pairs > 0
            and n * co * elem_bytes <= 0xFF000000 and n_in * ci * elem_bytes <= 0xFF000000
            and n_pairs * 4 + 256 <= 0xFF000000)


# Fewest rows from which NARROW_RESIDENT = "auto" takes the resident-row kernel.
NARROW_RESIDENT_MIN_ROWS = 32768
# ... and narrow products a neighbor cache serves on the streaming kernel before it gets the plan (below
# NARROW_RESIDENT_TRAINING_MIN_ROWS rows: the second number).
NARROW_RESIDENT_AFTER_CALLS = 3
NARROW_RESIDENT_AFTER_CALLS_SMALL = 16
# ... a cache made for training (it will serve weight gradients too) of this many rows and more: after one product.
NARROW_RESIDENT_TRAINING_MIN_ROWS = 524288
NARROW_RESIDENT_AFTER_CALLS_TRAINING = 1
# The gather GEMM's tiles are dealt by cost when there are more than this many rounds of items (tiles per persistent
# workgroup).
ITEM_ORDER_MIN_ROUNDS = 1
# ... for rows shorter than 512 bytes only up to this many rounds (beyond, the kernel's own order is even enough).
ITEM_ORDER_ANY_ROW_MAX_ROUNDS = 9
# The streaming weight gradient walks per-workgroup work lists balanced by pair count (fgx_wgrad_item_lists) where the
# library has them for the shape; False = the kernel's fixed interleave.  Same result bit for bit.
WGRAD_BALANCED_LISTS = True
# pacing of the wgrad sweep: sub-blocks a workgroup may run ahead of the slowest one of its XCD, and the looks at the
# others' progress after which it stops waiting (0 = no pacing, the default: the workgroups of an XCD stay close enough
# together by themselves, and waiting costs more time than the L2 misses it saves)
WGRAD_SWEEP_LEAD = 3
WGRAD_SWEEP_MAX_POLLS = 0


def _wgrad(grad_output: torch.Tensor, feats: torch.Tensor, cache, v: int, with_bias: bool = False, bias_offset: int = -1):
    """[Co, V, Ci] weight gradient from the pair lists of cache["neighbor_map"]: grad_output has one row per row of
    that map, feats one per row the map points at.  with_bias: also the bias gradient (column sums of grad_output),
    returned as a second value; bias_offset names an offset whose pairs hold every row of grad_output exactly once (the
    centre of a submanifold convolution), which lets the streaming kernel sum the rows it loads anyway."""
    n_in, ci = feats.shape
    n, co = grad_output.shape
    dt = feats.dtype
    dev = feats.device
    align = 16 // feats.element_size()
    f = _pad_cols(feats, align).contiguous()
    g = _pad_cols(grad_output, align).contiguous()
    cip, cop = f.shape[1], g.shape[1]
    if _narrow_wgrad_applies(cache, f, cip, cop, v, n, n_in):
        # narrow layers on a cache that has the resident-row plan: the chunk's rows gathered in LDS (fgx_conv_narrow_wgrad)
        L = nat.lib()
        gw = torch.empty((cop, v, cip), dtype=dt, device=dev)
        with torch.cuda.device(dev):
            scratch = nat.workspace(L.fgx_narrow_wgrad_scratch_bytes(C.c_int(v)), dev)
            nat.mark("wgrad", "start")
            nat.check(L.fgx_conv_narrow_wgrad(C.c_int(nat.DTYPE_CODE[dt]), nat.ptr(g), nat.ptr(f), nat.ptr(cache._narrow_plan()),
                                              nat.sz(n), nat.sz(n_in), C.c_int(cip), C.c_int(cop), C.c_int(v), nat.ptr(scratch),
                                              nat.ptr(gw), nat.stream()))
            gb = _colsum(g) if with_bias else None
            nat.mark("wgrad", "stop")
        if cip != ci or cop != co:
            gw = gw[:co, :, :ci].contiguous()
            gb = gb[:co].contiguous() if with_bias else None
        return (gw, gb) if with_bias else gw
    cache._ensure_pairs()
    seg_host = cache._seg_host()
    if len(seg_host) != v + 1 or seg_host[-1] > min(cache["valid_signal_i"].numel(), cache["valid_signal_o"].numel()):
        raise ValueError("valid_signal_seg does not fit the pair lists (V + 1 entries, the last one their length)")
    seg_arr = (C.c_uint32 * (v + 1))(*seg_host)
    sched = nat.table_lookup(nat.PASS_WGRAD, dt, n, cip, cop, v)
    gw = torch.empty((cop, v, cip), dtype=dt, device=dev)
    gb = torch.empty((cop,), dtype=dt, device=dev) if with_bias else None
    L = nat.lib()
    code = nat.DTYPE_CODE[dt]
    if sched.stream == 2 and not _sweep_fits(n, n_in, cip, cop, f.element_size(), seg_host[-1]):
        # very long operands (and empty pair lists) take the block-major kernel
        sched.stream, sched.block_rows = 1, 12288
    if sched.stream == 2:
        plan = cache._wgrad_sweep_plan(sched.block_rows)
        with torch.cuda.device(dev):
            scratch = nat.workspace(L.fgx_wgrad_sweep_scratch_bytes(C.c_int(cip), C.c_int(cop)), dev)
            nat.mark("wgrad", "start")
            nat.check(L.fgx_conv_wgrad_sweep(
                C.c_int(code), nat.ptr(g), nat.ptr(f), nat.ptr(cache["valid_signal_i"]), nat.ptr(cache["valid_signal_o"]),
                seg_arr, nat.ptr(plan), nat.sz(n), nat.sz(n_in), C.c_int(cip), C.c_int(cop), C.c_int(v), C.c_int(sched.tile_rows),
                C.c_int(sched.block_rows), C.c_int(WGRAD_SWEEP_LEAD), C.c_int(WGRAD_SWEEP_MAX_POLLS), nat.ptr(scratch), nat.ptr(gw),
                nat.ptr(gb), C.c_int(bias_offset), nat.stream()))
            nat.mark("wgrad", "stop")
        if cip != ci or cop != co:
            gw = gw[:co, :, :ci].contiguous()
            gb = gb[:co].contiguous() if with_bias else None
        return (gw, gb) if with_bias else gw
    bounds = cache._wgrad_bounds(sched.block_rows)
    lists = None
    if sched.stream == 1 and WGRAD_BALANCED_LISTS:
        lists = cache._wgrad_item_lists(sched.block_rows, sched.tile_rows, sched.tile_cols, cip, cop)
    with torch.cuda.device(dev):
        scratch = nat.workspace(L.fgx_wgrad_scratch_bytes(nat.sz(n), C.c_int(v), C.c_int(cip), C.c_int(cop),
                                                          C.c_int(sched.block_rows)), dev)
        nat.mark("wgrad", "start")
        nat.check(L.fgx_conv_wgrad_lists(
            C.c_int(code), nat.ptr(g), nat.ptr(f), nat.ptr(cache["valid_signal_i"]), nat.ptr(cache["valid_signal_o"]),
            seg_arr, nat.ptr(bounds), nat.ptr(lists), nat.sz(n), nat.sz(n_in), C.c_int(cip), C.c_int(cop), C.c_int(v), C.c_int(sched.tile_rows), C.c_int(sched.tile_cols),
            C.c_int(sched.block_rows), C.c_int(sched.stream), nat.ptr(scratch), nat.ptr(gw), nat.ptr(gb), C.c_int(bias_offset),
            nat.stream()))
        nat.mark("wgrad", "stop")
    if cip != ci or cop != co:
        gw = gw[:co, :, :ci].contiguous()
        gb = gb[:co].contiguous() if with_bias else None
    return (gw, gb) if with_bias else gw


def _colsum(grad_output: torch.Tensor) -> torch.Tensor:
    n, co = grad_output.shape
    out = torch.empty((co,), dtype=grad_output.dtype, device=grad_output.device)
    L = nat.lib()
    with torch.cuda.device(grad_output.device):
        scratch = nat.workspace(L.fgx_colsum_scratch_bytes(nat.sz(n), C.c_int(co)), grad_output.device)
        nat.check(L.fgx_colsum(C.c_int(nat.DTYPE_CODE[grad_output.dtype]), nat.ptr(grad_output), nat.sz(n), C.c_int(co),
                               nat.ptr(scratch), nat.ptr(out), nat.stream()))
    return out


def _gathered_rows(src: torch.Tensor, nmap: torch.Tensor) -> torch.Tensor:
    """[N, V*C] matrix whose (n, v) block is src[map[n, v]] or zeros (the explicit formulation's im2col)."""
    n, v = nmap.shape
    idx = nmap.view(torch.int32).to(torch.int64)
    idx = torch.where(idx < 0, torch.full_like(idx, src.shape[0]), idx)
    padded = torch.cat([src, src.new_zeros((1, src.shape[1]))], dim=0)
    return padded.index_select(0, idx.reshape(-1)).view(n, v * src.shape[1])


class SubMConv3dFunction(Function):
    @staticmethod
    def _compute_neighbor_cache(
        coords: torch.Tensor,
        shape: torch.Size,
        kernel_size: Tuple[int, int, int],
        dilation: Tuple[int, int, int],
        needs_grad: bool,
    ) -> SubMConv3dNeighborCache:
        """Build the neighbor tables for `coords` under the current algorithm
        (reference: submanifold_conv3d.py:46-107)."""
        assert coords.is_contiguous(), "Coords should be contiguous"
        assert coords.dtype in [torch.int32], "Unsupported coords dtype. Expect int32"
        algo = spconv.ALGORITHM
        if algo != Algorithm.EXPLICIT_GEMM and algo not in _IMPLICIT:
            raise ValueError(f"Unsupported algorithm {algo}")
        if not coords.is_cuda:
            raise NotImplementedError("CPU version of hashmap is not implemented")
        v = int(kernel_size[0]) * int(kernel_size[1]) * int(kernel_size[2])
        if algo == Algorithm.EXPLICIT_GEMM:
            nmap, _, _ = _build_neighbor_map(coords, shape, kernel_size, dilation, with_codes=False)
            return SubMConv3dNeighborCache(neighbor_map=nmap)
        assert v <= 32, "Currently, the max kernel volume is 32 because kernel mask is encoded as uint32"
        if algo not in _MASKED:
            # non-masked implicit GEMM: the cache is the map alone (reference: submanifold_conv3d.py:59-71); the
            # pair lists wgrad needs are derived from it on first use
            nmap, _, _ = _build_neighbor_map(coords, shape, kernel_size, dilation, with_codes=False)
            return SubMConv3dNeighborCache(neighbor_map=nmap)
        built = _build_cache_one_call(coords, shape, kernel_size, dilation, needs_grad) if CACHE_BUILD_ONE_CALL else None
        if built is not None:
            nmap, gray, binary, order, pairs = built
            cache = SubMConv3dNeighborCache(neighbor_map=nmap, gray_code=gray, sorted_idx=order)
            cache["_coords"] = coords
            cache["_needs_grad"] = bool(needs_grad)
            cache["_grid"] = (int(shape[0]), tuple(int(d) for d in shape[2:]))
            cache["_binary_code"] = binary
            if needs_grad:
                cache._attach_pairs(pairs)
            return cache
        nmap, gray, binary = _build_neighbor_map(coords, shape, kernel_size, dilation, with_codes=True)
        # The pair lists and the mask sort both start from the map and its codes and need nothing of each other: the lists
        # are made on a second stream while the sort runs on the caller's (both are chains of short kernels that leave
        # most of the chip idle: 0.065 + 0.089 ms one after the other at 669 288 voxels).
        pairs = None
        n = coords.shape[0]
        two_streams = needs_grad and n >= PAIR_LISTS_SIDE_STREAM_MIN_ROWS and not torch.cuda.is_current_stream_capturing()
        if two_streams:
            main = torch.cuda.current_stream(coords.device)
            map_made = torch.cuda.Event()
            map_made.record(main)
        gray, binary, order = _codes_and_order(nmap, gray, binary)      # (the longer of the two: enqueued first)
        if two_streams:
            side = _side_stream(coords.device)
            side.wait_event(map_made)
            with torch.cuda.stream(side):
                pairs = _pair_lists(nmap, gray)
            for t in (pairs["seg"],) + (pairs["pending"][:2] if "pending" in pairs else (pairs["sig_i"], pairs["sig_o"])):
                t.record_stream(main)       # allocated on the second stream, used on the caller's from here on
            main.wait_stream(side)
        cache = SubMConv3dNeighborCache(neighbor_map=nmap, gray_code=gray, sorted_idx=order)
        cache["_coords"] = coords           # for the private row order, built on first use by a short-row layer
        cache["_needs_grad"] = bool(needs_grad)
        cache["_grid"] = (int(shape[0]), tuple(int(d) for d in shape[2:]))
        cache["_binary_code"] = binary
        if needs_grad:
            cache._attach_pairs(pairs if pairs is not None else _pair_lists(nmap, gray))
        return cache

    @staticmethod
    def _compute_neighbor_cache_torch(
        coords: torch.Tensor,
        shape: torch.Size,
        kernel_size: Tuple[int, int, int],
        dilation: Tuple[int, int, int],
    ) -> SubMConv3dNeighborCache:
        """Hash-free builder in torch ops (any device): sort the flattened coordinates once and
        binary-search every shifted coordinate (reference: submanifold_conv3d.py:109-144; keys are
        int64 here, so the grid may exceed 2^31 cells)."""
        assert spconv.ALGORITHM == Algorithm.EXPLICIT_GEMM, "Only explicit_gemm is supported for torch implementation"
        _, _, W, H, D = [int(s) for s in shape]
        n = coords.shape[0]
        kw, kh, kd = [int(k) for k in kernel_size]
        c = coords.to(torch.int64)
        dev = coords.device
        keys = ((c[:, 0] * W + c[:, 1]) * H + c[:, 2]) * D + c[:, 3]
        skeys, order = torch.sort(keys)
        cols = []
        for i in range(kw):
            for j in range(kh):
                for k in range(kd):
                    x = c[:, 1] + (i - kw // 2) * int(dilation[0])
                    y = c[:, 2] + (j - kh // 2) * int(dilation[1])
                    z = c[:, 3] + (k - kd // 2) * int(dilation[2])
                    inside = (x >= 0) & (x < W) & (y >= 0) & (y < H) & (z >= 0) & (z < D)
                    q = ((c[:, 0] * W + x) * H + y) * D + z
                    col = torch.full((n,), EMPTY, dtype=torch.int64, device=dev)
                    if n:
                        pos = torch.searchsorted(skeys, q).clamp_(max=n - 1)
                        hit = inside & (skeys[pos] == q)
                        col[hit] = order[pos[hit]]
                    cols.append(col)
        nmap = torch.stack(cols, dim=1).to(torch.uint32) if cols else torch.empty((n, 0), dtype=torch.uint32, device=dev)
        return SubMConv3dNeighborCache(neighbor_map=nmap)

    @staticmethod
    def _sparse_submanifold_conv_forward(
        feats: torch.Tensor,
        neighbor_cache: SubMConv3dNeighborCache,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        relu: bool = False,
        relu_mask_out: Optional[list] = None,
    ) -> torch.Tensor:
        """relu (not in the reference): clamp the result at zero, in the GEMM's epilogue for the implicit algorithms.
        relu_mask_out: a list that receives the bit mask "output > 0" when the kernels wrote one (see _gather_gemm)."""
        assert feats.is_contiguous(), "Input features should be contiguous"
        assert feats.shape[0] == neighbor_cache["neighbor_map"].shape[0], \
            f"{feats.shape[0]} feature rows for a neighbor cache of {neighbor_cache['neighbor_map'].shape[0]} voxels"
        co, kw, kh, kd, ci = weight.shape
        v = kw * kh * kd
        algo = spconv.ALGORITHM
        if algo == Algorithm.EXPLICIT_GEMM:
            col = _gathered_rows(feats, neighbor_cache["neighbor_map"])
            w = weight.reshape(co, v * ci).t()
            out = torch.addmm(bias, col, w) if bias is not None else torch.mm(col, w)
            return torch.relu(out) if relu else out
        if algo in _IMPLICIT:
            _require_cuda(feats, "sparse_submanifold_conv3d")
            return _gather_gemm(feats, weight.reshape(co, v, ci), bias, neighbor_cache, 0, algo not in _NO_SPLITK,
                                masked=algo in _MASKED, weight_owner=weight,
                                activation=nat.ACT_RELU if relu else nat.ACT_NONE, relu_mask_out=relu_mask_out)
        raise ValueError(f"Unsupported algorithm {algo}")

    @staticmethod
    def _sparse_submanifold_conv_backward(
        grad_output: torch.Tensor,
        feats: torch.Tensor,
        neighbor_cache: SubMConv3dNeighborCache,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        weight_owner: Optional[torch.Tensor] = None,
    ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
        co, kw, kh, kd, ci = weight.shape
        v = kw * kh * kd
        algo = spconv.ALGORITHM
        n_rows = neighbor_cache["neighbor_map"].shape[0]
        assert feats.shape[0] == n_rows and grad_output.shape[0] == n_rows, \
            f"{feats.shape[0]} feature rows and {grad_output.shape[0]} gradient rows for a neighbor cache of {n_rows} voxels"
        grad_input = grad_weight = grad_bias = None
        if algo == Algorithm.EXPLICIT_GEMM:
            nmap = neighbor_cache["neighbor_map"]
            if feats.requires_grad:
                col = _gathered_rows(grad_output, torch.flip(nmap.view(torch.int32), [1]).view(torch.uint32))
                grad_input = torch.mm(col, weight.reshape(co, v, ci).transpose(0, 1).reshape(v * co, ci))
            if weight.requires_grad:
                col = _gathered_rows(feats.detach(), nmap)
                grad_weight = torch.mm(col.t(), grad_output).view(v, ci, co).permute(2, 0, 1).contiguous() \
                    .view(co, kw, kh, kd, ci)
            if bias is not None and bias.requires_grad:
                grad_bias = grad_output.sum(dim=0)
            return grad_input, grad_weight, grad_bias
        if algo in _IMPLICIT:
            _require_cuda(feats, "sparse_submanifold_conv3d backward")
            grad_output = grad_output.contiguous()
            if feats.requires_grad:
                grad_input = _gather_gemm(grad_output, weight.detach().reshape(co, v, ci), None, neighbor_cache, 1,
                                          algo not in _NO_SPLITK, masked=algo in _MASKED,
                                          weight_owner=weight if weight_owner is None else weight_owner)
            want_bias = bias is not None and bias.requires_grad
            if weight.requires_grad and want_bias:
                # odd kernel: the centre offset pairs every voxel with itself, so dbias rides along with wgrad
                centre = v // 2 if (kw % 2 and kh % 2 and kd % 2 and spconv.FUSE_DBIAS) else -1
                grad_weight, grad_bias = _wgrad(grad_output, feats.detach(), neighbor_cache, v, True, centre)
                grad_weight = grad_weight.reshape(co, kw, kh, kd, ci)
            elif weight.requires_grad:
                grad_weight = _wgrad(grad_output, feats.detach(), neighbor_cache, v).reshape(co, kw, kh, kd, ci)
            elif want_bias:
                grad_bias = _colsum(grad_output)
            return grad_input, grad_weight, grad_bias
        raise ValueError(f"Unsupported algorithm {algo}")

    @staticmethod
    def forward(
        ctx,
        feats: torch.Tensor,
        coords: torch.Tensor,
        shape: torch.Size,
        neighbor_cache: Optional[SubMConv3dNeighborCache],
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        dilation: Tuple[int, int, int] = (1, 1, 1),
        relu: bool = False,
    ) -> Tuple[torch.Tensor, SubMConv3dNeighborCache]:
        co, kw, kh, kd, ci = weight.shape
        assert feats.shape[-1] == ci, f"Input channels ({feats.shape[-1]}) should match weight channels ({ci})"
        need_grad = _gradients_possible(ctx)
        if neighbor_cache is None:
            neighbor_cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (kw, kh, kd), dilation, need_grad)
        masks = [] if (relu and need_grad and spconv.RELU_BIT_MASK) else None
        output = SubMConv3dFunction._sparse_submanifold_conv_forward(feats, neighbor_cache, weight, bias, relu=relu,
                                                                     relu_mask_out=masks)
        if relu and masks:
            ctx.save_for_backward(feats, weight, bias, masks[0])    # one bit per output: the activation's derivative
        elif relu:
            ctx.save_for_backward(feats, weight, bias, output)      # ... or the output itself, whose sign tells
        else:
            ctx.save_for_backward(feats, weight, bias)
        ctx.relu = relu
        ctx.relu_bits = bool(relu and masks)
        ctx.neighbor_cache = neighbor_cache
        ctx.weight_owner = weakref.ref(weight)      # the caller's tensor object: kept weight panels hang on it
        return output, neighbor_cache

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor, _):
        if ctx.relu and ctx.relu_bits:
            feats, weight, bias, mask = ctx.saved_tensors
            grad_output = _relu_mask_apply(grad_output, mask)
        elif ctx.relu:
            feats, weight, bias, output = ctx.saved_tensors
            grad_output = torch.where(output > 0, grad_output, torch.zeros((), dtype=grad_output.dtype, device=grad_output.device))
        else:
            feats, weight, bias = ctx.saved_tensors
        need_f, need_w, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[4], ctx.needs_input_grad[5]
        # the helper decides what to compute from requires_grad, as the reference does
        f = feats.detach().requires_grad_(need_f)
        w = weight.detach().requires_grad_(need_w)
        b = None if bias is None else bias.detach().requires_grad_(need_b)
        grad_input, grad_weight, grad_bias = SubMConv3dFunction._sparse_submanifold_conv_backward(
            grad_output, f, ctx.neighbor_cache, w, b, weight_owner=ctx.weight_owner())
        return grad_input, None, None, None, grad_weight, grad_bias, None, None


def sparse_submanifold_conv3d(
    feats: torch.Tensor,
    coords: torch.Tensor,
    shape: torch.Size,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    neighbor_cache: Optional[SubMConv3dNeighborCache] = None,
    dilation: Tuple[int, int, int] = (1, 1, 1),
) -> Tuple[torch.Tensor, SubMConv3dNeighborCache]:
    """
    Sparse submanifold convolution for 3D input.

    Args:
        feats (torch.Tensor): [N, C] tensor of input features.
        coords (torch.Tensor): [N, 4] int32 tensor of input coordinates (batch, x, y, z).
        shape (torch.Size): shape of the input tensor in NCWHD order.
        weight (torch.Tensor): [Co, Kw, Kh, Kd, Ci] tensor of weights.
        bias (Optional[torch.Tensor]): [Co] tensor of biases.
        neighbor_cache (Optional[SubMConv3dNeighborCache]): neighbor cache for this operation.
            Can be reused for multiple runs using the same coordinates; computed on the fly if None.
        dilation (Tuple[int, int, int]): dilation rate.

    Returns:
        (output [N, Co], neighbor_cache)
    """
    with _grad_mode_of_the_caller():
        return SubMConv3dFunction.apply(feats, coords, shape, neighbor_cache, weight, bias, dilation)


def sparse_submanifold_conv3d_relu(
    feats: torch.Tensor,
    coords: torch.Tensor,
    shape: torch.Size,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    neighbor_cache: Optional[SubMConv3dNeighborCache] = None,
    dilation: Tuple[int, int, int] = (1, 1, 1),
) -> Tuple[torch.Tensor, SubMConv3dNeighborCache]:
    """relu(sparse_submanifold_conv3d(...)) with the clamp done in the GEMM's epilogue: the output is written once,
    already activated (no counterpart in the reference; same arguments and return values as sparse_submanifold_conv3d).
    Differentiable: backward masks the incoming gradient with the sign of the saved output and runs the usual passes."""
    with _grad_mode_of_the_caller():
        return SubMConv3dFunction.apply(feats, coords, shape, neighbor_cache, weight, bias, dilation, True)
