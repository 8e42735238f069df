"""Generic sparse 3-D convolution (stride / padding / dilation, output coordinates of its own) on MI355X: host side.

Public surface and argument meaning follow the reference operator (flex_gemm/ops/spconv/sparse_conv3d.py):
`sparse_conv3d`, `SparseConv3dFunction` with its static helpers, and the attribute-bag
`SparseConv3dNeighborCache`.  Output coordinates and both neighbor maps come from gfx950 kernels behind the C ABI in
include/flexgemm_hip.h; the three GEMM passes are the submanifold operator's kernels, run over the forward map
(forward, weight gradient) and over the backward map (input gradient).
"""
from __future__ import annotations

import ctypes as C
import weakref
from typing import Optional, Tuple

import torch
from torch.autograd import Function

from ... import _native as nat
from .. import spconv, utils
from .. import serialize
from . import Algorithm, SerializationMode, SparseConv3dOutCoordAlgorithm
from .submanifold_conv3d import (EMPTY, _IMPLICIT, _MASKED, _NO_SPLITK, SubMConv3dNeighborCache, _codes_and_order, _colsum,
                                 _gather_gemm, _gathered_rows, _grad_mode_of_the_caller, _gradients_possible, _pair_lists,
                                 _relu_mask_apply, _require_cuda, _wgrad)


def _triple(x) -> Tuple[int, int, int]:
    a, b, c = [int(t) for t in x]
    return a, b, c


def _out_dims(shape, kernel_size, stride, padding, dilation) -> Tuple[int, int, int]:
    _, _, W, H, D = [int(s) for s in shape]
    return tuple((n + 2 * p - d * (k - 1) - 1) // s + 1
                 for n, k, s, p, d in zip((W, H, D), kernel_size, stride, padding, dilation))


class SparseConv3dNeighborCache(SubMConv3dNeighborCache):
    """Neighbor tables of one (input coordinates, output coordinates, geometry) triple.

    Fields (reference: sparse_conv3d.py:159-218): `neighbor_map` uint32 [L, V] (output row -> input rows),
    `neighbor_map_bwd` uint32 [M, V] (input row -> output rows; None without gradients); for the masked algorithms
    also `gray_code`, `sorted_idx` of the forward map, the pair lists `valid_signal_*` when gradients are needed, and
    `gray_code_bwd`, `sorted_idx_bwd` of the backward map when its masks are irregular (stride > 1 or output
    coordinates given by the caller).  A missing field reads as None, as in the reference (:14-15)."""

    def __getitem__(self, key):
        return getattr(self, key, None)

    def _bwd_view(self) -> SubMConv3dNeighborCache:
        """The backward map seen as a cache of its own (rows = input voxels), which is what the GEMM host code walks."""
        if not hasattr(self, "_bwd"):
            if getattr(self, "neighbor_map_bwd", None) is None:
                raise RuntimeError("this neighbor cache was built without gradients (needs_grad=False): "
                                   "it has no backward map")
            view = SubMConv3dNeighborCache(neighbor_map=self.neighbor_map_bwd)
            if hasattr(self, "gray_code_bwd") and hasattr(self, "sorted_idx_bwd"):
                view["gray_code"] = self.gray_code_bwd
                view["sorted_idx"] = self.sorted_idx_bwd
            self._bwd = view
        return self._bwd

    def compute_kernel_idx_bwd(self, block_size: int):
        """`valid_kernel_bwd_{B}` / `valid_kernel_bwd_seg_{B}` of the mask-sorted backward map
        (reference: sparse_conv3d.py:43-46)."""
        view = self._bwd_view()
        view._ensure_sorted()
        view.compute_kernel_idx(block_size)
        self[f"valid_kernel_bwd_{block_size}"] = view[f"valid_kernel_{block_size}"]
        self[f"valid_kernel_bwd_seg_{block_size}"] = view[f"valid_kernel_seg_{block_size}"]

    def valid_kernel_bwd_callback(self, block_size: int) -> torch.Tensor:
        if not hasattr(self, f"valid_kernel_bwd_{block_size}"):
            self.compute_kernel_idx_bwd(block_size)
        return self[f"valid_kernel_bwd_{block_size}"]

    def valid_kernel_bwd_seg_callback(self, block_size: int) -> torch.Tensor:
        if not hasattr(self, f"valid_kernel_bwd_seg_{block_size}"):
            self.compute_kernel_idx_bwd(block_size)
        return self[f"valid_kernel_bwd_seg_{block_size}"]


def _build_maps(coords: torch.Tensor, out_coords: torch.Tensor, shape, kernel_size, stride, padding, dilation,
                with_bwd: bool, with_codes: bool, hashmap_ratio: Optional[float] = None):
    """(map_fwd [L, V], map_bwd [M, V] | None, gray | None, binary | None), by hash probes or by sort and merge.
    hashmap_ratio: table slots per input voxel for the hash builder (default: spconv.HASHMAP_RATIO)."""
    ratio = spconv.HASHMAP_RATIO if hashmap_ratio is None else float(hashmap_ratio)
    m, l = coords.shape[0], out_coords.shape[0]
    _, _, W, H, D = [int(s) for s in shape]
    kw, kh, kd = kernel_size
    v = kw * kh * kd
    dev = coords.device
    nmap = torch.empty((l, v), dtype=torch.uint32, device=dev)
    nmap_bwd = torch.empty((m, v), dtype=torch.uint32, device=dev) if with_bwd else None
    gray = binary = None
    if with_codes:
        gray = torch.empty((l,), dtype=torch.int32, device=dev)
        binary = torch.empty((l,), dtype=torch.int32, device=dev)
    B = int(shape[0])
    builder = spconv.NEIGHBOR_MAP_BUILDER
    if builder == "auto":
        # (the generic builder sorts the queries as well, with wider keys: it needs more questions to pay off)
        builder = "sort" if l * v >= 4 * spconv.SORT_BUILDER_MIN_PROBES else "hash"
    vol = B * W * H * D
    geom = [C.c_int(x) for x in (kw, kh, kd, stride[0], stride[1], stride[2], padding[0], padding[1], padding[2],
                                 dilation[0], dilation[1], dilation[2])]
    if builder == "sort" and kw * kh <= 128 and vol <= 2 ** 62:
        key_bits = 32 if vol <= 2 ** 32 else 64
        with torch.cuda.device(dev):
            L = nat.lib()
            ws = nat.workspace(L.fgx_spconv_neighbor_map_sorted_workspace_bytes(nat.sz(m), nat.sz(l), C.c_int(key_bits),
                                                                                 C.c_int(kw), C.c_int(kh)), dev)
            nat.check(L.fgx_spconv_neighbor_map_sorted(
                nat.ptr(coords), nat.sz(m), nat.ptr(out_coords), nat.sz(l), C.c_int(B), C.c_int(W), C.c_int(H), C.c_int(D), *geom,
                C.c_int(key_bits), nat.ptr(ws), nat.sz(ws.numel()), nat.ptr(nmap), nat.ptr(nmap_bwd), nat.ptr(gray), nat.ptr(binary),
                nat.stream()))
        return nmap, nmap_bwd, gray, binary
    table = int(ratio * m)
    if m > 0 and table < m:
        raise ValueError(f"hashmap ratio {ratio} gives a table smaller than the input")
    keys = vals = None
    key_bits = 32
    with torch.cuda.device(dev):
        L = nat.lib()
        if m > 0:
            keys, vals = utils.init_hashmap(shape, table, dev)
            key_bits = 32 if keys.dtype == torch.uint32 else 64
            nat.check(L.fgx_hash_insert_3d_idx_as_val(nat.ptr(keys), C.c_int(key_bits), nat.ptr(vals), C.c_int(32),
                                                      nat.sz(table), nat.ptr(coords), nat.sz(m), C.c_int(W), C.c_int(H),
                                                      C.c_int(D), nat.stream()))
        nat.check(L.fgx_spconv_neighbor_map(
            nat.ptr(keys), C.c_int(key_bits), nat.ptr(vals), nat.sz(table), nat.ptr(out_coords), nat.sz(l), nat.sz(m),
            C.c_int(W), C.c_int(H), C.c_int(D), *geom,
            nat.ptr(nmap), nat.ptr(nmap_bwd), nat.ptr(gray), nat.ptr(binary), nat.stream()))
    return nmap, nmap_bwd, gray, binary


class SparseConv3dFunction(Function):
    @staticmethod
    def _get_output_coords(
        coords: torch.Tensor,
        shape: torch.Size,
        kernel_size: Tuple[int, int, int],
        stride: Tuple[int, int, int],
        padding: Tuple[int, int, int],
        dilation: Tuple[int, int, int],
        serialization_mode: Optional[int] = None,
    ) -> torch.Tensor:
        """int32 [L, 4] output coordinates (reference: sparse_conv3d.py:60-94), sorted by (b, x, y, z) under
        SerializationMode.BXYZ, along the z-order or Hilbert curve under the other two modes.

        Both of the reference's OUT_COORD_ALGO values name the same result; on gfx950 one streaming pass (candidate
        keys, radix sort, unique) serves both.  The curve modes re-sort the unique coordinates by their code; the bits
        per axis come from the INPUT grid, as in the reference (sparse_neighbor_map.cu:157-160), which fixes the
        orientation of the Hilbert curve.  serialization_mode overrides spconv.SERIALIZATION_MODE for this call."""
        mode = spconv.SERIALIZATION_MODE if serialization_mode is None else serialization_mode
        assert coords.is_contiguous(), "Coords should be contiguous"
        assert coords.dtype in [torch.int32], "Unsupported coords dtype. Expect int32"
        if not coords.is_cuda:
            raise NotImplementedError("CPU version is not implemented")
        if spconv.OUT_COORD_ALGO not in (SparseConv3dOutCoordAlgorithm.HASHMAP, SparseConv3dOutCoordAlgorithm.EXPAND_UNIQUE):
            raise ValueError(f"Unsupported output-coordinate algorithm {spconv.OUT_COORD_ALGO}")
        if mode not in (SerializationMode.BXYZ, SerializationMode.Z_ORDER, SerializationMode.HILBERT):
            raise ValueError("Unsupported serialize mode.")
        B, _, W, H, D = [int(s) for s in shape]
        ks, st, pd, dl = _triple(kernel_size), _triple(stride), _triple(padding), _triple(dilation)
        wo, ho, do = _out_dims(shape, ks, st, pd, dl)
        m = coords.shape[0]
        dev = coords.device
        if m == 0 or min(wo, ho, do) <= 0:
            return torch.empty((0, 4), dtype=torch.int32, device=dev)
        v = ks[0] * ks[1] * ks[2]
        vol = B * wo * ho * do
        if vol >= 2 ** 64 - 1:
            raise ValueError("The spatial size is too large. Require B*W*H*D < 2^64.")
        key_bits = 32 if vol < 2 ** 32 - 1 else 64
        L = nat.lib()
        with torch.cuda.device(dev):
            ws = nat.workspace(L.fgx_spconv_out_coords_workspace_bytes(nat.sz(m), C.c_int(v), C.c_int(key_bits)), dev)
            count = torch.empty((1,), dtype=torch.int64, device=dev)
            nat.check(L.fgx_spconv_out_coords_keys(
                nat.ptr(coords), nat.sz(m), C.c_int(B), C.c_int(W), C.c_int(H), C.c_int(D),
                C.c_int(ks[0]), C.c_int(ks[1]), C.c_int(ks[2]), C.c_int(st[0]), C.c_int(st[1]), C.c_int(st[2]),
                C.c_int(pd[0]), C.c_int(pd[1]), C.c_int(pd[2]), C.c_int(dl[0]), C.c_int(dl[1]), C.c_int(dl[2]),
                C.c_int(key_bits), nat.ptr(ws), nat.sz(ws.numel()), nat.ptr(count), nat.stream()))
            total = int(count.item())          # the one host sync: sizes the result
            out = torch.empty((total, 4), dtype=torch.int32, device=dev)
            nat.check(L.fgx_spconv_out_coords_decode(nat.ptr(ws), C.c_int(key_bits), nat.sz(total), C.c_int(wo), C.c_int(ho),
                                                     C.c_int(do), nat.ptr(out), nat.stream()))
        if mode != SerializationMode.BXYZ:
            bit_length = (max(W, H, D) - 1).bit_length()
            if max(wo, ho, do) > (1 << bit_length):
                raise ValueError("output grid exceeds the bits per axis of the input grid: curve codes would collide")
            out = serialize.reorder_coords(out, bit_length, (B - 1).bit_length(), int(mode))
        return out

    @staticmethod
    def _get_output_coords_torch(
        coords: torch.Tensor,
        shape: torch.Size,
        kernel_size: Tuple[int, int, int],
        stride: Tuple[int, int, int],
        padding: Tuple[int, int, int],
        dilation: Tuple[int, int, int],
    ) -> torch.Tensor:
        """The same list in torch ops on any device (reference: sparse_conv3d.py:96-127): every (voxel, kernel position)
        candidate, filtered, then torch.unique over rows."""
        ks, st, pd, dl = _triple(kernel_size), _triple(stride), _triple(padding), _triple(dilation)
        dims = _out_dims(shape, ks, st, pd, dl)
        dev = coords.device
        grid = torch.stack(torch.meshgrid(torch.arange(ks[0]), torch.arange(ks[1]), torch.arange(ks[2]), indexing="ij"), -1)
        k = grid.reshape(-1, 3).to(dev).long()
        c = coords.long()
        cand = c[:, None, 1:] + torch.tensor(pd, device=dev) - k[None] * torch.tensor(dl, device=dev)
        s = torch.tensor(st, device=dev)
        ok = (cand % s == 0).all(-1)
        q = torch.div(cand, s, rounding_mode="floor")
        ok &= ((q >= 0) & (q < torch.tensor(dims, device=dev))).all(-1)
        rows = torch.cat([c[:, None, :1].expand(-1, k.shape[0], -1), q], -1)[ok]
        if rows.shape[0] == 0:
            return torch.empty((0, 4), dtype=torch.int32, device=dev)
        return torch.unique(rows, dim=0).int()

    @staticmethod
    def _compute_neighbor_cache(
        coords: torch.Tensor,
        out_coords: torch.Tensor,
        shape: torch.Size,
        kernel_size: Tuple[int, int, int],
        stride: Tuple[int, int, int],
        padding: Tuple[int, int, int],
        dilation: Tuple[int, int, int],
        needs_grad: bool,
        is_out_coords_given: bool = False,
    ) -> SparseConv3dNeighborCache:
        """Build the neighbor tables under the current algorithm (reference: sparse_conv3d.py:130-222)."""
        assert coords.is_contiguous(), "Coords should be contiguous"
        assert coords.dtype in [torch.int32], "Unsupported coords dtype. Expect int32"
        algo = spconv.ALGORITHM
        if algo != Algorithm.EXPLICIT_GEMM and algo not in _IMPLICIT:
            raise ValueError(f"Unsupported algorithm {algo}")
        if not coords.is_cuda:
            raise NotImplementedError("CPU version of hashmap is not implemented")
        assert out_coords.is_cuda and out_coords.dtype == torch.int32, "Output coords should be an int32 tensor on the GPU"
        out_coords = out_coords.contiguous()
        ks, st, pd, dl = _triple(kernel_size), _triple(stride), _triple(padding), _triple(dilation)
        v = ks[0] * ks[1] * ks[2]
        if algo not in _MASKED:
            nmap, nmap_bwd, _, _ = _build_maps(coords, out_coords, shape, ks, st, pd, dl, needs_grad, with_codes=False)
            return SparseConv3dNeighborCache(neighbor_map=nmap, neighbor_map_bwd=nmap_bwd, _n_in=coords.shape[0])
        assert v <= 32, "Currently, the max kernel volume is 32 because kernel mask is encoded as uint32"
        nmap, nmap_bwd, gray, binary = _build_maps(coords, out_coords, shape, ks, st, pd, dl, needs_grad, with_codes=True)
        gray, binary, order = _codes_and_order(nmap, gray, binary)
        cache = SparseConv3dNeighborCache(neighbor_map=nmap, neighbor_map_bwd=nmap_bwd, gray_code=gray, sorted_idx=order,
                                          _n_in=coords.shape[0])
        if needs_grad:
            cache._attach_pairs(_pair_lists(nmap, gray))
            if any(s != 1 for s in st) or is_out_coords_given:
                # irregular backward masks: sort the input rows by theirs, as the reference does (:191-207); otherwise
                # nearly every input reaches every kernel position and the input gradient runs unsorted
                gray_b, _, order_b = _codes_and_order(nmap_bwd, None, None)
                cache["gray_code_bwd"] = gray_b
                cache["sorted_idx_bwd"] = order_b
        return cache

    @staticmethod
    def _compute_neighbor_cache_torch(
        coords: torch.Tensor,
        out_coords: torch.Tensor,
        shape: torch.Size,
        kernel_size: Tuple[int, int, int],
        stride: Tuple[int, int, int],
        padding: Tuple[int, int, int],
        dilation: Tuple[int, int, int],
        needs_grad: bool,
    ) -> SparseConv3dNeighborCache:
        """Hash-free builder in torch ops on any device: sort the flattened input coordinates once and binary-search
        every probed cell (reference: sparse_conv3d.py:224-278; keys are int64 here)."""
        assert spconv.ALGORITHM == Algorithm.EXPLICIT_GEMM, "Only explicit_gemm is supported for torch implementation"
        _, _, W, H, D = [int(s) for s in shape]
        ks, st, pd, dl = _triple(kernel_size), _triple(stride), _triple(padding), _triple(dilation)
        m, l = coords.shape[0], out_coords.shape[0]
        v = ks[0] * ks[1] * ks[2]
        dev = coords.device
        c = coords.long()
        o = out_coords.long()
        keys = ((c[:, 0] * W + c[:, 1]) * H + c[:, 2]) * D + c[:, 3]
        skeys, order = torch.sort(keys)
        fwd = torch.full((l, v), EMPTY, dtype=torch.int64, device=dev)
        bwd = torch.full((m, v), EMPTY, dtype=torch.int64, device=dev) if needs_grad else None
        if m and l:
            rows = torch.arange(l, device=dev)
            for j in range(v):
                kx, ky, kz = j // (ks[1] * ks[2]), j // ks[2] % ks[1], j % ks[2]
                x = o[:, 1] * st[0] - pd[0] + kx * dl[0]
                y = o[:, 2] * st[1] - pd[1] + ky * dl[1]
                z = o[:, 3] * st[2] - pd[2] + kz * dl[2]
                inside = (x >= 0) & (x < W) & (y >= 0) & (y < H) & (z >= 0) & (z < D)
                q = ((o[:, 0] * W + x) * H + y) * D + z
                pos = torch.searchsorted(skeys, q).clamp_(max=m - 1)
                hit = inside & (skeys[pos] == q)
                src = order[pos[hit]]
                fwd[hit, j] = src
                if needs_grad:
                    bwd[src, j] = rows[hit]
        return SparseConv3dNeighborCache(neighbor_map=fwd.to(torch.uint32),
                                         neighbor_map_bwd=bwd.to(torch.uint32) if needs_grad else None)

    @staticmethod
    def _sparse_conv_forward(
        feats: torch.Tensor,
        neighbor_cache: SparseConv3dNeighborCache,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        relu: bool = False,
        relu_mask_out: Optional[list] = None,
    ) -> torch.Tensor:
        """relu (not in the reference): clamp the result at zero, in the GEMM's epilogue for the implicit algorithms.
        relu_mask_out: a list that receives the bit mask "output > 0" when the kernels wrote one (see _gather_gemm)."""
        assert feats.is_contiguous(), "Input features should be contiguous"
        n_in = neighbor_cache["_n_in"]          # input voxels the maps were built for (absent on a hand-made cache)
        if n_in is None and neighbor_cache["neighbor_map_bwd"] is not None:
            n_in = neighbor_cache["neighbor_map_bwd"].shape[0]
        assert n_in is None or feats.shape[0] == n_in, f"{feats.shape[0]} feature rows for a neighbor cache of {n_in} input voxels"
        co, kw, kh, kd, ci = weight.shape
        v = kw * kh * kd
        algo = spconv.ALGORITHM
        if algo == Algorithm.EXPLICIT_GEMM:
            col = _gathered_rows(feats, neighbor_cache["neighbor_map"])
            w = weight.reshape(co, v * ci).t()
            out = torch.addmm(bias, col, w) if bias is not None else torch.mm(col, w)
            return torch.relu(out) if relu else out
        if algo in _IMPLICIT:
            _require_cuda(feats, "sparse_conv3d")
            return _gather_gemm(feats, weight.reshape(co, v, ci), bias, neighbor_cache, 0, algo not in _NO_SPLITK,
                                masked=algo in _MASKED, weight_owner=weight,
                                activation=nat.ACT_RELU if relu else nat.ACT_NONE, relu_mask_out=relu_mask_out)
        raise ValueError(f"Unsupported algorithm {algo}")

    @staticmethod
    def _sparse_conv_backward(
        grad_output: torch.Tensor,
        feats: torch.Tensor,
        neighbor_cache: SparseConv3dNeighborCache,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        weight_owner: Optional[torch.Tensor] = None,
    ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
        co, kw, kh, kd, ci = weight.shape
        v = kw * kh * kd
        algo = spconv.ALGORITHM
        assert grad_output.shape[0] == neighbor_cache["neighbor_map"].shape[0], \
            f"{grad_output.shape[0]} gradient rows for a neighbor cache of {neighbor_cache['neighbor_map'].shape[0]} output voxels"
        if neighbor_cache["neighbor_map_bwd"] is not None:
            assert feats.shape[0] == neighbor_cache["neighbor_map_bwd"].shape[0], \
                f"{feats.shape[0]} feature rows for a neighbor cache of {neighbor_cache['neighbor_map_bwd'].shape[0]} input voxels"
        grad_input = grad_weight = grad_bias = None
        if algo == Algorithm.EXPLICIT_GEMM:
            if feats.requires_grad:
                col = _gathered_rows(grad_output, neighbor_cache["neighbor_map_bwd"])
                grad_input = torch.mm(col, weight.reshape(co, v, ci).transpose(0, 1).reshape(v * co, ci))
            if weight.requires_grad:
                col = _gathered_rows(feats.detach(), neighbor_cache["neighbor_map"])
                grad_weight = torch.mm(col.t(), grad_output).view(v, ci, co).permute(2, 0, 1).contiguous() \
                    .view(co, kw, kh, kd, ci)
            if bias is not None and bias.requires_grad:
                grad_bias = grad_output.sum(dim=0)
            return grad_input, grad_weight, grad_bias
        if algo in _IMPLICIT:
            _require_cuda(feats, "sparse_conv3d backward")
            grad_output = grad_output.contiguous()
            if feats.requires_grad:
                view = neighbor_cache._bwd_view()
                # mask-sorted walk only where the cache carries the backward order (reference: sparse_conv3d.py:191-207)
                masked = algo in _MASKED and hasattr(view, "sorted_idx")
                grad_input = _gather_gemm(grad_output, weight.detach().reshape(co, v, ci), None, view, 2,
                                          algo not in _NO_SPLITK, masked=masked,
                                          weight_owner=weight if weight_owner is None else weight_owner)
            if weight.requires_grad:
                grad_weight = _wgrad(grad_output, feats.detach(), neighbor_cache, v).reshape(co, kw, kh, kd, ci)
            if bias is not None and bias.requires_grad:
                grad_bias = _colsum(grad_output)
            return grad_input, grad_weight, grad_bias
        raise ValueError(f"Unsupported algorithm {algo}")

    @staticmethod
    def forward(
        ctx,
        feats: torch.Tensor,
        coords: torch.Tensor,
        shape: torch.Size,
        neighbor_cache: Optional[SparseConv3dNeighborCache],
        weight: torch.Tensor,
        bias: Optional[torch.Tensor] = None,
        out_coords: Optional[torch.Tensor] = None,
        stride: Tuple[int, int, int] = (1, 1, 1),
        padding: Tuple[int, int, int] = (0, 0, 0),
        dilation: Tuple[int, int, int] = (1, 1, 1),
        relu: bool = False,
    ):
        co, kw, kh, kd, ci = weight.shape
        assert feats.shape[-1] == ci, f"Input channels ({feats.shape[-1]}) should match weight channels ({ci})"
        need_grad = _gradients_possible(ctx)
        given = out_coords is not None
        if out_coords is None:
            out_coords = SparseConv3dFunction._get_output_coords(coords, shape, (kw, kh, kd), stride, padding, dilation)
        if neighbor_cache is None:
            neighbor_cache = SparseConv3dFunction._compute_neighbor_cache(coords, out_coords, shape, (kw, kh, kd), stride,
                                                                          padding, dilation, need_grad, given)
        masks = [] if (relu and need_grad and spconv.RELU_BIT_MASK) else None
        output = SparseConv3dFunction._sparse_conv_forward(feats, neighbor_cache, weight, bias, relu=relu, relu_mask_out=masks)
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
        ctx.mark_non_differentiable(out_coords)
        return output, out_coords, neighbor_cache

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor, _, __):
        if ctx.relu and ctx.relu_bits:
            feats, weight, bias, mask = ctx.saved_tensors
            grad_output = _relu_mask_apply(grad_output, mask)
        elif ctx.relu:
            feats, weight, bias, output = ctx.saved_tensors
            grad_output = torch.where(output > 0, grad_output, torch.zeros((), dtype=grad_output.dtype, device=grad_output.device))
        else:
            feats, weight, bias = ctx.saved_tensors
        need_f, need_w, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[4], ctx.needs_input_grad[5]
        f = feats.detach().requires_grad_(need_f)
        w = weight.detach().requires_grad_(need_w)
        b = None if bias is None else bias.detach().requires_grad_(need_b)
        grad_input, grad_weight, grad_bias = SparseConv3dFunction._sparse_conv_backward(grad_output, f, ctx.neighbor_cache, w, b,
                                                                                        weight_owner=ctx.weight_owner())
        return grad_input, None, None, None, grad_weight, grad_bias, None, None, None, None, None


def sparse_conv3d(
    feats: torch.Tensor,
    coords: torch.Tensor,
    shape: torch.Size,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    neighbor_cache: Optional[SparseConv3dNeighborCache] = None,
    out_coords: Optional[torch.Tensor] = None,
    stride: Tuple[int, int, int] = (1, 1, 1),
    padding: Tuple[int, int, int] = (0, 0, 0),
    dilation: Tuple[int, int, int] = (1, 1, 1),
) -> Tuple[torch.Tensor, torch.Tensor, SparseConv3dNeighborCache]:
    """
    Sparse convolution for 3D input.

    Args:
        feats (torch.Tensor): [N, C] tensor of input features.
        coords (torch.Tensor): [N, 4] int32 tensor of input coordinates (batch, x, y, z).
        shape (torch.Size): shape of the input tensor in NCWHD order.
        weight (torch.Tensor): [Co, Kw, Kh, Kd, Ci] tensor of weights.
        bias (Optional[torch.Tensor]): [Co] tensor of biases.
        neighbor_cache (Optional[SparseConv3dNeighborCache]): neighbor cache for this operation.
            Can be reused for multiple runs using the same coordinates; computed on the fly if None.
        out_coords (Optional[torch.Tensor]): [M, 4] int32 tensor of output coordinates.  If None, every cell some
            input voxel reaches is an output, in (b, x, y, z) order.
        stride, padding, dilation (Tuple[int, int, int]): geometry of the convolution.

    Returns:
        (out_feats [M, Co], out_coords [M, 4], neighbor_cache)
    """
    with _grad_mode_of_the_caller():
        return SparseConv3dFunction.apply(feats, coords, shape, neighbor_cache, weight, bias, out_coords, stride, padding,
                                          dilation)


def sparse_conv3d_relu(
    feats: torch.Tensor,
    coords: torch.Tensor,
    shape: torch.Size,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    neighbor_cache: Optional[SparseConv3dNeighborCache] = None,
    out_coords: Optional[torch.Tensor] = None,
    stride: Tuple[int, int, int] = (1, 1, 1),
    padding: Tuple[int, int, int] = (0, 0, 0),
    dilation: Tuple[int, int, int] = (1, 1, 1),
) -> Tuple[torch.Tensor, torch.Tensor, SparseConv3dNeighborCache]:
    """relu(sparse_conv3d(...)) with the clamp done in the GEMM's epilogue (no counterpart in the reference; same
    arguments and return values as sparse_conv3d).  Differentiable: backward masks the incoming gradient with the sign
    of the saved output and runs the usual passes."""
    with _grad_mode_of_the_caller():
        return SparseConv3dFunction.apply(feats, coords, shape, neighbor_cache, weight, bias, out_coords, stride, padding,
                                          dilation, True)
