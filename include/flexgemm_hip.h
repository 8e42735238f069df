/*
 * flexgemm_hip.h -- C ABI of libflexgemm_hip.so (gfx950 / MI355X).
 *
 * One shared library replaces the native side of FlexGEMM's submanifold sparse-conv path:
 * the hash-map neighbor-map builder, its post-processing for the masked implicit GEMM, and
 * the masked implicit GEMM forward / dgrad / wgrad with split-K.  Each entry point cites the
 * reference interface it stands in for (paths relative to the reference checkout).
 *
 * Conventions
 *   - every function returns 0 on success or a negative FGX_ERR_* code; fgx_last_error() gives
 *     the message of the calling thread's last failure;
 *   - all pointers are DEVICE pointers unless the name ends in _host; the library never
 *     allocates or frees device memory: the caller owns every buffer, and data-dependent sizes
 *     are obtained through a "count" call, a 4-byte read-back by the caller, then a "fill" call;
 *   - `stream` is a hipStream_t (passed as void*); all work is enqueued on it and nothing
 *     synchronises the host;
 *   - neighbor tables use 0xFFFFFFFF for "no neighbor".
 */
#ifndef FLEXGEMM_HIP_H
#define FLEXGEMM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FGX_OK 0
#define FGX_ERR_ARG (-1)      /* bad argument (shape, dtype, alignment, workspace too small) */
#define FGX_ERR_HIP (-2)      /* a HIP runtime call or kernel launch failed */
#define FGX_ERR_UNSUPPORTED (-3)

/* element types of feature / weight tensors */
#define FGX_F16 0
#define FGX_BF16 1
#define FGX_F32 2

/* epilogue of the gather GEMMs: what is applied to (sum + bias) before it is rounded and stored */
#define FGX_ACT_NONE 0
#define FGX_ACT_RELU 1

typedef void* fgx_stream_t;

/* Library identity and error text.  fgx_abi_version() is 2 for this header.  Against version 1:
 * fgx_subm_neighbor_map_sorted has a `presorted` argument before its workspace, fgx_schedule.stream may be 2 for the
 * weight gradient (call fgx_conv_wgrad_sweep then; fgx_conv_wgrad refuses `streaming` values other than 0 and 1), and the
 * sweep entry points exist.  A caller checks the version once after loading the library. */
int fgx_abi_version(void);
const char* fgx_last_error(void);

/* Profiling aid (no counterpart in the reference, which is timed from outside with CUDA events, tests/utils.py:35-65):
 * calls that enqueue several kernels name their phases.  With a hook set, the calling thread invokes
 * hook(phase_name, stream) right before the kernels of each phase are enqueued and hook("", stream) after the last
 * one; a caller records an event on `stream` in it and reads the time per phase.  NULL (the default) switches it off.
 * Process-wide; set it only while no other thread is inside the library. */
typedef void (*fgx_phase_hook_t)(const char* phase_name, fgx_stream_t stream);
void fgx_set_phase_hook(fgx_phase_hook_t hook);

/* ---------------------------------------------------------------------------------------------
 * Hash table (open addressing, linear probing, Murmur3 finaliser, all-ones key = empty slot).
 * key_bits / val_bits are 32 or 64.
 * ------------------------------------------------------------------------------------------- */

/* Fill the key table with the empty sentinel.
 * Replaces: init_hashmap's torch.full, flex_gemm/ops/utils.py:4-19. */
int fgx_hash_init(void* keys, int key_bits, size_t table_size, fgx_stream_t stream);

/* keys[] <- flattened (b,x,y,z), vals[] <- row index.
 * Replaces: hashmap_insert_3d_idx_as_val, flex_gemm/kernels/cuda/hash/hash.cu:425-449. */
int fgx_hash_insert_3d_idx_as_val(void* keys, int key_bits, void* vals, int val_bits, size_t table_size,
                                  const int32_t* coords, size_t n, int W, int H, int D, fgx_stream_t stream);

/* Generic key -> value insert / lookup on pre-serialised keys.
 * Replaces: hashmap_insert / hashmap_lookup, flex_gemm/kernels/cuda/hash/hash.cu:60-89, 139-172. */
int fgx_hash_insert(void* keys, int key_bits, void* vals, int val_bits, size_t table_size,
                    const void* in_keys, const void* in_vals, size_t m, fgx_stream_t stream);
int fgx_hash_lookup(const void* keys, int key_bits, const void* vals, int val_bits, size_t table_size,
                    const void* in_keys, void* out_vals, size_t m, fgx_stream_t stream);

/* (b,x,y,z) -> user value insert / lookup; a query outside [0,W)x[0,H)x[0,D) yields all ones.
 * Replaces: hashmap_insert_3d / hashmap_lookup_3d, flex_gemm/kernels/cuda/hash/hash.cu:237-266, 336-365. */
int fgx_hash_insert_3d(void* keys, int key_bits, void* vals, int val_bits, size_t table_size,
                       const int32_t* coords, const void* in_vals, size_t m, int W, int H, int D,
                       fgx_stream_t stream);
int fgx_hash_lookup_3d(const void* keys, int key_bits, const void* vals, int val_bits, size_t table_size,
                       const int32_t* coords, void* out_vals, size_t m, int W, int H, int D,
                       fgx_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Neighbor map and its post-processing.
 * ------------------------------------------------------------------------------------------- */

/* Insert all voxels (value = row index) into the caller-initialised table, then write the
 * [n, V] uint32 neighbor table, V = Kw*Kh*Kd (odd kernel sizes).  If gray / binary are non-NULL
 * (requires V <= 32) the per-voxel validity mask and its Gray-decoded sort key are written in the
 * same pass (int32 [n] each).
 * Replaces: hashmap_build_submanifold_conv_neighbour_map,
 *           flex_gemm/kernels/cuda/spconv/subm_neighbor_map.h:40-47 (.cu:104-162); the fused codes
 *           replace neighbor_map_to_gray_binary_code_kernel, migemm_neighmap_pp.cu:19-44. */
int fgx_subm_neighbor_map(void* keys, int key_bits, uint32_t* vals, size_t table_size,
                          const int32_t* coords, size_t n, int W, int H, int D,
                          int Kw, int Kh, int Kd, int Dw, int Dh, int Dd,
                          uint32_t* out_map, int32_t* gray, int32_t* binary, fgx_stream_t stream);

/* The same table as fgx_subm_neighbor_map without a hash table: (flattened key, row) pairs are radix-sorted, and a
 * workgroup of 256 consecutive sorted voxels finds, for every (dx, dy), all its neighbors in one contiguous window of
 * the sorted array (two binary searches, one coalesced read into LDS, per-lane searches there).  Meant for large or
 * shuffled coordinate sets, where hash probes are cache-line fetches at random addresses.  key_bits: 32 when
 * B*W*H*D <= 2^32, else 64 (grids up to 2^63 cells).  workspace: fgx_subm_neighbor_map_sorted_workspace_bytes bytes,
 * 256-byte aligned.  gray / binary as above.  presorted = 1 promises that the flattened keys ((b*W + x)*H + y)*D + z
 * never descend from one voxel to the next (voxels listed in scan order): the radix sort is skipped.  presorted = 2
 * leaves the question to the device: the kernel that makes the keys also notes whether one descends, the sort's kernels
 * return at once when none does, and the search takes the unsorted arrays then -- nothing is read back (32-bit keys and up
 * to 2^21 voxels; otherwise 2 means 0: the keys are sorted without asking).  presorted = 0 always sorts.
 * fgx_coords_key_order answers the question for a caller that wants to know: it sets descents[0] (device, cleared by the
 * caller beforehand) to 1 when some key is smaller than its predecessor's.
 * Replaces: the same reference function as fgx_subm_neighbor_map (the result is identical; only the search differs). */
size_t fgx_subm_neighbor_map_sorted_workspace_bytes(size_t n, int key_bits, int Kw, int Kh);
int fgx_coords_key_order(const int32_t* coords, size_t n, int W, int H, int D, uint32_t* descents, fgx_stream_t stream);
int fgx_subm_neighbor_map_sorted(const int32_t* coords, size_t n, int B, int W, int H, int D,
                                 int Kw, int Kh, int Kd, int Dw, int Dh, int Dd, int key_bits, int presorted,
                                 void* workspace, size_t workspace_bytes,
                                 uint32_t* out_map, int32_t* gray, int32_t* binary, fgx_stream_t stream);

/* Validity mask (bit v <=> map[n, v] present) and Gray-decoded key from an existing map.
 * Replaces: neighbor_map_to_gray_binary_code_kernel, migemm_neighmap_pp.cu:19-44. */
int fgx_mask_codes(const uint32_t* map, size_t n, int V, int32_t* gray, int32_t* binary, fgx_stream_t stream);

/* Stable ascending sort of voxels by key (signed int32 compare) -> int64 permutation.
 * Replaces: torch::argsort(binary_code), migemm_neighmap_pp.cu:79,221 (whose tie order is unspecified;
 *           this one keeps equal keys in ascending row order).
 * Workspace: fgx_sort_workspace_bytes(n) bytes, 256-byte aligned. */
size_t fgx_sort_workspace_bytes(size_t n);
int fgx_sort_by_code(const int32_t* binary, size_t n, int V, int64_t* sorted_idx,
                     void* workspace, size_t workspace_bytes, fgx_stream_t stream);

/* Row order for the gather GEMM that keeps gathers cache-resident: voxels are ranked along a Z-order curve of their
 * coordinates, cut into chunks of `chunk_rows` consecutive ranks, and sorted by mask key inside each chunk (stable).
 * Tiles of this order are still mask-homogeneous (their OR-masks come from fgx_tile_codes on this order) but all rows
 * a run of tiles gathers lie in one small region, so an XCD's L2 serves the ~10 re-reads of every feature row.
 * No counterpart in the reference, whose kernels walk the globally mask-sorted order (migemm_neighmap_pp.cu:79,221).
 * Workspace: fgx_locality_workspace_bytes(n) bytes, 256-byte aligned. */
size_t fgx_locality_workspace_bytes(size_t n);
int fgx_locality_order(const int32_t* coords, const int32_t* binary, size_t n, int V, int chunk_rows, int64_t* order,
                       void* workspace, size_t workspace_bytes, fgx_stream_t stream);
/* The same order when the grid is known (coordinates below 2^bits_per_axis, batch indices below 2^batch_bits): both sorts
 * then run over the key bits in use alone, the first on 32-bit keys when 3 * bits_per_axis + batch_bits <= 32 (4.1 M voxels
 * of a 1024-cube: 9 radix passes instead of 14).  fgx_locality_order is this function with 16 and 16 bits. */
int fgx_locality_order_grid(const int32_t* coords, const int32_t* binary, size_t n, int V, int chunk_rows, int bits_per_axis,
                            int batch_bits, int64_t* order, void* workspace, size_t workspace_bytes, fgx_stream_t stream);

/* The plain Z-order of the rows (what fgx_locality_order gives with chunk_rows = 1) when the grid is known: coordinates
 * below 2^bits_per_axis, batch indices below 2^batch_bits -- the sort then runs over 3 * bits_per_axis + batch_bits key bits
 * instead of 64 (2.67 M voxels of a 1024-cube: four passes instead of eight).  Coordinates outside that range are sorted
 * by their low bits (still a permutation).  Workspace: fgx_locality_workspace_bytes(n).  The row order of fgx_narrow_plan. */
int fgx_zorder_rows(const int32_t* coords, size_t n, int bits_per_axis, int batch_bits, int64_t* order, void* workspace,
                    size_t workspace_bytes, fgx_stream_t stream);

/* Pair lists for wgrad: all (v, n) with map[n, v] present, ordered by v then n.
 *   count: seg[V+1] <- exclusive offsets per v (seg[V] = L); caller reads seg[V] back, allocates
 *          sig_i / sig_o of L uint32 each, then calls fill with the same workspace.
 * Replaces: neighbor_map_post_process_for_masked_implicit_gemm_1's transposed map + cumsum +
 *           gather_idx_val_seg_from_prefix_sum_kernel, migemm_neighmap_pp.cu:157-178, 207-240. */
size_t fgx_pair_workspace_bytes(size_t n, int V);
int fgx_pair_count(const int32_t* gray, size_t n, int V, uint32_t* seg,
                   void* workspace, size_t workspace_bytes, fgx_stream_t stream);
int fgx_pair_fill(const uint32_t* map, const int32_t* gray, size_t n, int V,
                  const void* workspace, uint32_t* sig_i, uint32_t* sig_o, fgx_stream_t stream);

/* The whole neighbor cache of a submanifold convolution in one call: fgx_subm_neighbor_map_sorted (map, gray / binary
 * codes), fgx_sort_by_code (sorted_idx) and, with_pairs != 0, fgx_pair_count and fgx_pair_fill (seg[V + 1], sig_i / sig_o
 * with room for one entry per slot of the map, n * V) -- same arguments, same results, nothing between the kernels for
 * the GPU to wait for.  From 393 216 voxels on the pair lists are enqueued on a second stream of the library's own
 * (default priority, one per device, made on first use) beside the mask sort, and `stream` waits for it before the call
 * returns; never during a stream capture.  Kernel volumes up to 32.  workspace: fgx_subm_cache_workspace_bytes bytes,
 * 256-byte aligned.  Replaces: SubMConv3dFunction._compute_neighbor_cache's sequence of extension calls
 * (flex_gemm/ops/spconv/submanifold_conv3d.py:46-107: hashmap insert, neighbor map, gray-code sort, kernel_map post-pass). */
size_t fgx_subm_cache_workspace_bytes(size_t n, int key_bits, int Kw, int Kh, int Kd, int with_pairs);
int fgx_subm_cache_build(const int32_t* coords, size_t n, int B, int W, int H, int D, int Kw, int Kh, int Kd, int Dw, int Dh, int Dd,
                         int key_bits, int presorted, int with_pairs, void* workspace, size_t workspace_bytes, uint32_t* out_map,
                         int32_t* gray, int32_t* binary, int64_t* sorted_idx, uint32_t* seg, uint32_t* sig_i, uint32_t* sig_o,
                         fgx_stream_t stream);

/* Per row-tile (block consecutive rows of the sorted order) OR of the masks.
 *   codes: tile_code[nb] <- OR mask, seg[nb+1] <- exclusive offsets of popcounts (seg[nb] = total);
 *   fill : valid_kernel[total] <- set-bit positions, ascending per tile.
 * Replaces: neighbor_map_post_process_for_masked_implicit_gemm_2 (reduce_code_kernel, cumsum,
 *           scatter_reduced_code_kernel), migemm_neighmap_pp.cu:246-368.  Any block >= 1 is accepted. */
size_t fgx_tile_workspace_bytes(size_t n, int block);
int fgx_tile_codes(const int32_t* gray, const int64_t* sorted_idx, size_t n, int block,
                   int32_t* tile_code, int32_t* seg, void* workspace, size_t workspace_bytes,
                   fgx_stream_t stream);
int fgx_tile_fill(const int32_t* tile_code, const int32_t* seg, size_t num_tiles, int32_t* valid_kernel,
                  fgx_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Masked implicit GEMM.
 * ------------------------------------------------------------------------------------------- */

/* Fixed gfx950 schedule for a problem (replaces the Triton autotuner and autotune_cache.json:
 * flex_gemm/utils/autotuner.py:18-291, flex_gemm/kernels/triton/spconv/config.py:10-83 and the
 * SPLITK searches in ..._masked_implicit_gemm_splitk.py).  `pass_kind`: 0 fwd, 1 dgrad, 2 wgrad. */
typedef struct fgx_schedule {
    int tile_rows;      /* fwd/dgrad: sorted voxel rows per tile (B1); wgrad: Co rows per tile */
    int tile_cols;      /* fwd/dgrad: output channels per tile (B2);   wgrad: Ci columns per tile */
    int slab_bytes;     /* fwd/dgrad: bytes of K staged per row and pipeline step (64 or 128) */
    int splitk;         /* fwd/dgrad: number of K splits (1 = none) */
    int block_rows;     /* wgrad: voxel rows per partial-sum block */
    int stream;         /* 1 = persistent streaming kernel (fwd/dgrad: fgx_conv_gather_gemm_stream; wgrad: the
                         * `streaming` argument of fgx_conv_wgrad), 0 = tiled kernel; wgrad only: 2 = the sweep
                         * fgx_conv_wgrad_sweep with tile = tile_rows and sub_rows = block_rows */
} fgx_schedule;
int fgx_table_lookup(int pass_kind, int dtype, size_t n, int Ci, int Co, int V, fgx_schedule* out);

/* Re-layout the [Co, V, Ci] weight into K-slab-major panels consumed by fgx_conv_gather_gemm.
 *   mode 0 (forward): panel[v][slab][co][k]  = w[co][v][slab*SK + k]          (K = Ci, cols = Co)
 *   mode 1 (dgrad)  : panel[v][slab][ci][k]  = w[slab*SK + k][V-1-v][ci]      (K = Co, cols = Ci)
 *   mode 2 (dgrad through a separate backward map, generic sparse convolution):
 *                     panel[v][slab][ci][k]  = w[slab*SK + k][v][ci]          (K = Co, cols = Ci)
 * SK = slab_bytes / element size (slab_bytes = 64 or 128: the schedule's value); K is zero-padded to a whole
 * slab and cols to a multiple of col_pad (a multiple of 32; pass the tile_cols the GEMM will run with).
 * Replaces: the strided weight-tile loads of the Triton kernels
 *           (..._fwd_masked_implicit_gemm.py:79, ..._bwd_masked_implicit_gemm.py:74). */
size_t fgx_weight_panel_bytes(int dtype, int mode, int Ci, int Co, int V, int slab_bytes, int col_pad);
int fgx_pack_weight(int dtype, int mode, const void* weight, int Ci, int Co, int V, int slab_bytes, int col_pad,
                    void* panel, fgx_stream_t stream);

/* `sorted_idx` may be ANY permutation of the rows (the mask-sorted order or fgx_locality_order's); `tile_code` must
 * come from fgx_tile_codes on that same permutation with block = tile_rows.
 * out[sorted[r], :] = sum over offsets v present in row r of src[map[sorted[r], v], :] . panel_v  (+ bias)
 * for K = src channels, cols = out channels.  Forward: src = feats, panel mode 0, bias optional.
 * dgrad: src = grad_output, panel mode 1, bias = NULL.  Tiles of `tile_rows` sorted rows skip every
 * offset whose bit is clear in tile_code[tile].  splitk > 1 needs `scratch` of
 * fgx_conv_scratch_bytes() bytes (fp32 partial sums, reduced in a second kernel).
 * Replaces: sparse_submanifold_conv_fwd_masked_implicit_gemm[_splitk] (kernels
 *           ..._fwd_masked_implicit_gemm.py:20-100, ..._splitk.py:22-106, wrapper :133-172) and
 *           sparse_submanifold_conv_bwd_input_masked_implicit_gemm[_splitk]
 *           (..._bwd_masked_implicit_gemm.py:19-91, ..._splitk.py:24-100, 209-251). */
size_t fgx_conv_scratch_bytes(size_t n, int cols, int splitk);
int fgx_conv_gather_gemm(int dtype, const void* src, const void* panel, const void* bias,
                         const uint32_t* map, const int64_t* sorted_idx, const int32_t* tile_code,
                         size_t n, int K, int cols, int V, int tile_rows, int tile_cols, int slab_bytes, int splitk,
                         void* scratch, void* out, fgx_stream_t stream);

/* fgx_conv_gather_gemm with an activation (FGX_ACT_*) applied to (sum + bias) in the kernel's epilogue -- with split-K, in
 * the reduction of the partial sums -- so that out = act(conv + bias) costs no pass over the output of its own.
 * No counterpart in the reference, whose kernels end with the bias add (..._fwd_masked_implicit_gemm.py:97-100); for
 * inference graphs whose normalisation layers are folded into weight and bias. */
int fgx_conv_gather_gemm_act(int dtype, const void* src, const void* panel, const void* bias,
                             const uint32_t* map, const int64_t* sorted_idx, const int32_t* tile_code,
                             size_t n, int K, int cols, int V, int tile_rows, int tile_cols, int slab_bytes, int splitk,
                             void* scratch, int activation, void* out, fgx_stream_t stream);

/* ... which also leaves the activation's derivative as one bit per output: bit (c mod 8) of relu_mask[(r * cols + c) / 8]
 * is set when out[r][c] > 0.  For the backward pass of a fused ReLU, which then reads n * cols / 8 bytes instead of the
 * output again (fgx_relu_mask_apply).  relu_mask may be NULL (no mask); otherwise activation must be FGX_ACT_RELU, the type
 * 16-bit and cols a multiple of 8.  No counterpart in the reference. */
int fgx_conv_gather_gemm_act_mask(int dtype, const void* src, const void* panel, const void* bias,
                                  const uint32_t* map, const int64_t* sorted_idx, const int32_t* tile_code,
                                  size_t n, int K, int cols, int V, int tile_rows, int tile_cols, int slab_bytes, int splitk,
                                  void* scratch, int activation, void* out, uint8_t* relu_mask, fgx_stream_t stream);
/* out[i] = bit i of relu_mask ? grad[i] : 0 for i < numel (a multiple of 8; 16-bit types; grad and out 16-byte aligned,
 * out may be grad): the gradient of a fused ReLU from the mask its forward pass wrote.  One pass, numel / 8 bytes of mask
 * read beside the gradient.  No counterpart in the reference. */
int fgx_relu_mask_apply(int dtype, const void* grad, const uint8_t* relu_mask, size_t numel, void* out, fgx_stream_t stream);

/* Gather plan of a row order for tiles of `tile_rows` rows: for tile t and the k-th offset v present in it
 * (the set bits of tile_code[t], ascending; a tile whose code is 0 gets one row with every neighbor missing),
 *   plan_idx[(plan_seg[t] + k) * tile_rows + r] = map[order[t * tile_rows + r], v]     (0xFFFFFFFF for rows past n),
 *   plan_band[plan_seg[t] + k] bit b = 1 iff rows [32 b, 32 b + 32) of the tile have a neighbor at v   (optional).
 * count: plan_seg[num_tiles + 1] <- exclusive offsets, plan_seg[num_tiles] = plan rows; the caller reads that back,
 * allocates plan_idx (tile_rows uint32 per plan row, 16-byte aligned) and plan_band (one uint32 per plan row, may be
 * NULL; needs tile_rows <= 1024) and calls fill.  `tile_code` comes from
 * fgx_tile_codes on the same order and tile size; workspace: fgx_tile_workspace_bytes(num_tiles, 1) bytes,
 * 256-byte aligned.
 * Replaces: the neighbor[sorted_idx[rows], v] double gather inside the Triton kernels
 *           (..._fwd_masked_implicit_gemm.py:69-76, ..._bwd_masked_implicit_gemm.py:64-71) by a table built once per
 *           coordinate set. */
int fgx_gather_plan_count(const int32_t* tile_code, size_t num_tiles, int32_t* plan_seg, void* workspace,
                          size_t workspace_bytes, fgx_stream_t stream);
int fgx_gather_plan_fill(const uint32_t* map, const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                         size_t n, int V, int tile_rows, uint32_t* plan_idx, uint32_t* plan_band, fgx_stream_t stream);

/* Same result as fgx_conv_gather_gemm (splitk = 1) from the gather plan of `order`, by persistent workgroups that
 * stream all their tiles' (offset, K-slab) steps back to back; meant for voxel counts that give every CU several
 * tiles.  `max_groups`: workgroups to launch (<= 0: as many as are resident at once, at most two per CU).  Operands are addressed with 32-bit offsets:
 * returns FGX_ERR_UNSUPPORTED when src, the panel or the plan exceed ~4 GB, or when no kernel exists for the
 * schedule -- callers then use fgx_conv_gather_gemm.  `plan_band` (from fgx_gather_plan_fill; NULL = every band
 * present) lets the kernel skip the loads and products of 32-row bands without a neighbor at an offset.
 * `n` counts the output rows (rows of the map behind the plan), `n_src` the rows of `src`; they differ for the
 * generic sparse convolution only.
 * `item_at` (device, may be NULL): a permutation of the items 0 .. row_tiles * col_tiles - 1 (item = row tile *
 * col_tiles + column tile, row_tiles = ceil(n / tile_rows), col_tiles = ceil(cols / tile_cols)).  Workgroup w of G
 * works through the positions p(w), p(w) + G, ... of that sequence, p(w) = (w % 8) * (G / 8) + w / 8 when 8 divides
 * G, else w: a caller that knows the tiles' costs (offsets per tile = popcount of tile_code) orders the items so that
 * the workgroups' sums come out even.  NULL: last tile first.  The result does not depend on it.
 * fgx_conv_gather_gemm_stream_groups tells G for max_groups <= 0.
 * Replaces: the same reference kernels as fgx_conv_gather_gemm. */
int fgx_conv_gather_gemm_stream(int dtype, const void* src, const void* panel, const void* bias,
                                const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                                const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows, size_t n,
                                size_t n_src, int K, int cols, int V,
                                int tile_rows, int tile_cols, int slab_bytes, const uint32_t* item_at,
                                int max_groups, void* out, fgx_stream_t stream);
/* ... with an activation (FGX_ACT_*) in the epilogue, as fgx_conv_gather_gemm_act; no counterpart in the reference. */
int fgx_conv_gather_gemm_stream_act(int dtype, const void* src, const void* panel, const void* bias,
                                    const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                                    const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows, size_t n,
                                    size_t n_src, int K, int cols, int V,
                                    int tile_rows, int tile_cols, int slab_bytes, const uint32_t* item_at,
                                    int max_groups, int activation, void* out, fgx_stream_t stream);
/* ... and with the ReLU mask of fgx_conv_gather_gemm_act_mask. */
int fgx_conv_gather_gemm_stream_act_mask(int dtype, const void* src, const void* panel, const void* bias,
                                         const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                                         const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows, size_t n,
                                         size_t n_src, int K, int cols, int V,
                                         int tile_rows, int tile_cols, int slab_bytes, const uint32_t* item_at,
                                         int max_groups, int activation, void* out, uint8_t* relu_mask, fgx_stream_t stream);
int fgx_conv_gather_gemm_stream_groups(int dtype, int cols, int tile_rows, int tile_cols, int slab_bytes, int* groups);

/* Gather GEMM for narrow layers with the gathered rows resident in LDS: 16-bit types, K and cols of 8, 16, 24 or 32
 * channels (rows of at most 64 bytes), `panel` from fgx_pack_weight with slab_bytes = 64 and col_pad = 32.  Rows walk in
 * chunks of 128 along `order` (any permutation; a Z-order curve of the coordinates -- fgx_locality_order with
 * chunk_rows = 1 -- makes a chunk's rows neighbors in space); fgx_narrow_plan names, once per neighbor map and order, every
 * chunk's distinct source rows (about 1.7 per output row on a surface, where the streaming kernel requests 10.5) and the
 * LDS slot of the source of every (row, offset); its first 256 bytes are a header whose first uint32 counts the chunks
 * with more distinct sources than slots.  Per chunk the kernel loads those rows once and multiplies all V offsets
 * for all rows (a missing neighbor is a row of zeros): same function as fgx_conv_gather_gemm_stream, sums in offset
 * order.  A chunk with more than 448 distinct sources (rows ordered without locality) stays correct: the surplus is read
 * from memory through `map`.  same_rows = 1 when output row i and source row i are the same voxel (submanifold layers,
 * forward and dgrad): every chunk row then sits in the LDS slot of its own number, which keeps the multipliers' reads of
 * neighboring rows on different banks.  activation / relu_mask as in fgx_conv_gather_gemm_act_mask.
 * plan: fgx_narrow_plan_bytes(n, V) bytes, 16-byte aligned.
 * No counterpart in the reference, whose kernels gather every row per (tile, offset) from memory
 * (..._fwd_masked_implicit_gemm.py:20-100). */
size_t fgx_narrow_plan_bytes(size_t n, int V);
int fgx_narrow_plan(const uint32_t* map, const int64_t* order, size_t n, int V, int same_rows, void* plan, fgx_stream_t stream);
int fgx_conv_narrow_gemm(int dtype, const void* src, const void* panel, const void* bias, const uint32_t* map, const void* plan,
                         size_t n, size_t n_src, int K, int cols, int V, int activation, void* out, uint8_t* relu_mask,
                         fgx_stream_t stream);

/* The weight gradient of such a layer on the same plan: grad_weight[co][v][ci] = sum over rows r with a neighbor at offset
 * v of grad_out[r][co] * feats[source(r, v)][ci], for 16-bit types and Ci, Co of 8, 16, 24 or 32.  Per chunk of 128 rows
 * the chunk's own grad_out rows and its distinct source rows are loaded into LDS once (the block-major kernel of
 * fgx_conv_wgrad fetches two rows per pair), the gather happens in the transposing LDS reads.  Every workgroup keeps the
 * accumulators of all V offsets over its chunks and writes one partial product; a second kernel adds the partial
 * products in workgroup order (same bits on every run; against fgx_conv_wgrad the sums differ by fp32 rounding of a
 * different order).  The plan must have been made with same_rows = 1 and must have NO overflowing chunk: the first
 * uint32 of the plan counts them -- read it back once per plan and call fgx_conv_wgrad instead when it is not 0.
 * scratch: fgx_narrow_wgrad_scratch_bytes(V) bytes, 16-byte aligned.  The bias gradient is not made here (fgx_colsum).
 * No counterpart in the reference (..._bwd_masked_implicit_gemm_splitk.py:108-182 gathers both operands per pair). */
size_t fgx_narrow_wgrad_scratch_bytes(int V);
int fgx_conv_narrow_wgrad(int dtype, const void* grad_out, const void* feats, const void* plan, size_t n, size_t n_src, int Ci,
                          int Co, int V, void* scratch, void* grad_weight, fgx_stream_t stream);

/* item_at for fgx_conv_gather_gemm_stream, made on the device from the tile codes: items sorted by cost (offsets per
 * row tile x `slabs` K-slabs + an epilogue), the incomplete last round of `groups` positions filled with the cheapest,
 * every full round dealt most-expensive-item to least-loaded-slot.  One workgroup, deterministic, no read-back;
 * groups <= 1024.  workspace: fgx_gather_item_order_workspace_bytes bytes, 256-byte aligned; item_at: uint32 per item.
 * No counterpart in the reference (Triton's grid is one program per tile). */
size_t fgx_gather_item_order_workspace_bytes(size_t num_tiles, int col_tiles);
int fgx_gather_item_order(const int32_t* tile_code, size_t num_tiles, int col_tiles, int slabs, int groups,
                          void* workspace, size_t workspace_bytes, uint32_t* item_at, fgx_stream_t stream);

/* grad_weight[co, v, ci] = sum over pairs k in [seg[v], seg[v+1]) of grad_out[sig_o[k], co] * feats[sig_i[k], ci].
 * seg_host is the HOST copy of valid_signal_seg (V+1 entries); sig_o must ascend inside every segment (it does
 * when it comes from fgx_pair_fill).  The voxels are cut into blocks of `block_rows` rows; every (block, offset)
 * partial product goes to `scratch` in fp32 (fgx_wgrad_scratch_bytes bytes, 256-byte aligned) and a second kernel
 * adds them per offset in block order.  `streaming` != 0 asks for the persistent kernel with loader / multiplier
 * wavefronts (16-bit types, 128x128 or 64x64 tiles, operands below ~4 GB); outside that range the tiled kernel runs.
 * `n` = rows of grad_out (the range of sig_o), `n_in` = rows of feats (the range of sig_i); equal for the submanifold
 * convolution.  `block_bounds` (optional): the table fgx_wgrad_block_bounds makes from the same pair lists and
 * block_rows -- block_bounds[v * (nb + 1) + b] = first pair of offset v whose grad_out row is >= b * block_rows,
 * nb = ceil(n / block_rows) -- for callers that keep it with their neighbor cache; NULL = computed here, per call.
 * The 32x32 streaming tile writes four partial products per block; the scratch size accounts for it where that tile
 * may stream, i.e. with at most 32 channels on a side -- a 32x32 tile with wider channels runs the tiled kernel.
 * `grad_bias` (optional, Co elements of the tensors' type): the column sums of grad_out over its n rows, the bias
 * gradient.  `bias_offset` names an offset whose pairs hold every grad_out row exactly once (the centre offset of a
 * submanifold convolution; -1 when there is none): the streaming kernel then sums the grad_out rows it loads for that
 * offset anyway and grad_out is not read a third time.  Without such an offset, or on the tiled path, the call runs
 * fgx_colsum itself (the scratch size accounts for that too).
 * Replaces: sparse_submanifold_conv_bwd_weight_masked_implicit_gemm[_splitk]
 *           (..._bwd_masked_implicit_gemm.py:99-170, ..._splitk.py:108-182, 278-317), and with grad_bias
 *           grad_output.sum(0) (..._splitk.py:365-366). */
size_t fgx_wgrad_scratch_bytes(size_t n, int V, int Ci, int Co, int block_rows);
size_t fgx_wgrad_block_bounds_count(size_t n, int V, int block_rows);
int fgx_wgrad_block_bounds(const uint32_t* sig_o, const uint32_t* seg_host, size_t n, int V, int block_rows,
                           uint32_t* block_bounds, fgx_stream_t stream);
int fgx_conv_wgrad(int dtype, const void* grad_out, const void* feats,
                   const uint32_t* sig_i, const uint32_t* sig_o, const uint32_t* seg_host, const uint32_t* block_bounds,
                   size_t n, size_t n_in, int Ci, int Co, int V, int tile_rows, int tile_cols, int block_rows,
                   int streaming, void* scratch, void* grad_weight, void* grad_bias, int bias_offset,
                   fgx_stream_t stream);

/* Balanced work lists for the streaming kernel of fgx_conv_wgrad (streaming = 1).  Its work items are (voxel block, offset,
 * tile) and cost what their pair count says (the centre offset pairs every row of a block, a corner offset a fraction);
 * dealt out in a fixed order, the workgroup with the most pairs sets the launch's time.  fgx_wgrad_item_lists reads the
 * block table and deals the items longest-first to the least loaded XCD and workgroup (on the device, one small kernel:
 * once per neighbor cache, block_rows and tile shape); fgx_conv_wgrad_lists is fgx_conv_wgrad walking those lists
 * (item_lists = NULL: the fixed order; lists made for another shape are ignored).  The result is the same bit for bit
 * either way: every item is still summed by one workgroup in the same order.  fgx_wgrad_item_lists_count gives the
 * uint32 words of the lists, 0 where they do not apply (fewer than 2 048 voxels; more than 12 voxel blocks (16 with several tiles) or 4 096 items: the fixed order, which
 * keeps the offsets of a voxel block on one XCD, is balanced well enough then).
 * No counterpart in the reference, whose Triton launch leaves the order of its programs to the hardware scheduler
 * (..._bwd_masked_implicit_gemm_splitk.py:278-317). */
size_t fgx_wgrad_item_lists_count(size_t n, int V, int Ci, int Co, int tile_rows, int tile_cols, int block_rows);
int fgx_wgrad_item_lists(const uint32_t* block_bounds, size_t n, int V, int Ci, int Co, int tile_rows, int tile_cols,
                         int block_rows, uint32_t* item_lists, fgx_stream_t stream);
int fgx_conv_wgrad_lists(int dtype, const void* grad_out, const void* feats,
                         const uint32_t* sig_i, const uint32_t* sig_o, const uint32_t* seg_host, const uint32_t* block_bounds,
                         const uint32_t* item_lists, size_t n, size_t n_in, int Ci, int Co, int V, int tile_rows, int tile_cols,
                         int block_rows, int streaming, void* scratch, void* grad_weight, void* grad_bias, int bias_offset,
                         fgx_stream_t stream);

/* The same weight gradient as a sweep over the voxels, for 16-bit types, a single Co x Ci tile (`tile` = 128 or 64 >= Co,
 * Ci) and at most 2^24 rows per operand: each XCD takes a contiguous range of sub-blocks of `sub_rows` voxels holding an
 * eighth of the pairs, and every workgroup keeps the accumulators of two "units" (an offset, or a share of the 64-pair
 * steps of an offset) over that whole range -- 2 x (compute units) partial products in all.  The table's schedule for such
 * weights (fgx_schedule.stream = 2).  Optional pacing: nobody starts a sub-block more than `lead` ahead of the slowest
 * workgroup of its XCD; after `max_polls` looks at the others' progress a workgroup stops waiting, so the kernel ends
 * whatever happens; max_polls = 0 switches the pacing off (faster; pacing keeps the gathered rows in the XCD's L2).
 * fgx_wgrad_sweep_plan builds the units and the per-workgroup step lists from the pair lists alone, which must ascend in
 * the output row inside every offset (once per neighbor cache and sub_rows; fgx_wgrad_sweep_plan_bytes bytes, 256-byte
 * aligned); fgx_conv_wgrad_sweep needs fgx_wgrad_sweep_scratch_bytes of scratch.  Sums are taken in a fixed order: same
 * bits on every run, fp32 rounding differences against fgx_conv_wgrad.  grad_bias / bias_offset as for fgx_conv_wgrad.
 * Replaces: the same Triton kernels as fgx_conv_wgrad (its SPLITK slices become the units). */
size_t fgx_wgrad_sweep_plan_bytes(size_t n, size_t n_pairs, int V, int sub_rows);
int fgx_wgrad_sweep_plan(const uint32_t* sig_o, const uint32_t* seg_host, size_t n, int V, int sub_rows, void* plan,
                         size_t plan_bytes, fgx_stream_t stream);
size_t fgx_wgrad_sweep_scratch_bytes(int Ci, int Co);
int fgx_conv_wgrad_sweep(int dtype, const void* grad_out, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                         const uint32_t* seg_host, const void* plan, size_t n, size_t n_in, int Ci, int Co, int V, int tile,
                         int sub_rows, int lead, int max_polls, void* scratch, void* grad_weight, void* grad_bias,
                         int bias_offset, fgx_stream_t stream);

/* A wavefront of the sweep that waits for data (rows that have not landed, a ring stage that has not been read) looks at
 * the progress word a bounded number of times and then goes on, so that the kernel ends whatever happens; it then sets its
 * give-up word in the scratch, and the sweep's reduction writes NaN into all of grad_weight and grad_bias instead of sums
 * that may be wrong.  (The optional pacing wait is not data: giving up on it costs speed only and sets nothing.)
 * fgx_wgrad_sweep_giveup_words returns the number of 32-bit give-up words and their byte offset inside the scratch;
 * fgx_wgrad_sweep_reduce runs the reduction alone over a scratch that a fgx_conv_wgrad_sweep call with the same plan and
 * shapes has filled (grad_bias non-null: that call made the bias gradient inside the sweep).  Both exist for tests of the
 * NaN path and for diagnosis; no counterpart in the reference. */
size_t fgx_wgrad_sweep_giveup_words(int Ci, int Co, size_t* byte_offset);
int fgx_wgrad_sweep_reduce(int dtype, const void* plan, size_t n, size_t n_pairs, int Ci, int Co, int V, int sub_rows,
                           void* scratch, void* grad_weight, void* grad_bias, int bias_offset, fgx_stream_t stream);

/* grad_bias[co] = sum over rows of grad_out[:, co], accumulated in fp32.
 * `scratch`: fgx_colsum_scratch_bytes bytes of fp32 partial sums.
 * Replaces: grad_output.sum(0), ..._bwd_masked_implicit_gemm_splitk.py:365-366. */
size_t fgx_colsum_scratch_bytes(size_t n, int cols);
int fgx_colsum(int dtype, const void* grad_out, size_t n, int cols, void* scratch, void* out,
               fgx_stream_t stream);

/* fgx_colsum without a scratch argument, for callers that cannot allocate (code under HIP graph capture, serving loops
 * with a fixed memory plan, harnesses that forbid hipMalloc): the fp32 partial sums go to an array the library itself
 * holds on every GPU it runs on (8 MiB, for up to fgx_colsum_static_max_cols() = 2048 columns; wider tensors are
 * refused with FGX_ERR_ARG).  Allocates nothing, same kernels and same bits as fgx_colsum.  All calls on one GPU share
 * that array: calls that may overlap there (different streams, different threads) race -- serialise them.  Every
 * call overwrites the part it reads, so nothing has to be cleared between calls.
 * The first use on a device looks up that device's address of the array, which may load the code object and is no
 * stream operation: it cannot happen under capture.  Call fgx_colsum_static_prepare() once per device, with that device
 * current, before capturing (any earlier fgx_colsum_static call on the device does the same); a first use on a stream
 * that is being captured is refused with FGX_ERR_ARG.  A caller that also wants the kernels loaded before the capture
 * makes one ordinary call of the same dtype first.
 * No counterpart in the reference (torch allocates its reduction buffers itself). */
int fgx_colsum_static_prepare(void);
int fgx_colsum_static_max_cols(void);
int fgx_colsum_static(int dtype, const void* grad_out, size_t n, int cols, void* out, fgx_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Generic sparse convolution (stride / padding / dilation): output coordinates and neighbor maps.
 * The GEMM passes are the ones above: forward gathers feats through map_fwd (n = output rows, n_src = input
 * rows), the input gradient gathers grad_out through map_bwd with the mode-2 weight panel, wgrad takes the pair
 * lists of map_fwd.
 * ------------------------------------------------------------------------------------------- */

/* (Wo, Ho, Do) = floor((N + 2P - D(K-1) - 1) / S) + 1 per axis.
 * Replaces: the size formula in flex_gemm/kernels/cuda/spconv/sparse_neighbor_map.cu:86-88. */
int fgx_spconv_out_dims(int W, int H, int D, int Kw, int Kh, int Kd, int Sw, int Sh, int Sd,
                        int Pw, int Ph, int Pd, int Dw, int Dh, int Dd, int* Wo, int* Ho, int* Do);

/* Output coordinates, two steps around the one read-back that sizes the result:
 *   fgx_spconv_out_coords_keys    every cell o = (i + P - k*D) / S reached by an input voxel i through a kernel
 *                                 position k (exact division, inside the output grid) as a flattened key
 *                                 ((b*Wo + x)*Ho + y)*Do + z, sorted ascending and unique, left at the start of
 *                                 `workspace`; their number goes to `count` (DEVICE memory, 8 bytes).
 *   fgx_spconv_out_coords_decode  keys -> int32 (b, x, y, z) rows, `count` of them (the value read back).
 * key_bits: 32 when B*Wo*Ho*Do < 2^32 - 1, else 64.  workspace: fgx_spconv_out_coords_workspace_bytes bytes,
 * 256-byte aligned.  The order is the reference's with BXYZ serialisation (its default), i.e. torch.unique(dim=0).
 * Replaces: hashmap_build_sparse_conv_out_coords and expand_unique_build_sparse_conv_out_coords,
 *           flex_gemm/kernels/cuda/spconv/sparse_neighbor_map.h:42-86 (.cu:76-131, 275-345). */
size_t fgx_spconv_out_coords_workspace_bytes(size_t n_in, int V, int key_bits);
int fgx_spconv_out_coords_keys(const int32_t* coords, size_t n_in, int B, int W, int H, int D,
                               int Kw, int Kh, int Kd, int Sw, int Sh, int Sd, int Pw, int Ph, int Pd,
                               int Dw, int Dh, int Dd, int key_bits, void* workspace, size_t workspace_bytes,
                               uint64_t* count, fgx_stream_t stream);
int fgx_spconv_out_coords_decode(const void* workspace, int key_bits, size_t count, int Wo, int Ho, int Do,
                                 int32_t* out_coords, fgx_stream_t stream);

/* map_fwd[o, v] = row of the input voxel at out_coords[o]*S - P + k_v*D (same batch, inside the input grid), all
 * ones when there is none; map_bwd[i, v] = o for every map_fwd[o, v] = i, all ones elsewhere (NULL = not wanted;
 * [n_in, V], filled here).  `keys` / `vals` is the hash table of the INPUT voxels (fgx_hash_init +
 * fgx_hash_insert_3d_idx_as_val over the input grid).  gray / binary (optional, V <= 32): validity mask of every
 * map_fwd row and its Gray-decoded sort key, as fgx_mask_codes would give.
 * Replaces: hashmap_build_sparse_conv_neighbour_map, sparse_neighbor_map.h:88-131 (.cu:431-567). */
int fgx_spconv_neighbor_map(const void* keys, int key_bits, const uint32_t* vals, size_t table_size,
                            const int32_t* out_coords, size_t n_out, size_t n_in, int W, int H, int D,
                            int Kw, int Kh, int Kd, int Sw, int Sh, int Sd, int Pw, int Ph, int Pd,
                            int Dw, int Dh, int Dd, uint32_t* map_fwd, uint32_t* map_bwd,
                            int32_t* gray, int32_t* binary, fgx_stream_t stream);

/* The same two maps (and codes) without a hash table, as fgx_subm_neighbor_map_sorted finds the submanifold map: the
 * input voxels are sorted by flattened key, the output voxels by the key of the cell their kernel position (0, 0, 0)
 * reads, and every group of 256 consecutive output voxels finds its neighbors of one (kx, ky) in one window of the
 * sorted inputs.  Takes the coordinates themselves; out_coords may be in any order.  key_bits: 32 when
 * B*W*H*D <= 2^32, else 64 (grids up to 2^62 cells).  workspace: fgx_spconv_neighbor_map_sorted_workspace_bytes bytes,
 * 256-byte aligned.
 * Replaces: the same reference function as fgx_spconv_neighbor_map. */
size_t fgx_spconv_neighbor_map_sorted_workspace_bytes(size_t n_in, size_t n_out, int key_bits, int Kw, int Kh);
int fgx_spconv_neighbor_map_sorted(const int32_t* in_coords, size_t n_in, const int32_t* out_coords, size_t n_out,
                                   int B, int W, int H, int D, int Kw, int Kh, int Kd, int Sw, int Sh, int Sd,
                                   int Pw, int Ph, int Pd, int Dw, int Dh, int Dd, int key_bits,
                                   void* workspace, size_t workspace_bytes, uint32_t* map_fwd, uint32_t* map_bwd,
                                   int32_t* gray, int32_t* binary, fgx_stream_t stream);

/* ---- Space-filling-curve codes of voxel coordinates -----------------------------------------------------------
 * mode: 1 = z-order (Morton), 2 = Hilbert (the values of SerializationMode, flex_gemm/ops/spconv/__init__.py:20-24).
 * coords int32[n, 4] = (b, x, y, z), 16-byte aligned.  bit_length = bits per spatial coordinate; x, y, z give bit i to
 * code bits 3i+2, 3i+1, 3i, the batch index sits above bit 3*bit_length.  code_bits: 32 (uint32 codes,
 * bit_length <= 10) or 64 (uint64, bit_length <= 21) -- the caller applies the width rule of
 * flex_gemm/ops/serialize.py:26-31.
 * Replace: z_order_encode / hilbert_encode and z_order_decode / hilbert_decode, flex_gemm/kernels/cuda/serialize/api.h:22-76
 * (device code z_order.h:22-40, hilbert.h:22-118).  Unlike z_order.h:29 the batch index is widened before the shift. */
int fgx_serialize_encode(int mode, const int32_t* coords, size_t n, int bit_length, int code_bits, void* codes,
                         fgx_stream_t stream);
int fgx_serialize_decode(int mode, const void* codes, size_t n, int bit_length, int code_bits, int32_t* coords,
                         fgx_stream_t stream);

/* out_coords = coords sorted by code (unsigned, ascending): encode, radix sort over batch_bits + 3*bit_length bits,
 * decode.  This is the order the reference leaves the output coordinates of the generic convolution in when
 * SERIALIZATION_MODE is Z_ORDER or HILBERT (its keys are these codes: sparse_neighbor_map.cu:156-187,
 * spconv/utils.h:47-107).  Coordinates must fit bit_length bits, batch indices batch_bits bits.
 * workspace: fgx_serialize_reorder_workspace_bytes(n, code_bits) bytes, 256-byte aligned; out_coords != coords. */
size_t fgx_serialize_reorder_workspace_bytes(size_t n, int code_bits);
int fgx_serialize_reorder_coords(int mode, const int32_t* coords, size_t n, int bit_length, int batch_bits, int code_bits,
                                 void* workspace, size_t workspace_bytes, int32_t* out_coords, fgx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FLEXGEMM_HIP_H */
