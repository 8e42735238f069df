// Fixed gfx950 schedules for the masked implicit GEMM.
//
// The reference times every tile shape and every power-of-two SPLITK on first use and caches the
// winner per (2^floor(log2 N), Ci, Co, V) (flex_gemm/utils/autotuner.py:194-291; candidate ranges in
// ..._masked_implicit_gemm_splitk.py:109-126 and ..._bwd_..._splitk.py:185-202, 254-271).  Here the
// choice is a static function of (floor(log2 N), Ci, Co): a table of measured entries for the shapes
// that were tuned on an MI355X, and a rule for everything else.
#include "fgx_common.h"

namespace fgx {
namespace {

constexpr int kCUs = 256;

struct Entry {
    int pass_kind, dtype_bytes, log2n, ci, co;   // dtype_bytes: 2 or 4; 0 = any
    fgx_schedule s;
};

// Measured entries (MI355X).  Rows are matched exactly on (pass, element size, floor(log2 N), Ci, Co).
const Entry kTable[] = {
    // pass dtype log2n  Ci    Co    {rows, cols, slab_bytes, splitk, block_rows, stream}
    {0, 2, 19, 128, 128, {256, 128, 128, 1, 0, 1}},
    {1, 2, 19, 128, 128, {256, 128, 128, 1, 0, 1}},
    {2, 2, 19, 128, 128, {128, 128, 64, 1, 2048, 2}},
    {0, 2, 17, 256, 256, {128, 256, 128, 1, 0, 1}},
    {1, 2, 17, 256, 256, {128, 256, 128, 1, 0, 1}},
    {0, 2, 21, 32, 32, {256, 32, 64, 1, 0, 1}},
    {1, 2, 21, 32, 32, {256, 32, 64, 1, 0, 1}},
    {0, 2, 15, 1024, 1024, {256, 128, 128, 1, 0, 1}},
    {1, 2, 15, 1024, 1024, {256, 128, 128, 1, 0, 1}},
};

int floor_log2(size_t n) {
    int l = 0;
    while (n > 1) { n >>= 1; ++l; }
    return l;
}

int pick_cols(int c) { return c > 64 ? 128 : (c > 32 ? 64 : 32); }

size_t round_up(size_t x, size_t m) { return (x + m - 1) / m * m; }

void rule(int pass_kind, int es, size_t n, int Ci, int Co, int V, fgx_schedule* out) {
    if (pass_kind == 2) {
        // wgrad: tiles over (Co, Ci) and voxel blocks; an item is (block, offset, tile), every item costs an exposed
        // epilogue and a partial product, and the fp32 partial products (blocks x V x Co x Ci) stay below 256 MiB.
        int t = pick_cols(Ci < Co ? Ci : Co);
        out->tile_rows = t;
        out->tile_cols = t;
        out->slab_bytes = 64;
        out->splitk = 1;
        // persistent streaming kernel: 16-bit types; measured ahead of the tiled kernel from a few hundred voxels on
        // (848 voxels: C = 32 0.024 -> 0.020 ms, C = 64 0.023 -> 0.020, C = 128 0.031 -> 0.020, C = 256 0.033 -> 0.023).
        // Under a weight of 512 x 512 channels and more it is ahead from the smallest layers on (C = 1024: 192 voxels 0.053 ->
        // 0.048 ms, 848 voxels 0.084 -> 0.072, 1 976 voxels 0.134 -> 0.115; C = 512: 1 976 voxels 0.055 -> 0.043).
        out->stream = (es == 2 && (n >= 512 || (n >= 128 && (size_t)Ci * Co >= (size_t)512 * 512))) ? 1 : 0;
        // A weight of one 64 x 64 or 128 x 128 tile (33 ... 128 channels on both sides): the sweep (stream = 2) --
        // every workgroup keeps two accumulators over an eighth of the voxels, block_rows is its sub-block size.
        // Measured 20 % to 30 % ahead of the block-major kernel from ten thousand voxels (C = 128: 0.051 against
        // 0.067 ms) to 2.7 million (1.32 against 1.70 ms), for C = 64, 96, 128, coordinates in scan order or shuffled.
        if (es == 2 && n >= 8192 && n <= ((size_t)1 << 24) && t >= 64 && Ci <= t && Co <= t && V <= 2 * (kCUs / 8)) {
            out->stream = 2;
            out->block_rows = 2048;
            return;
        }
        // Streaming kernel with balanced work lists (fgx_wgrad_item_lists): a launch takes as long as its most loaded
        // workgroup, and the lists even the loads out as far as the items allow -- the largest item is the centre
        // offset of a voxel block (one pair per row), the mean load is about 0.45 V pairs per voxel x tiles / CUs.
        // So: the largest tile shape whose items still fill the chip one and a half times with blocks of 4096 rows or
        // more, and as few blocks as keep a block's centre item below the mean load (CUs / (0.45 V x tiles) blocks).
        // Measured on shells with the lists (ms, best of the swept tile shapes and block counts):
        //   C = 256:  848 voxels 64 x 64 tiles 1 block 0.023 (tiled kernel 0.033);  3 840: 64 x 64, 1 block 0.035
        //             (256 x 128: 0.063);  15 192: 128 x 128, 4 blocks 0.059 (256 x 128, 4: 0.077);  64 160: 256 x 128,
        //             8 blocks 0.156, 11: 0.169 (16: 0.176);  166 232: 256 x 128, 11 blocks 0.295 (8: 0.337, 24: 0.329)
        //   C = 512:  3 840: 128 x 128, 1 block 0.054 (256 x 128: 0.072);  15 192: 256 x 128, 2 blocks 0.144, 3: 0.150
        //             (4: 0.162);  64 160: 256 x 128, 3 blocks 0.484 (5: 0.503, 8: 0.520)
        //   C = 1024: 3 840 ... 64 160 voxels: 256 x 128, 1 block (42 608 voxels: 0.957, 2 blocks 1.02, 4: 1.12)
        //   C = 32:   15 192: 8 blocks 0.026 (1: 0.040);  64 160: 11 blocks 0.030 (4: 0.046, 32: 0.040)
        // Tiles of 256 x 128 (or 128 x 256 where only Ci is wide) where they pad no more than 128 x 128 ones do: a step
        // then loads 48 KiB of rows for twice the products, and these shapes are bound by what the CUs can pull out
        // of L2.  Below about three thousand voxels the square tile's larger number of items counts for more.
        if (out->stream == 1) {
            struct Shape { int rows, cols; };
            Shape shapes[3];
            int ns = 0;
            if (t == 128) {
                if (n >= 3072 && Co > 128 && cdiv(Co, 256) * 256 == cdiv(Co, 128) * 128) shapes[ns++] = {256, 128};
                else if (n >= 3072 && Ci > 128 && cdiv(Ci, 256) * 256 == cdiv(Ci, 128) * 128) shapes[ns++] = {128, 256};
                shapes[ns++] = {128, 128};
                shapes[ns++] = {64, 64};
            } else {
                shapes[ns++] = {t, t};
            }
            size_t nb = 1, tiles = 1;
            int slices = 1;
            for (int i = 0; i < ns; ++i) {
                const bool last = i == ns - 1;
                slices = shapes[i].rows == 32 ? 4 : 1;           // the 32 x 32 tile splits a step's pairs over its four wavefronts
                tiles = (size_t)cdiv(Co, shapes[i].rows) * cdiv(Ci, shapes[i].cols);
                const size_t per_voxel = (size_t)V * 4 / 9 * (slices == 4 ? 2 : 1);
                const size_t wanted = cdiv((size_t)kCUs, (per_voxel ? per_voxel : 1) * tiles);
                const size_t shortest = slices == 4 ? 2048 : 4096;
                const size_t most = n > shortest ? cdiv(n, shortest) : 1;
                nb = wanted < most ? wanted : most;
                out->tile_rows = shapes[i].rows;
                out->tile_cols = shapes[i].cols;
                const bool fills = 2 * (size_t)V * tiles * nb >= 3 * (size_t)kCUs;
                if (last && !fills) {                           // nothing fills the chip: blocks down to 2048 rows
                    const size_t most_short = n > 2048 ? cdiv(n, (size_t)2048) : 1;
                    nb = wanted < most_short ? wanted : most_short;
                }
                if (last || fills) break;
            }
            // long blocks overflow an XCD's L2 when few tiles share their rows; partial products stay below 256 MiB
            const size_t longest = tiles <= 4 ? 16384 : (tiles <= 8 ? 24576 : 65536);
            if (nb < cdiv(n, longest)) nb = cdiv(n, longest);
            size_t max_blocks = (size_t)(268435456.0 / (4.0 * V * (double)Co * (double)Ci * slices));
            if (max_blocks < 1) max_blocks = 1;
            if (nb > max_blocks) nb = max_blocks;
            // The lists exist for up to 12 voxel blocks (16 when a block has several tiles per offset); beyond, the fixed
            // interleave runs (it keeps the offsets of a voxel block on one XCD, and with that many blocks it is balanced
            // well enough) on the blocks below.
            if (nb <= (tiles >= 2 ? 16u : 12u)) {
                size_t rows = round_up(cdiv(n, nb), 1024);
                if (rows > 0x40000000) rows = 0x40000000;
                out->block_rows = (int)rows;
                return;
            }
        }
        // Fixed interleave (the tiled kernel: fp32 or few voxels; the streaming kernel over more than 12 blocks): voxel
        // blocks of 4096 to 12288 rows -- as long as that still leaves about four items per CU: blocks beyond ~12K rows
        // overflow an XCD's L2 (measured at C = 128 ... 512: 12288 rows are 4 % to 11 % ahead of 4096 once there are enough
        // voxels; 16384 under 256-row tiles and for the 32 x 32 streaming tile, which writes four partial products per
        // block: 1 026 536 voxels at 32 channels, 16384 rows 0.161 ms, 32768 0.170, 65536 0.185).
        const int slices = (out->stream && out->tile_rows == 32) ? 4 : 1;
        const double per_block = 4.0 * V * (double)Co * (double)Ci * slices;
        size_t max_blocks = (size_t)(268435456.0 / per_block);
        if (max_blocks < 1) max_blocks = 1;
        const size_t tiles = (size_t)cdiv(Co, out->tile_rows) * cdiv(Ci, out->tile_cols);
        size_t blocks_wanted = cdiv((size_t)4 * kCUs, (size_t)V * tiles);
        if (blocks_wanted < 1) blocks_wanted = 1;
        size_t rows = round_up(cdiv(n ? n : 1, blocks_wanted), 1024);
        if (rows < (size_t)4096 * slices) rows = (size_t)4096 * slices;        // (32 x 32: 16384, its longest as well)
        const size_t longest = (out->tile_rows == 256 || out->tile_cols == 256 || slices == 4) ? 16384 : 12288;
        if (rows > longest) rows = longest;
        const size_t rows_mem = round_up((n + max_blocks - 1) / max_blocks, 1024);
        if (rows < rows_mem) rows = rows_mem;
        // even blocks: with a handful of them a short last block leaves its workgroups idle (two blocks of 12288 + 2904
        // rows: 0.86 ms, of 8192 + 7000: 0.62 ms at C = 1024)
        if (n > 0) rows = round_up(cdiv(n, cdiv(n, rows)), 1024);
        if (rows > 0x40000000) rows = 0x40000000;
        out->block_rows = (int)rows;
        return;
    }
    const int cols = pass_kind == 0 ? Co : Ci;
    out->tile_cols = pick_cols(cols);
    out->tile_rows = n >= 4096 ? 128 : (n >= 1024 ? 64 : 32);
    if (out->tile_rows == 64 && out->tile_cols == 128) out->tile_rows = 128;
    if (out->tile_rows == 32 && out->tile_cols != 32) out->tile_rows = out->tile_cols == 64 ? 64 : 128;
    // narrow outputs with fewer 128-row tiles than CUs: 64-row tiles before any split of K (15 192 voxels, C = 64: 0.036 ->
    // 0.030 ms)
    if (out->tile_rows == 128 && out->tile_cols == 64 && (size_t)cdiv(n, 128) * cdiv(cols, 64) < (size_t)kCUs) out->tile_rows = 64;
    out->block_rows = 0;
    out->stream = 0;
    out->slab_bytes = 64;
    // split K only when the tiles cannot fill the chip (reference: candidates start at #SM / blocks)
    size_t tiles = (size_t)cdiv(n, out->tile_rows) * cdiv(cols, out->tile_cols);
    int s = 1;
    while (tiles * s < (size_t)kCUs && s < 16) s *= 2;
    out->splitk = s;
    // persistent streaming kernel (256-row tiles): rows of at least 64 bytes -- 128-byte K-slabs from 128 bytes on, 64-byte
    // ones below, where 32 output columns get a tile of their own.  With 128-byte slabs it is ahead of the tiled kernel
    // as soon as there is an item for a little under half of the CUs (measured: 120 items 10 % ahead, 64 items 13 %
    // behind); the short-row form, two workgroups per CU, keeps the bar of two items per CU.
    const int K = pass_kind == 0 ? Ci : Co;
    const size_t row_bytes = (size_t)K * es;
    // 16-bit rows of 128 ... 255 bytes (64 ... 127 channels) also take the 64-byte slabs: their rings leave room for two
    // workgroups per CU, which is worth more than the longer pieces (measured forward, C = 64: 143 616 / 252 392 / 577 592 /
    // 1 026 536 voxels -5 / -22 / -7 / -12 %; C = 80 and 96: -2 ... -5 %; from 256 bytes on the 128-byte slabs are ahead,
    // C = 128: 0.049 against 0.056 ms at 64 160 voxels)
    // ... given two items per CU to keep both workgroups busy (64 160 voxels, 251 items: 0.028 ms on 128-byte slabs, 0.031 on
    // 64-byte ones)
    const bool short_slabs = es == 2 && row_bytes >= 128 && row_bytes < 256 &&
                             (size_t)cdiv(n, 256) * cdiv(cols, cols > 64 ? 128 : 64) >= 2 * (size_t)kCUs;
    const int slab = (row_bytes >= 128 && !short_slabs) ? 128 : 64;
    int scols = cols > 64 ? 128 : ((cols > 32 || row_bytes >= 128) ? 64 : 32);
    const size_t enough = row_bytes >= 128 ? (size_t)kCUs * 7 / 16 : 2 * (size_t)kCUs;
    if (row_bytes >= 64 && (slab == 64 || cols >= 64) && (size_t)cdiv(n, 256) * cdiv(cols, scols) >= enough &&
        stream_lds_fits(256, scols, slab, cols)) {      // (from ~1900 output columns on the staged bias no longer fits)
        out->tile_rows = 256;
        out->tile_cols = scols;
        out->slab_bytes = slab;
        out->splitk = 1;
        out->stream = 1;
        // 129 ... 256 output columns on 128-byte slabs: one tile of 128 rows x 256 columns instead of two of 256 x 128 -- the
        // same bytes loaded per product, every row gathered once instead of twice, and 128-row tiles pad less (measured,
        // C = 256: -6 % at 15 192 voxels, -5 % at 252 392, -2 % at 1 026 536; C = 160 and 192 at 252 392 voxels: -8 %, -7 %;
        // beyond 256 columns the 256-row tile stays ahead)
        if (slab == 128 && cols > 128 && cols <= 256 && stream_lds_fits(128, 256, slab, cols)) {
            out->tile_rows = 128;
            out->tile_cols = 256;
        }
        // Half a chip's worth of items or fewer: tiles of 64 columns make twice as many, and a gathered row read twice
        // from L2 costs less than idle CUs (measured forward: 15 192 voxels C = 256, 119 items, 0.074 -> 0.064 ms; 3 840
        // voxels C = 1024, 120 items, 0.270 -> 0.223 ms).
        if (slab == 128 && out->tile_cols >= 128 &&
            (size_t)cdiv(n, out->tile_rows) * cdiv(cols, out->tile_cols) <= (size_t)kCUs / 2 && stream_lds_fits(256, 64, slab, cols)) {
            out->tile_rows = 256;
            out->tile_cols = 64;
        }
    } else if (es == 2 && row_bytes >= 1024 && cols >= 128) {
        // Too few tiles to stream and rows of 1 KiB or more (512 channels of a 16-bit type): a few hundred or thousand voxels
        // under a weight of tens of megabytes.  The tiled kernel on 256 x 128 tiles and 128-byte slabs, with as many K
        // splits as give every CU one workgroup, keeps more of the weight in flight than 128 x 128 tiles on 64-byte slabs
        // (measured forward, C = 1024: 192 voxels 0.048 -> 0.042 ms, 848 voxels 0.090 -> 0.084, 1 976 voxels 0.227 -> 0.138;
        // C = 512: 1 976 voxels 0.073 -> 0.054, 3 840 voxels 0.094 -> 0.085, 5 816 voxels 0.145 -> 0.133; at C = 256 the
        // smaller tiles are level).
        out->tile_rows = 256;
        out->tile_cols = 128;
        out->slab_bytes = 128;
        const size_t wide_items = (size_t)cdiv(n ? n : 1, 256) * cdiv(cols, 128);
        int sk = 1;
        while (wide_items * (size_t)sk * 2 <= (size_t)kCUs && sk < 32) sk *= 2;
        out->splitk = sk;
    }
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" int fgx_table_lookup(int pass_kind, int dtype, size_t n, int Ci, int Co, int V, fgx_schedule* out) {
    FGX_CHECK_ARG(out != nullptr, "fgx_table_lookup: null output");
    FGX_CHECK_ARG(pass_kind >= 0 && pass_kind <= 2, "fgx_table_lookup: pass_kind must be 0 (fwd), 1 (dgrad) or 2 (wgrad)");
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16 || dtype == FGX_F32, "fgx_table_lookup: unknown dtype %d", dtype);
    FGX_CHECK_ARG(Ci > 0 && Co > 0 && V >= 1, "fgx_table_lookup: bad shape");
    const int es = dtype == FGX_F32 ? 4 : 2;
    const int l2 = floor_log2(n ? n : 1);
    for (const Entry& e : kTable) {
        if (e.pass_kind == pass_kind && (e.dtype_bytes == 0 || e.dtype_bytes == es) && e.log2n == l2 && e.ci == Ci && e.co == Co) {
            *out = e.s;
            if (pass_kind != 2 && out->stream && !stream_lds_fits(out->tile_rows, out->tile_cols, out->slab_bytes, pass_kind == 0 ? Co : Ci))
                break;      // (cannot happen for the shapes listed; the rule decides then)
            return FGX_OK;
        }
    }
    rule(pass_kind, es, n, Ci, Co, V, out);
    return FGX_OK;
}
