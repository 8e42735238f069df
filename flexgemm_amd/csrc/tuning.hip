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
    {2, 2, 17, 256, 256, {256, 128, 64, 1, 16384, 1}},
    {0, 2, 21, 32, 32, {256, 32, 64, 1, 0, 1}},
    {1, 2, 21, 32, 32, {256, 32, 64, 1, 0, 1}},
    {2, 2, 21, 32, 32, {32, 32, 64, 1, 16384, 1}},
    {0, 2, 15, 1024, 1024, {256, 128, 128, 1, 0, 1}},
    {1, 2, 15, 1024, 1024, {256, 128, 128, 1, 0, 1}},
    {2, 2, 15, 1024, 1024, {256, 128, 64, 1, 65536, 1}},
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
        // wgrad: square tiles over (Co, Ci); voxel blocks of 4096 to 12288 rows -- as long as that still leaves about
        // four items (block, offset, tile) per CU: every item costs an exposed epilogue and a partial product, while
        // blocks beyond ~12K rows overflow an XCD's L2 (measured at C = 128 ... 512: 12288 rows are 4 % to 11 % ahead of
        // 4096 once there are enough voxels) -- enlarged further until the fp32 partial products (blocks x V x Co x Ci)
        // stay below 256 MiB.
        int t = pick_cols(Ci < Co ? Ci : Co);
        out->tile_rows = t;
        out->tile_cols = t;
        out->slab_bytes = 64;
        out->splitk = 1;
        // persistent streaming kernel: 16-bit types; measured ahead of the tiled kernel from about two thousand voxels
        // on (both walk the same item list).  Its 32 x 32 tile
        // writes four partial products per voxel block (one per multiplying wavefront), so its blocks are four times
        // as long.
        // Under a weight of 512 x 512 channels and more it is ahead from the smallest layers on (C = 1024: 192 voxels 0.053 ->
        // 0.048 ms, 848 voxels 0.084 -> 0.072, 1 976 voxels 0.134 -> 0.115; C = 512: 1 976 voxels 0.055 -> 0.043).
        out->stream = (es == 2 && (n >= 2048 || (n >= 128 && (size_t)Ci * Co >= (size_t)512 * 512))) ? 1 : 0;
        // A weight of one 64 x 64 or 128 x 128 tile (33 ... 128 channels on both sides): the sweep (stream = 2) --
        // every workgroup keeps two accumulators over an eighth of the voxels, block_rows is its sub-block size.
        // Measured 20 % to 30 % ahead of the block-major kernel from ten thousand voxels (C = 128: 0.051 against
        // 0.067 ms) to 2.7 million (1.32 against 1.70 ms), for C = 64, 96, 128, coordinates in scan order or shuffled.
        if (es == 2 && n >= 8192 && n <= ((size_t)1 << 24) && t >= 64 && Ci <= t && Co <= t && V <= 2 * (kCUs / 8)) {
            out->stream = 2;
            out->block_rows = 2048;
            return;
        }
        // Wide weights on the streaming kernel: tiles of 256 (Co) x 128 (Ci) where they pad no more than 128 x 128 ones do.
        // A step then loads 48 KiB of rows for twice the products (24 instead of 32 KiB per 512 MFMA cycles), and these
        // shapes are bound by what the CUs can pull out of L2: C = 1024, 42 608 voxels 1.54 -> 1.34 ms; C = 512, 64 160
        // voxels 0.70 -> 0.58; C = 256, 252 392 voxels 0.71 -> 0.54 (with blocks of 16 384 rows, which suit the longer
        // tile better than 12 288: 0.58).
        // The same with the long side along Ci (128 x 256 tiles) where only the input side is wide.
        // (from about three thousand voxels on: below, the square tile's larger number of items counts for more)
        const bool tall = out->stream == 1 && n >= 3072 && t == 128 && Co > 128 && cdiv(Co, 256) * 256 == cdiv(Co, 128) * 128;
        const bool wide = out->stream == 1 && n >= 3072 && t == 128 && !tall && Ci > 128 && cdiv(Ci, 256) * 256 == cdiv(Ci, 128) * 128;
        if (tall) out->tile_rows = 256;
        if (wide) out->tile_cols = 256;
        const int slices = (out->stream && t == 32) ? 4 : 1;
        const double per_block = 4.0 * V * (double)Co * (double)Ci * slices;
        size_t max_blocks = (size_t)(268435456.0 / per_block);
        if (max_blocks < 1) max_blocks = 1;
        const size_t tiles = (size_t)cdiv(Co, out->tile_rows) * cdiv(Ci, out->tile_cols);
        size_t blocks_wanted = cdiv((size_t)4 * kCUs, (size_t)V * tiles);
        if (blocks_wanted < 1) blocks_wanted = 1;
        size_t rows = round_up(cdiv(n ? n : 1, blocks_wanted), 1024);
        if (rows < (size_t)4096 * slices) rows = (size_t)4096 * slices;
        const size_t longest = (tall || wide) ? 16384 : (size_t)12288 * slices;
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
