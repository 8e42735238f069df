/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement (plain C, single thread) of the reference's
 * integer algorithms on the submanifold-conv hot path.  Nothing in the shipped package may
 * link, load or call this file; only tests/, the smoke check and the bench's cpu_baseline
 * leg use it, and only as the checker.
 *
 * Every function names the reference source it restates (paths relative to the reference
 * checkout).  The restatement is sequential: where the reference resolves races with
 * atomicCAS the sequential order "row 0, row 1, ..." is one of its legal executions.
 *
 * Pinning (see tests/test_oracle_*.py): fmix32/fmix64 against MurmurHash3 known answers;
 * the neighbor map against an independent numpy sort+searchsorted builder and a Python
 * dict brute force; gray/binary code against the closed forms; pair lists against
 * numpy.nonzero of the transposed map; tile masks against a direct OR over sorted rows.
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define REF_EMPTY32 0xFFFFFFFFu
#define REF_EMPTY64 0xFFFFFFFFFFFFFFFFull

/* flex_gemm/kernels/cuda/hash/hash.cuh:5-12 -- 32-bit Murmur3 finaliser */
uint32_t ref_fmix32(uint32_t k) {
    k ^= k >> 16;
    k *= 0x85ebca6bu;
    k ^= k >> 13;
    k *= 0xc2b2ae35u;
    k ^= k >> 16;
    return k;
}

/* flex_gemm/kernels/cuda/hash/hash.cuh:15-23 -- 64-bit Murmur3 finaliser */
uint64_t ref_fmix64(uint64_t k) {
    k ^= k >> 33;
    k *= 0xff51afd7ed558ccdull;
    k ^= k >> 33;
    k *= 0xc4ceb9fe1a85ec53ull;
    k ^= k >> 33;
    return k;
}

static size_t slot_of(uint64_t key, int key_bits, size_t table) {
    if (key_bits == 32) return (size_t)(ref_fmix32((uint32_t)key) % table);
    return (size_t)(ref_fmix64(key) % table);
}

static uint64_t load_key(const void* keys, int key_bits, size_t slot) {
    if (key_bits == 32) {
        uint32_t k = ((const uint32_t*)keys)[slot];
        return k == REF_EMPTY32 ? REF_EMPTY64 : (uint64_t)k;
    }
    return ((const uint64_t*)keys)[slot];
}

static void store_key(void* keys, int key_bits, size_t slot, uint64_t key) {
    if (key_bits == 32) ((uint32_t*)keys)[slot] = (uint32_t)key;
    else ((uint64_t*)keys)[slot] = key;
}

/* flex_gemm/ops/utils.py:4-19 -- key table filled with the all-ones sentinel */
void ref_hash_init(void* keys, int key_bits, size_t table) {
    memset(keys, 0xFF, table * (size_t)(key_bits / 8));
}

/* flex_gemm/kernels/cuda/hash/hash.cuh:65-107 -- linear probing insert (CAS -> plain compare) */
static void ref_insert(void* keys, int key_bits, uint32_t* vals, size_t table, uint64_t key, uint32_t val) {
    uint64_t cmp = key_bits == 32 ? (uint64_t)(uint32_t)key : key;
    size_t slot = slot_of(cmp, key_bits, table);
    for (;;) {
        uint64_t prev = load_key(keys, key_bits, slot);
        if (prev == REF_EMPTY64 || prev == cmp) {
            store_key(keys, key_bits, slot, cmp);
            vals[slot] = val;
            return;
        }
        slot = slot + 1;
        if (slot >= table) slot = 0;
    }
}

/* flex_gemm/kernels/cuda/hash/hash.cuh:110-129 -- lock-free lookup, absent -> all ones */
static uint32_t ref_lookup(const void* keys, int key_bits, const uint32_t* vals, size_t table, uint64_t key) {
    uint64_t cmp = key_bits == 32 ? (uint64_t)(uint32_t)key : key;
    size_t slot = slot_of(cmp, key_bits, table);
    for (;;) {
        uint64_t prev = load_key(keys, key_bits, slot);
        if (prev == REF_EMPTY64) return REF_EMPTY32;
        if (prev == cmp) return vals[slot];
        slot = slot + 1;
        if (slot >= table) slot = 0;
    }
}

static uint64_t flat_key(int64_t b, int64_t x, int64_t y, int64_t z, int W, int H, int D) {
    /* flex_gemm/kernels/cuda/hash/hash.cu:385 -- size_t arithmetic */
    return (uint64_t)b * (uint64_t)W * (uint64_t)H * (uint64_t)D + (uint64_t)x * (uint64_t)H * (uint64_t)D
         + (uint64_t)y * (uint64_t)D + (uint64_t)z;
}

/* flex_gemm/kernels/cuda/hash/hash.cu:368-391 -- value = row index */
void ref_hash_insert_idx_as_val(void* keys, int key_bits, uint32_t* vals, size_t table,
                                const int32_t* coords, size_t n, int W, int H, int D) {
    for (size_t i = 0; i < n; i++) {
        const int32_t* c = coords + 4 * i;
        ref_insert(keys, key_bits, vals, table, flat_key(c[0], c[1], c[2], c[3], W, H, D), (uint32_t)i);
    }
}

/* flex_gemm/kernels/cuda/hash/hash.cu:177-232 (insert_3d) -- user-supplied uint32 values */
void ref_hash_insert_3d(void* keys, int key_bits, uint32_t* vals, size_t table,
                        const int32_t* coords, const uint32_t* values, size_t n, int W, int H, int D) {
    for (size_t i = 0; i < n; i++) {
        const int32_t* c = coords + 4 * i;
        ref_insert(keys, key_bits, vals, table, flat_key(c[0], c[1], c[2], c[3], W, H, D), values[i]);
    }
}

/* flex_gemm/kernels/cuda/hash/hash.cu:272-331 (lookup_3d) -- out-of-grid query -> all ones */
void ref_hash_lookup_3d(const void* keys, int key_bits, const uint32_t* vals, size_t table,
                        const int32_t* coords, size_t n, int W, int H, int D, uint32_t* out) {
    for (size_t i = 0; i < n; i++) {
        const int32_t* c = coords + 4 * i;
        if (c[1] < 0 || c[1] >= W || c[2] < 0 || c[2] >= H || c[3] < 0 || c[3] >= D) { out[i] = REF_EMPTY32; continue; }
        out[i] = ref_lookup(keys, key_bits, vals, table, flat_key(c[0], c[1], c[2], c[3], W, H, D));
    }
}

/*
 * flex_gemm/kernels/cuda/spconv/subm_neighbor_map.cu:33-83 -- V/2+1 "threads" per voxel:
 * offsets 0..V/2-1 probe the table and also mirror-write the partner's row, offset V/2 is
 * the voxel itself.  `out` must be pre-filled with all ones (torch::full at :123).
 */
void ref_subm_neighbor_map(const void* keys, int key_bits, const uint32_t* vals, size_t table,
                           const int32_t* coords, size_t n, int W, int H, int D,
                           int Kw, int Kh, int Kd, int Dw, int Dh, int Dd, uint32_t* out) {
    int V = Kw * Kh * Kd;
    int half = V / 2 + 1;
    memset(out, 0xFF, n * (size_t)V * sizeof(uint32_t));
    for (size_t idx = 0; idx < n; idx++) {
        const int32_t* c = coords + 4 * idx;
        int b = c[0];
        int x = c[1] - Kw / 2 * Dw, y = c[2] - Kh / 2 * Dh, z = c[3] - Kd / 2 * Dd;
        for (int v = 0; v < half; v++) {
            uint32_t value = REF_EMPTY32;
            if (v == half - 1) {
                value = (uint32_t)idx;
            } else {
                int kx = x + v / (Kh * Kd) * Dw;
                int ky = y + v / Kd % Kh * Dh;
                int kz = z + v % Kd * Dd;
                if (kx >= 0 && kx < W && ky >= 0 && ky < H && kz >= 0 && kz < D) {
                    value = ref_lookup(keys, key_bits, vals, table, flat_key(b, kx, ky, kz, W, H, D));
                    if (value != REF_EMPTY32) out[(size_t)value * V + V - 1 - v] = (uint32_t)idx;
                }
            }
            out[idx * V + v] = value;
        }
    }
}

/* flex_gemm/kernels/cuda/spconv/migemm_neighmap_pp.cu:19-44 -- validity mask and its Gray decode */
void ref_gray_binary(const uint32_t* map, size_t n, int V, int32_t* gray, int32_t* binary) {
    for (size_t i = 0; i < n; i++) {
        uint32_t g = 0;
        for (int v = 0; v < V; v++) if (map[i * V + v] != REF_EMPTY32) g += 1u << v;
        uint32_t b = g;
        for (int v = 1; v < V; v++) b ^= g >> v;
        gray[i] = (int32_t)g;
        binary[i] = (int32_t)b;
    }
}

/*
 * flex_gemm/kernels/cuda/spconv/migemm_neighmap_pp.cu:85-154 (transposed map + 0/1 mask),
 * :224-225 (inclusive prefix sum) and :157-178 (compaction).  Pass sig_o = sig_i = NULL to
 * only obtain the segment table (and through seg[V] the pair count L).
 */
void ref_pair_lists(const uint32_t* map, size_t n, int V, uint32_t* sig_i, uint32_t* sig_o, uint32_t* seg) {
    size_t total = n * (size_t)V;
    uint32_t* map_t = (uint32_t*)malloc((total ? total : 1) * sizeof(uint32_t));
    int32_t* prefix = (int32_t*)malloc((total ? total : 1) * sizeof(int32_t));
    for (size_t i = 0; i < n; i++)
        for (int v = 0; v < V; v++) map_t[(size_t)v * n + i] = map[i * V + v];
    int32_t run = 0;
    for (size_t t = 0; t < total; t++) { run += map_t[t] != REF_EMPTY32; prefix[t] = run; }
    for (size_t t = 0; t < total; t++) {
        uint32_t value = map_t[t];
        if (value != REF_EMPTY32 && sig_i && sig_o) {
            int32_t to = prefix[t] - 1;
            sig_o[to] = (uint32_t)(t % n);
            sig_i[to] = value;
        }
    }
    for (int t = 0; t <= V; t++) seg[t] = t == 0 ? 0u : (n ? (uint32_t)prefix[(size_t)t * n - 1] : 0u);
    free(map_t);
    free(prefix);
}

/*
 * flex_gemm/kernels/cuda/spconv/migemm_neighmap_pp.cu:246-368 -- per tile of `block` consecutive
 * rows of the sorted order: OR of the masks, popcount -> exclusive offsets, set-bit positions.
 * Returns the number of entries written to valid_kernel (pass NULL to count only).
 */
int64_t ref_tile_masks(const int32_t* gray, const int64_t* sorted_idx, size_t n, int block,
                       int32_t* valid_kernel, int32_t* seg) {
    size_t nb = (n + (size_t)block - 1) / (size_t)block;
    int64_t total = 0;
    seg[0] = 0;
    for (size_t b = 0; b < nb; b++) {
        uint32_t code = 0;
        for (size_t r = b * block; r < (b + 1) * (size_t)block && r < n; r++) code |= (uint32_t)gray[sorted_idx[r]];
        uint32_t c = code;
        while (c) {
            int pos = __builtin_ctz(c);
            if (valid_kernel) valid_kernel[total] = pos;
            total++;
            c &= c - 1;
        }
        seg[b + 1] = (int32_t)total;
    }
    return total;
}
