// Device side of the open-addressing hash table (Murmur3 finaliser modulo the table size, linear probing with
// wrap-around, all-ones key = empty slot, compare-and-swap insert, lock-free lookup), shared by the kernels that build
// and probe it.  Semantics follow the reference, flex_gemm/kernels/cuda/hash/hash.cuh:5-129.
#pragma once

#include <limits>

#include "fgx_common.h"

namespace fgx {

__device__ __forceinline__ uint32_t fmix(uint32_t k) {
    k ^= k >> 16;
    k *= 0x85ebca6bu;
    k ^= k >> 13;
    k *= 0xc2b2ae35u;
    k ^= k >> 16;
    return k;
}

__device__ __forceinline__ uint64_t fmix(uint64_t k) {
    k ^= k >> 33;
    k *= 0xff51afd7ed558ccdull;
    k ^= k >> 33;
    k *= 0xc4ceb9fe1a85ec53ull;
    k ^= k >> 33;
    return k;
}

template <typename K>
__device__ __forceinline__ size_t first_slot(K key, size_t table) {
    return (size_t)(fmix(key) % (K)table);
}
// 32-bit keys with a table of 2^32 slots or more: the modulus cannot be narrowed.
template <>
__device__ __forceinline__ size_t first_slot<uint32_t>(uint32_t key, size_t table) {
    uint32_t h = fmix(key);
    return table > 0xFFFFFFFFull ? (size_t)h : (size_t)(h % (uint32_t)table);
}

__device__ __forceinline__ uint32_t cas(uint32_t* p, uint32_t cmp, uint32_t val) { return atomicCAS(p, cmp, val); }
__device__ __forceinline__ uint64_t cas(uint64_t* p, uint64_t cmp, uint64_t val) {
    return (uint64_t)atomicCAS(reinterpret_cast<unsigned long long*>(p), (unsigned long long)cmp,
                               (unsigned long long)val);
}

template <typename K, typename Val>
__device__ __forceinline__ void probe_insert(K* keys, Val* vals, K key, Val val, size_t table) {
    constexpr K kEmpty = std::numeric_limits<K>::max();
    size_t slot = first_slot<K>(key, table);
    // A full table without the key would never end; bound the walk to one lap.
    for (size_t step = 0; step < table; ++step) {
        K prev = cas(&keys[slot], kEmpty, key);
        if (prev == kEmpty || prev == key) {
            vals[slot] = val;
            return;
        }
        slot = slot + 1;
        if (slot >= table) slot = 0;
    }
}

template <typename K, typename Val>
__device__ __forceinline__ Val probe_lookup(const K* keys, const Val* vals, K key, size_t table) {
    constexpr K kEmpty = std::numeric_limits<K>::max();
    size_t slot = first_slot<K>(key, table);
    for (size_t step = 0; step < table; ++step) {
        K prev = keys[slot];
        if (prev == kEmpty) break;
        if (prev == key) return vals[slot];
        slot = slot + 1;
        if (slot >= table) slot = 0;
    }
    return std::numeric_limits<Val>::max();
}

__device__ __forceinline__ uint64_t flat_key(int b, int x, int y, int z, int W, int H, int D) {
    return (((uint64_t)(uint32_t)b * (uint64_t)W + (uint64_t)x) * (uint64_t)H + (uint64_t)y) * (uint64_t)D + (uint64_t)z;
}

}  // namespace fgx
