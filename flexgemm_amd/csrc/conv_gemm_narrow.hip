// Gather GEMM for narrow layers (16-bit types, source rows and output rows of at most 64 bytes: up to 32 channels on
// both sides) with the gathered rows RESIDENT in LDS.
//
// The streaming kernel gathers every source row once per (tile, offset): 10.5 row requests per voxel on a shell, each
// for a 64-byte row, and the memory system serves such requests at ~95 G/s whatever asks for them -- configuration 4
// (2.67 M voxels, 28.1 M pairs) cannot go below 0.29 ms that way.  Here the rows walk in chunks of 128 consecutive
// voxels of a Z-order curve; a chunk's output rows need ~220 distinct source rows (1.72 per voxel instead of 10.5), which
// a plan names once per neighbor cache.  Per chunk the loaders put those rows into LDS (direct-to-LDS loads), together
// with the chunk's table "which LDS slot holds the source of (row, offset)", and the multipliers run ALL offsets for
// all rows -- a missing neighbor is the slot of zeros -- because with K = 32 a product is two MFMAs and skipping would
// cost more instructions than it saves.  The weight (V x 2 KiB) stays in LDS for the whole launch.
//
// (the plan's layout: narrow_plan.h)
//
// Workgroup: 4 multiplying wavefronts (32 chunk rows each, one 32 x 32 accumulator) + 4 loading wavefronts; two LDS
// buffers (the loads run one chunk ahead), one barrier per chunk.  Persistent: XCD x walks the x-th eighth of the chunks, its workgroups interleave, so
// that neighboring chunks -- which share their halo rows -- run on one L2 at one time.
#include "gemm_device.h"
#include "narrow_plan.h"

namespace fgx {
namespace {

using rsrc_t = __amdgpu_buffer_rsrc_t;

__device__ __forceinline__ rsrc_t narrow_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

constexpr int kNarrowHash = 1024;                // hash table of the plan builder (a power of two)

// ------------------------------------------------------------------------------------------------
// Plan builder: one workgroup per chunk.  The distinct neighbors of the chunk's rows go through a hash table in LDS;
// slots are numbered in table order, so the plan depends on the chunk's set of sources alone.
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(64) narrow_plan_header_kernel(uint32_t* __restrict__ header) { header[threadIdx.x] = 0u; }

__global__ void __launch_bounds__(256) narrow_plan_kernel(const uint32_t* __restrict__ nmap, const int64_t* __restrict__ order,
                                                          uint32_t n, int V, int own_rows, unsigned char* __restrict__ plan) {
    __shared__ uint32_t keys[kNarrowHash];
    __shared__ uint16_t slot_of[kNarrowHash];
    __shared__ uint32_t scan[256];
    __shared__ uint32_t row_flags[kNarrowRows / 32];
    __shared__ uint32_t grow_of[kNarrowRows];                                       // the chunk's rows (FGX_EMPTY32 beyond n)
    __shared__ __attribute__((aligned(16))) uint16_t table_lds[kNarrowRows * kNarrowTableStride];   // leaves as 16-byte stores
    const int tid = threadIdx.x;
    const uint32_t chunk = blockIdx.x;
    unsigned char* mine = plan + kNarrowHeader + (size_t)chunk * kNarrowPlanStride;
    uint32_t* sources = (uint32_t*)(mine + kNarrowTableBytes);
    uint32_t* rows = sources + kNarrowSlots;
    for (int i = tid; i < kNarrowHash; i += 256) keys[i] = FGX_EMPTY32;
    if (tid < kNarrowRows / 32) row_flags[tid] = 0u;
    for (int r = tid; r < kNarrowRows; r += 256) {
        const uint32_t gr = chunk * kNarrowRows + (uint32_t)r;
        grow_of[r] = gr < n ? (order ? (uint32_t)order[gr] : gr) : FGX_EMPTY32;
    }
    // entries from V on: the row of zeros (entry 31, the row's overflow flag, is written at the end)
    for (int i = tid; i < kNarrowRows * kNarrowTableStride; i += 256) table_lds[i] = (uint16_t)(kNarrowZeroSlot * 64u);
    __syncthreads();
    const int entries = kNarrowRows * V;
    auto source_of = [&](int e) -> uint32_t {
        const uint32_t grow = grow_of[e / V];
        if (grow == FGX_EMPTY32) return FGX_EMPTY32;
        return nmap[(size_t)grow * V + (e % V)];
    };
    auto hash = [](uint32_t x) -> uint32_t { return (x * 2654435761u) >> 22; };      // 10 bits
    auto insert = [&](uint32_t idx) -> int {                                         // table position, -1 when the table is full
        uint32_t h = hash(idx);
        for (int probe = 0; probe < kNarrowHash; ++probe) {
            const uint32_t old = atomicCAS(&keys[h], FGX_EMPTY32, idx);
            if (old == FGX_EMPTY32 || old == idx) return (int)h;
            h = (h + 1) & (kNarrowHash - 1);
        }
        return -1;
    };
    // A chunk row that is also a source row (the same voxels on both sides: every row is its own centre neighbor) takes
    // the slot of its chunk row number: the 16 rows of a fragment read then fall on 16 different slots modulo 16 for
    // the centre offset and on nearly as many for the others -- the neighbors of consecutive rows are mostly
    // consecutive rows -- which is what keeps the reads of arbitrary slots off each other's banks.
    for (int i = tid; i < kNarrowHash; i += 256) slot_of[i] = (uint16_t)kNarrowOverflow;
    __syncthreads();
    if (own_rows) {
        for (int r = tid; r < kNarrowRows; r += 256) {
            if (grow_of[r] != FGX_EMPTY32) {
                const int pos = insert(grow_of[r]);
                if (pos >= 0) slot_of[pos] = (uint16_t)r;
            }
        }
        __syncthreads();
    }
    // (a thread's entries stay in registers for the second pass: kNarrowRows * kNarrowMaxV / 256 of them at most; all
    // of them are fetched before the first goes into the table, so that their latencies overlap)
    constexpr int kPerThread = (kNarrowRows * 32 + 255) / 256;
    uint32_t mine_idx[kPerThread];
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const int e = tid + j * 256;
        mine_idx[j] = e < entries ? source_of(e) : FGX_EMPTY32;
    }
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
        if (mine_idx[j] != FGX_EMPTY32) insert(mine_idx[j]);
    __syncthreads();
    // the other sources: slots from `base` on in table order (exclusive scan of their positions, four per thread)
    const uint32_t base = own_rows ? (uint32_t)kNarrowRows : 0u;
    if (own_rows) {
        for (int r = tid; r < kNarrowRows; r += 256) sources[r] = grow_of[r];
    }
    uint32_t own = 0;
    for (int j = 0; j < 4; ++j) own += (keys[tid * 4 + j] != FGX_EMPTY32 && slot_of[tid * 4 + j] == kNarrowOverflow) ? 1u : 0u;
    scan[tid] = own;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
        const uint32_t add = tid >= d ? scan[tid - d] : 0u;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    uint32_t next = base + scan[tid] - own;
    for (int j = 0; j < 4; ++j) {
        const int pos = tid * 4 + j;
        if (keys[pos] != FGX_EMPTY32 && slot_of[pos] == kNarrowOverflow) {
            if (next < (uint32_t)kNarrowSlots) {
                slot_of[pos] = (uint16_t)next;
                sources[next] = keys[pos];
            }
            ++next;
        }
    }
    const uint32_t total = base + scan[255];
    for (uint32_t s = total + tid; s < (uint32_t)kNarrowSlots; s += 256) sources[s] = FGX_EMPTY32;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const int e = tid + j * 256;
        if (e >= entries) break;
        const uint32_t idx = mine_idx[j];
        uint16_t out = (uint16_t)kNarrowZeroSlot;
        if (idx != FGX_EMPTY32) {
            out = (uint16_t)kNarrowOverflow;
            uint32_t h = hash(idx);
            for (int probe = 0; probe < kNarrowHash; ++probe) {
                const uint32_t k = keys[h];
                if (k == idx) { out = slot_of[h]; break; }
                if (k == FGX_EMPTY32) break;
                h = (h + 1) & (kNarrowHash - 1);
            }
        }
        // what the multipliers read: the byte offset of the row's logical piece 0 in the row buffer
        if (out != (uint16_t)kNarrowOverflow) out = (uint16_t)(out * 64u + (((uint32_t)out >> 2) & 3u) * 16u);
        table_lds[(e / V) * kNarrowTableStride + (e % V)] = out;
        if (out == (uint16_t)kNarrowOverflow) atomicOr(&row_flags[(e / V) >> 5], 1u << ((e / V) & 31));
    }
    __syncthreads();
    for (int r = tid; r < kNarrowRows; r += 256)
        table_lds[r * kNarrowTableStride + kNarrowTableStride - 1] = (uint16_t)((row_flags[r >> 5] >> (r & 31)) & 1u);
    if (tid == 0 && (row_flags[0] | row_flags[1] | row_flags[2] | row_flags[3]) != 0u) atomicAdd((uint32_t*)plan, 1u);
    for (int r = tid; r < kNarrowRows; r += 256) rows[r] = grow_of[r];
    __syncthreads();
    {
        const uint4* from = (const uint4*)table_lds;
        uint4* to = (uint4*)mine;                       // (the plan and its chunks are 16-byte aligned)
        for (int i = tid; i < kNarrowTableBytes / 16; i += 256) to[i] = from[i];
    }
}

// ------------------------------------------------------------------------------------------------
// The GEMM.  LDS: weight [V][32 cols][64 B], two buffers of { rows [kNarrowSlots + 1][64 B], table, output rows },
// (a multiplier stages its output tile in its own rows of the table).  64-byte rows are kept with their four 16-byte pieces exchanged by
// (slot >> 2) & 3, so that the 32 lanes of a fragment read, which fall on arbitrary slots, spread over the banks.
// ------------------------------------------------------------------------------------------------
constexpr int kNarrowMult = 4, kNarrowLoad = 4, kNarrowThreads = 64 * (kNarrowMult + kNarrowLoad);
constexpr int kNarrowBuffers = 2;                              // chunks in LDS: one multiplied, one on its way (a third, two
                                                               // chunks ahead, measured the same)

__host__ __device__ constexpr int narrow_buffer_bytes(int V) { return kNarrowRowBufPad + kNarrowTableBytes + 1024; }
__host__ __device__ constexpr size_t narrow_lds_bytes(int V) {
    return (size_t)V * 2048 + (size_t)kNarrowBuffers * narrow_buffer_bytes(V);
}

// four fp32 values rounded (to nearest even) to four 16-bit ones
template <typename T> __device__ __forceinline__ uint64_t pack4(const float (&x)[4]);
template <> __device__ __forceinline__ uint64_t pack4<_Float16>(const float (&x)[4]) {
    using h4 = _Float16 __attribute__((ext_vector_type(4)));
    using f4 = float __attribute__((ext_vector_type(4)));
    const f4 v = {x[0], x[1], x[2], x[3]};
    return __builtin_bit_cast(uint64_t, __builtin_convertvector(v, h4));
}
template <> __device__ __forceinline__ uint64_t pack4<__bf16>(const float (&x)[4]) {
    using b4 = __bf16 __attribute__((ext_vector_type(4)));
    using f4 = float __attribute__((ext_vector_type(4)));
    const f4 v = {x[0], x[1], x[2], x[3]};
    return __builtin_bit_cast(uint64_t, __builtin_convertvector(v, b4));
}

// VT: the kernel volume when it is known at compile time (the offsets' loop is then unrolled and the compiler runs the
// LDS reads of later offsets under the MFMAs of earlier ones), 0: any V <= 32
template <typename Tag, int VT>
__global__ void __launch_bounds__(kNarrowThreads)
narrow_gemm_kernel(const typename Tag::type* __restrict__ src, const typename Tag::type* __restrict__ panel,
                   const typename Tag::type* __restrict__ bias, const uint32_t* __restrict__ nmap,
                   const unsigned char* __restrict__ plan, uint32_t chunks, uint32_t plan_bytes, uint32_t src_bytes, int V,
                   int K, int cols, int activation, typename Tag::type* __restrict__ out, uint8_t* __restrict__ relu_mask) {
    using T = typename Tag::type;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    unsigned char* weight_lds = lds;                                            // [V][32][64 B], pieces exchanged by (col >> 2) & 3
    unsigned char* buffers = lds + (size_t)V * 2048;
    const int buffer_bytes = narrow_buffer_bytes(V);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool loader = wave >= kNarrowMult;
    const int row_bytes = K * 2, out_row_bytes = cols * 2;
    const int stride = kNarrowPlanStride, table_bytes = kNarrowTableBytes;

    // ---- chunks of this workgroup: XCD x owns the x-th eighth, its workgroups interleave ----
    const unsigned G = gridDim.x;
    const unsigned xcd = blockIdx.x % kXcds, slot_in_xcd = blockIdx.x / kXcds, per_round = G / kXcds;
    const unsigned per_xcd = (chunks + kXcds - 1) / kXcds;
    const unsigned range_lo = xcd * per_xcd, range_hi = (xcd + 1) * per_xcd < chunks ? (xcd + 1) * per_xcd : chunks;
    const unsigned first = range_lo + slot_in_xcd;

    // ---- once: the weight into LDS, zeros into the zero slot of both buffers ----
    for (int u = tid; u < V * 128; u += kNarrowThreads) {                        // 16-byte pieces: [v][col][piece]
        const int col = (u >> 2) & 31, piece = u & 3;
        const u32x4 w = *reinterpret_cast<const u32x4*>((const unsigned char*)panel + (size_t)u * 16);
        *reinterpret_cast<u32x4*>(weight_lds + (u >> 2) * 64 + ((piece ^ ((col >> 2) & 3)) << 4)) = w;
    }
    if (tid < 4 * kNarrowBuffers) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4*>(buffers + (size_t)(tid >> 2) * buffer_bytes + kNarrowSlots * 64 + (tid & 3) * 16) = zero;
    }
    if (first >= range_hi) return;                                              // whole workgroup

    const rsrc_t src_rs = narrow_rsrc(src, src_bytes);
    const rsrc_t plan_rs = narrow_rsrc(plan, plan_bytes);

    // Loaders: wavefront lw issues, per chunk, the row loads of the slot groups (j * 4 + lw) * 16 ... + 15 (j = 0 ... 5),
    // every fourth KiB of the table, and (lw == 3) the output rows.  The source rows of the chunk after next are fetched
    // into registers while the current loads fly.
    const int lw = loader ? wave - kNarrowMult : 0;
    constexpr int kGroups = kNarrowSlots / 16 / kNarrowLoad;                     // 6
    uint32_t ids[kGroups];
    auto fetch_ids = [&](unsigned chunk) {
#pragma unroll
        for (int j = 0; j < kGroups; ++j) {
            const uint32_t s = (uint32_t)((j * kNarrowLoad + lw) * 16 + (lane >> 2));
            ids[j] = __builtin_amdgcn_raw_buffer_load_b32(plan_rs, (uint32_t)kNarrowHeader + chunk * (uint32_t)stride + (uint32_t)table_bytes + s * 4u, 0, 0);
        }
    };
    auto enqueue = [&](unsigned chunk, int b) {
        unsigned char* buf = buffers + (size_t)b * buffer_bytes;
#pragma unroll
        for (int j = 0; j < kGroups; ++j) {
            const int group = j * kNarrowLoad + lw;
            const uint32_t s = (uint32_t)(group * 16 + (lane >> 2));
            const uint32_t piece = (uint32_t)(lane & 3) ^ ((s >> 2) & 3u);       // LDS position lane & 3 holds this piece
            const bool live = ids[j] != FGX_EMPTY32 && (int)(piece * 16) < row_bytes;
            const uint32_t vo = live ? ids[j] * (uint32_t)row_bytes + piece * 16u : kNarrowOob;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src_rs, FGX_LDS_PTR(buf + group * 1024), 16, vo, 0, 0, 0);
        }
        const int table_insts = kNarrowTableBytes / 1024;
        for (int j = lw; j < table_insts; j += kNarrowLoad)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(plan_rs, FGX_LDS_PTR(buf + kNarrowRowBufPad + j * 1024), 16,
                                                     (uint32_t)kNarrowHeader + chunk * (uint32_t)stride + (uint32_t)(j * 1024 + lane * 16), 0, 0, 0);
        if (lw == kNarrowLoad - 1) {
            const uint32_t vo = lane < kNarrowRows * 4 / 16
                                    ? (uint32_t)kNarrowHeader + chunk * (uint32_t)stride + (uint32_t)table_bytes + kNarrowSlots * 4u + (uint32_t)lane * 16u
                                    : kNarrowOob;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(plan_rs, FGX_LDS_PTR(buf + kNarrowRowBufPad + kNarrowTableBytes), 16, vo, 0, 0, 0);
        }
    };

    // Multipliers: wavefront mw owns chunk rows mw * 32 ... + 31.
    const int mw = loader ? 0 : wave;
    const int l32 = lane & 31, g = lane >> 5;
    float bias_e[16];                                                           // accumulator element e is column ...
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int col = (e >> 2) * 8 + g * 4 + (e & 3);
        bias_e[e] = (bias != nullptr && col < cols) ? to_float<T>(bias[col]) : 0.f;
    }

    // One chunk ahead: in the iteration that multiplies chunk i the loaders enqueue chunk i + 1 (its source rows are in
    // registers since the iteration before) and fetch the source rows of chunk i + 2; at the end of the iteration they
    // wait until chunk i + 1 has landed -- everything but the fetch, which was issued last (loads return in order).
    if (loader) {
        fetch_ids(first);
        enqueue(first, 0);
        if (first + per_round < range_hi) fetch_ids(first + per_round);
    }
    __builtin_amdgcn_s_waitcnt(0);                                              // the weight and zero stores, the first loads
    __syncthreads();

    int b = 0;
    for (unsigned chunk = first; chunk < range_hi; chunk += per_round, b ^= 1) {
        if (loader) {
            const unsigned next = chunk + per_round;
            const bool enqueues = next < range_hi, fetches = next + per_round < range_hi;
            if (enqueues) {
                enqueue(next, b ^ 1);
                if (fetches) fetch_ids(next + per_round);
            }
            if (fetches) wait_vmcnt<kGroups>();
            else wait_vmcnt<0>();
        } else {
            const unsigned char* buf = buffers + (size_t)b * buffer_bytes;
            const uint16_t* table = (const uint16_t*)(buf + kNarrowRowBufPad);
            const uint32_t* out_rows = (const uint32_t*)(buf + kNarrowRowBufPad + kNarrowTableBytes);
            const int r = mw * 32 + l32;
            // Products are taken as (weight fragment) x (row fragment): the accumulator then holds, per lane, ONE chunk row
            // (r) and sixteen output columns in four runs of four -- 8 bytes each, stored straight from the registers.
            // One accumulator per half of K (sums in a fixed order, like everything here).
            f32x16 acc, acc1;
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[e] = acc1[e] = 0.f;
            // this row's table entries: 32 x uint16 in four 16-byte reads; entry 31 says whether any of them is kNarrowOverflow
            u32x4 ent[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) ent[q] = *reinterpret_cast<const u32x4*>((const unsigned char*)table + r * (kNarrowTableStride * 2) + q * 16);
            auto entry = [&](int v) -> uint32_t {
                const uint32_t word = ent[v >> 3][(v >> 1) & 3];
                return (v & 1) ? word >> 16 : word & 0xFFFFu;
            };
            const uint32_t grow = out_rows[r];
            const uint32_t wkey = ((uint32_t)l32 >> 2) & 3u;
            const unsigned char* wrow0 = weight_lds + l32 * 64 + (((uint32_t)g ^ wkey) << 4);
            const unsigned char* wrow1 = weight_lds + l32 * 64 + (((uint32_t)(g + 2) ^ wkey) << 4);
            // (a table entry is the byte offset of a row's logical piece 0; piece q sits at entry ^ (q << 4))
            if (__builtin_expect(__any(entry(kNarrowTableStride - 1) != 0u), 0)) {
                // a chunk with more distinct sources than slots: lanes whose source is not resident read it from memory
                for (int v = 0; v < V; ++v) {
                    const uint32_t s = table[r * kNarrowTableStride + v];
                    const uint32_t off = s == kNarrowOverflow ? kNarrowZeroSlot * 64u : s;
                    u32x4 a0 = *reinterpret_cast<const u32x4*>(buf + (off ^ ((uint32_t)g << 4)));
                    u32x4 a1 = *reinterpret_cast<const u32x4*>(buf + (off ^ ((uint32_t)g << 4) ^ 32u));
                    if (s == kNarrowOverflow && grow != FGX_EMPTY32) {
                        const uint32_t id = nmap[(size_t)grow * V + v];
                        if (id != FGX_EMPTY32) {
                            const u32x4 zero = {0u, 0u, 0u, 0u};
                            const unsigned char* p = (const unsigned char*)src + (size_t)id * row_bytes;
                            a0 = g * 16 < row_bytes ? *reinterpret_cast<const u32x4*>(p + g * 16) : zero;
                            a1 = (g + 2) * 16 < row_bytes ? *reinterpret_cast<const u32x4*>(p + (g + 2) * 16) : zero;
                        }
                    }
                    mma<Tag>(acc, *reinterpret_cast<const u32x4*>(wrow0 + v * 2048), a0);
                    mma<Tag>(acc1, *reinterpret_cast<const u32x4*>(wrow1 + v * 2048), a1);
                }
            } else if constexpr (VT > 0) {
                // The fragment reads run kAhead offsets ahead of the products (kAhead + 1 register sets): with one multiplying
                // wavefront per SIMD nothing else hides the LDS latency, and left to itself the compiler issues every
                // read right before its use.
                constexpr int kAhead = 2, kSets = kAhead + 1;        // (3, 4 and 6 ahead measure the same)
                u32x4 fa0[kSets], fa1[kSets], fb0[kSets], fb1[kSets];
                auto fetch = [&](int v, int set) __attribute__((always_inline)) {
                    const uint32_t at = entry(v) ^ ((uint32_t)g << 4);
                    fa0[set] = *reinterpret_cast<const u32x4*>(buf + at);
                    fa1[set] = *reinterpret_cast<const u32x4*>(buf + (at ^ 32u));
                    fb0[set] = *reinterpret_cast<const u32x4*>(wrow0 + v * 2048);
                    fb1[set] = *reinterpret_cast<const u32x4*>(wrow1 + v * 2048);
                };
#pragma unroll
                for (int v = 0; v < kAhead && v < VT; ++v) fetch(v, v % kSets);
#pragma unroll
                for (int v = 0; v < VT; ++v) {
                    if (v + kAhead < VT) fetch(v + kAhead, (v + kAhead) % kSets);
                    __builtin_amdgcn_sched_barrier(0);
                    mma<Tag>(acc, fb0[v % kSets], fa0[v % kSets]);
                    mma<Tag>(acc1, fb1[v % kSets], fa1[v % kSets]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll 4
                for (int v = 0; v < V; ++v) {
                    const uint32_t at = (uint32_t)table[r * kNarrowTableStride + v] ^ ((uint32_t)g << 4);
                    const u32x4 a0 = *reinterpret_cast<const u32x4*>(buf + at);
                    const u32x4 a1 = *reinterpret_cast<const u32x4*>(buf + (at ^ 32u));
                    mma<Tag>(acc, *reinterpret_cast<const u32x4*>(wrow0 + v * 2048), a0);
                    mma<Tag>(acc1, *reinterpret_cast<const u32x4*>(wrow1 + v * 2048), a1);
                }
            }
            // epilogue: accumulator element e is column (e >> 2) * 8 + g * 4 + (e & 3) of chunk row r
            if (grow != FGX_EMPTY32) {
                unsigned char* orow = (unsigned char*)out + (size_t)grow * out_row_bytes;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int col0 = i * 8 + g * 4;
                    if (i * 8 < cols) {                                          // cols is a multiple of 8: whole pieces
                        float x[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) x[j] = activate(acc[i * 4 + j] + acc1[i * 4 + j] + bias_e[i * 4 + j], activation);
                        const uint64_t packed = pack4<T>(x);
                        *reinterpret_cast<uint64_t*>(orow + col0 * 2) = packed;
                        if (relu_mask != nullptr) {
                            // the piece's other four columns are in lane ^ 32
                            uint32_t bits = 0;
#pragma unroll
                            for (int j = 0; j < 4; ++j) bits |= (x[j] > 0.f ? 1u : 0u) << j;
                            const uint32_t other = (uint32_t)__shfl_xor((int)bits, 32, 64);
                            if (g == 0) relu_mask[((size_t)grow * out_row_bytes >> 4) + i] = (uint8_t)(bits | (other << 4));
                        }
                    }
                }
            }
        }
        if (!loader) __builtin_amdgcn_s_waitcnt(0);          // the stage has been read, the output is on its way
        __syncthreads();
    }
}

template <typename Tag>
int launch_narrow(const void* src, const void* panel, const void* bias, const uint32_t* nmap, const void* plan, size_t n,
                  size_t n_src, int V, int K, int cols, int activation, void* out, uint8_t* relu_mask, hipStream_t s) {
    using T = typename Tag::type;
    const uint32_t chunks = (uint32_t)((n + kNarrowRows - 1) / kNarrowRows);
    int dev = 0, cus = 0;
    FGX_CHECK_HIP(hipGetDevice(&dev));
    FGX_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    unsigned groups = (unsigned)(cus > 0 ? cus : 256);
    groups = groups / kXcds * kXcds;
    if (groups < (unsigned)kXcds) groups = kXcds;
    auto kern = V == 27 ? narrow_gemm_kernel<Tag, 27> : narrow_gemm_kernel<Tag, 0>;
    const size_t lds = narrow_lds_bytes(V);
    static thread_local bool raised = false;
    if (!raised) {
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)narrow_gemm_kernel<Tag, 27>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)narrow_gemm_kernel<Tag, 0>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    kern<<<groups, kNarrowThreads, lds, s>>>((const T*)src, (const T*)panel, (const T*)bias, nmap, (const unsigned char*)plan, chunks,
                                             (uint32_t)(kNarrowHeader + (size_t)chunks * kNarrowPlanStride), (uint32_t)(n_src * (size_t)K * 2), V, K,
                                             cols, activation, (T*)out, relu_mask);
    FGX_CHECK_LAUNCH("fgx_conv_narrow_gemm");
    return FGX_OK;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

size_t fgx_narrow_plan_bytes(size_t n, int V) {
    if (V < 1 || V > kNarrowMaxV) return 0;
    return kNarrowHeader + ((n + kNarrowRows - 1) / kNarrowRows) * (size_t)kNarrowPlanStride;
}

int fgx_narrow_plan(const uint32_t* map, const int64_t* order, size_t n, int V, int same_rows, void* plan, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= kNarrowMaxV, "fgx_narrow_plan: bad kernel volume %d", V);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_narrow_plan: too many rows");
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(map && plan, "fgx_narrow_plan: null buffer");
    FGX_CHECK_ARG(((uintptr_t)plan & 15) == 0, "fgx_narrow_plan: plan must be 16-byte aligned");
    FGX_CHECK_ARG(fgx_narrow_plan_bytes(n, V) < 0xFF000000ull, "fgx_narrow_plan: plan of %zu rows passes the 32-bit offset range", n);
    const unsigned chunks = (unsigned)((n + kNarrowRows - 1) / kNarrowRows);
    narrow_plan_header_kernel<<<1, 64, 0, (hipStream_t)stream>>>((uint32_t*)plan);
    FGX_CHECK_LAUNCH("fgx_narrow_plan(header)");
    narrow_plan_kernel<<<chunks, 256, 0, (hipStream_t)stream>>>(map, order, (uint32_t)n, V, same_rows ? 1 : 0, (unsigned char*)plan);
    FGX_CHECK_LAUNCH("fgx_narrow_plan");
    return FGX_OK;
}

int fgx_conv_narrow_gemm(int dtype, const void* src, const void* panel, const void* bias, const uint32_t* map, const void* plan,
                         size_t n, size_t n_src, int K, int cols, int V, int activation, void* out, uint8_t* relu_mask,
                         fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16, "fgx_conv_narrow_gemm: 16-bit types only, got dtype %d", dtype);
    FGX_CHECK_ARG(V >= 1 && V <= kNarrowMaxV, "fgx_conv_narrow_gemm: bad kernel volume %d", V);
    FGX_CHECK_ARG(K >= 8 && K <= 32 && K % 8 == 0 && cols >= 8 && cols <= 32 && cols % 8 == 0,
                  "fgx_conv_narrow_gemm: K = %d and cols = %d must be 8, 16, 24 or 32", K, cols);
    FGX_CHECK_ARG(activation == FGX_ACT_NONE || activation == FGX_ACT_RELU, "fgx_conv_narrow_gemm: unknown activation %d", activation);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull && (double)n_src * K * 2 < (double)0xFF000000u, "fgx_conv_narrow_gemm: operand too large for 32-bit offsets");
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(src && panel && map && plan && out, "fgx_conv_narrow_gemm: null buffer");
    FGX_CHECK_ARG((((uintptr_t)src | (uintptr_t)panel | (uintptr_t)out | (uintptr_t)plan) & 15) == 0, "fgx_conv_narrow_gemm: buffers must be 16-byte aligned");
    FGX_CHECK_ARG(fgx_narrow_plan_bytes(n, V) < 0xFF000000ull, "fgx_conv_narrow_gemm: plan passes the 32-bit offset range");
    FGX_CHECK_ARG(narrow_lds_bytes(V) <= 160 * 1024, "fgx_conv_narrow_gemm: kernel volume %d does not fit LDS", V);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FGX_F16) return launch_narrow<F16>(src, panel, bias, map, plan, n, n_src, V, K, cols, activation, out, relu_mask, s);
    return launch_narrow<BF16>(src, panel, bias, map, plan, n, n_src, V, K, cols, activation, out, relu_mask, s);
}

}  // extern "C"
