// Plan of the resident-row kernels for narrow layers (conv_gemm_narrow.hip: forward and dgrad; wgrad_narrow.hip: weight
// gradient): the layout both read and fgx_narrow_plan writes.
//
//   header (kNarrowHeader bytes): word 0 = number of chunks that have more distinct sources than slots
//   then, per chunk of kNarrowRows rows (in the row order the plan was made for), narrow_plan_stride() bytes:
//     table    uint16 [kNarrowRows][32]   per (row, offset): byte offset, in the LDS row buffer, of the source row's first
//                                         16-byte piece (a row's four pieces are exchanged by its slot number, see
//                                         narrow_piece_key); the row of zeros when the neighbor is missing; entries from
//                                         V to 30: the row of zeros; kNarrowOverflow when the chunk has more distinct
//                                         sources than slots; entry 31: whether any entry of the row is kNarrowOverflow
//     sources  uint32 [kNarrowSlots]      source row of every slot, FGX_EMPTY32 beyond the chunk's count
//     rows     uint32 [kNarrowRows]       the chunk's rows (output rows of the gather GEMM), FGX_EMPTY32 beyond n
#pragma once
#include <stdint.h>

namespace fgx {
namespace {

constexpr int kNarrowRows = 128;                       // rows per chunk
constexpr int kNarrowSlots = 448;                      // source rows resident per chunk (a multiple of 64)
constexpr uint32_t kNarrowZeroSlot = kNarrowSlots;     // one more slot, all zeros
constexpr uint32_t kNarrowOverflow = 0xFFFFu;
constexpr uint32_t kNarrowOob = 0xFF000000u;           // buffer offset no tensor reaches: the load returns zeros
constexpr int kNarrowMaxV = 31;                        // (table entry 31 of a row is its overflow flag)
constexpr int kNarrowTableStride = 32;                 // table entries per row: a row's entries are four 16-byte reads
constexpr int kNarrowHeader = 256;
constexpr int kNarrowTableBytes = kNarrowRows * kNarrowTableStride * 2;                         // 8 KiB
constexpr int kNarrowPlanStride = kNarrowTableBytes + kNarrowSlots * 4 + kNarrowRows * 4;
constexpr int kNarrowRowBufBytes = (kNarrowSlots + 1) * 64;                                      // + the slot of zeros
constexpr int kNarrowRowBufPad = (kNarrowRowBufBytes + 1023) / 1024 * 1024;

// LDS position p of a row in slot s holds its logical 16-byte piece p ^ narrow_piece_key(s): the 16 lanes of a fragment
// read, which fall on arbitrary slots, then spread over the banks
__host__ __device__ constexpr uint32_t narrow_piece_key(uint32_t slot) { return (slot >> 2) & 3u; }

}  // namespace
}  // namespace fgx
