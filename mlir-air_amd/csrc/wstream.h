// Stream order: the device layout of one AWQ matrix W[K, N] for the whole-K streaming kernels.
//
// The checkpoint layout (qweight [K, N/8] int32, 8 columns per word) gives a workgroup that owns
// whole columns 4-byte pieces of rows that are N/2 bytes apart.  Like the reference, which re-packs
// every Linear into the order its cores consume it at load time (repack_for_gemv,
// programming_examples/llms/llama32_1b_int4/awq_repacker.py:112-135; pack_inputs,
// programming_examples/matrix_vector_multiplication/int4_awq/matvec_int4_packed.py:57-103), the
// weights are re-packed once into the order this GPU's kernels read them:
//
//   tile   = 16 output columns, all K rows: one contiguous slab of (NB + G) KiB, G = K / 128
//            groups, NB = ceil(G / 16) blocks; tile t starts at t * (NB + G) KiB
//   block  = 16 consecutive groups of a tile: [1 KiB of scales and zero points][one 1 KiB cell per
//            group]; block b starts 17 b KiB into the tile (only the last block can be short)
//   cell   = 16 columns x 128 rows of uint4 = 64 lanes x 16 bytes, i.e. one global_load_dwordx4
//            of a wavefront.  Lane l = 16 lg + ln, dword t (0..3), nibble at bits 4p..4p+3:
//                row    k = 128 g + 32 t + 8 lg + {0,2,4,6,1,3,5,7}[p]
//                column n = 16 tile + ln
//            which is the B operand of v_mfma_f32_16x16x32_bf16 for K-step t of the group: lane
//            (lg, ln) holds rows 8 lg .. 8 lg + 7 of column ln, and (dword >> 4 v) & 0x000F000F
//            is the pair (row 2 v, row 2 v + 1) that the operand's register v wants.
//   scales and zero points of a block: lane l, dword i (0..3) belongs to group 16 b + 4 lg + i and
//            column 16 tile + ln:  bits 0..15 the bf16 scale, bits 16..31 the bf16 value
//            -(128 + z) (0xC300 | z, exact).  Groups past the end of K hold 0.
//
// A matrix takes (N / 16) * (NB + G) KiB: K N / 2 bytes of nibbles plus 4 bytes per (group, column),
// 1.5 bytes more than the checkpoint's 2.5 (scales bf16 + packed zero points); for G a multiple of
// 16 that is 1.023 x the checkpoint bytes.
//
// Q4NX order (32-row sub-groups with a scale and a min each, w = s q + min'): the same tiles and cells; a block
// carries 4 KiB of scale / min words instead of 1: KiB t (0..3) belongs to K-step t of the cells, lane l, dword i to
// group 16 b + 4 lg + i, rows 32 t .. 32 t + 31 of it, column 16 tile + ln: bits 0..15 the bf16 scale, bits 16..31 the
// bf16 min'.  A tile is (4 NB + G) KiB, block b starts 20 b KiB into it: 5 bits per weight, as in the codec.
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace w4a16 {

constexpr int kWsTileCols = 16;
constexpr int kWsBlockGroups = 16;
constexpr size_t kWsCellBytes = 1024;

__host__ __device__ constexpr int ws_blocks(int K) { return (K / 128 + kWsBlockGroups - 1) / kWsBlockGroups; }
__host__ __device__ constexpr size_t ws_tile_bytes(int K) { return (size_t)(ws_blocks(K) + K / 128) * kWsCellBytes; }
__host__ __device__ constexpr size_t ws_matrix_bytes(int K, int N) { return (size_t)(N / kWsTileCols) * ws_tile_bytes(K); }
// Q4NX order: KiB of scale / min words per block, bytes of a tile and of a matrix
constexpr int kWsQ4MdKiB = 4;
__host__ __device__ constexpr size_t ws_q4_tile_bytes(int K) { return (size_t)(kWsQ4MdKiB * ws_blocks(K) + K / 128) * kWsCellBytes; }
__host__ __device__ constexpr size_t ws_q4_matrix_bytes(int K, int N) { return (size_t)(N / kWsTileCols) * ws_q4_tile_bytes(K); }

}  // namespace w4a16
