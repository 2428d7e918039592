// layout.h — resident ("tiled SoA") weight layout shared by the host repacker
// and the device kernels.
//
// The reference keeps GPU weights as [all scales][all codes] (SoA) and lets one
// warp walk one row (crates/oxibonsai-kernels/src/gpu_backend/cuda_graph/
// cudagraph_reformat_q1_aos_to_soa_group.rs:21-41, ..._tq2_blocks_to_soa_group.rs:16-27).
// Here the codes section is additionally tiled for the gfx950 int8 MFMA
// (v_mfma_i32_16x16x64_i8): a *row tile* is 16 weight rows, a *superblock* is 4
// consecutive 128-weight blocks (512 weights) and one wave64 dwordx4 load
// fetches exactly one 1 KiB unit that feeds 8 MFMAs with no shuffling.
//
// Lane numbering inside a wave: lane = g*16 + r, r = row within the tile
// (MFMA row), g = 32-weight group within a block (MFMA k-group).
//
//  Q1_0_g128 codes : unit (tile, sb) = 64 lanes x 16 B.
//     lane (r,g), dword q (0..3) = sign bits 32g..32g+31 of block 4*sb+q, row 16*tile+r
//     (bit i of the dword = weight 128*(4sb+q) + 32g + i; 1 -> +d, 0 -> -d).
//     The fp4 route of the GEMV (v_mfma_scale_f32_16x16x128_f8f6f4) reads the same dword as eight E2M1 nibbles:
//     bit m of nibble n is weight 4n + m, and the lane is again (row r, k-group g) of the B operand.
//
//  TQ2_0_g128 codes: unit (tile, sb, half) = 64 lanes x 16 B, half = 0,1.
//     lane (r,g), dword 2*e+m (e,m in 0..1) = the 16 two-bit fields of weights
//     32g+16m .. 32g+16m+15 of block 4*sb+2*half+e, field i at bits 2i..2i+1.
//     Fields are re-encoded so an AND with 0x03030303 << 2jj yields a usable
//     signed byte:   i%4 < 3 : field = value+1  (0,1,2  for -1,0,+1)
//                    i%4 == 3: field = value as 2-bit two's complement (3,0,1)
//     The reserved reference code 0b11 decodes to 0 like 0b01 and is stored as 0.
//
//  scales (both)   : unit (tile, sb) = 16 rows x 4 f16 = 128 B.
//     element [r][q] = f16 scale of block 4*sb+q, row 16*tile + r: the four scales a lane needs for one
//     superblock of its row are one 8-byte load.
//
// Rows are padded to a multiple of 16 and blocks to a multiple of 4 with zero
// scales and zero codes; padded entries contribute exactly 0.
#pragma once
#include <stddef.h>
#include <stdint.h>

#define OXB_QK 128
#define OXB_FMT_Q1 0
#define OXB_FMT_TQ2 1
#define OXB_Q1_AOS_BYTES 18
#define OXB_TQ2_AOS_BYTES 34

#ifdef __HIPCC__
#define OXB_HD __host__ __device__ inline
#else
#define OXB_HD inline
#endif

struct OxbLayout {
    uint32_t fmt;
    uint32_t n_rows, k;          // logical shape
    uint32_t n_tiles;            // ceil(n_rows / 16)
    uint32_t n_sb;               // ceil(k / 512)
    uint32_t unit_dwords;        // dwords per (tile, sb) code unit: 256 (Q1) or 512 (TQ2)
    uint64_t codes_bytes;        // size of the codes section (multiple of 1024)
    uint64_t scales_bytes;       // size of the scales section
};

OXB_HD OxbLayout oxb_make_layout(uint32_t fmt, uint32_t n_rows, uint32_t k) {
    OxbLayout L;
    L.fmt = fmt;
    L.n_rows = n_rows;
    L.k = k;
    L.n_tiles = (n_rows + 15u) / 16u;
    L.n_sb = (k + 511u) / 512u;
    L.unit_dwords = fmt == OXB_FMT_Q1 ? 256u : 512u;
    L.codes_bytes = (uint64_t)L.n_tiles * L.n_sb * L.unit_dwords * 4u;
    L.scales_bytes = (uint64_t)L.n_tiles * L.n_sb * 128u;
    return L;
}

// Dword index (within the codes section) holding the sign bits of weights
// 32g..32g+31 of block `blk`, row `row`.
OXB_HD uint64_t oxb_q1_dword_index(const OxbLayout& L, uint32_t row, uint32_t blk, uint32_t g) {
    uint32_t tile = row >> 4, r = row & 15u, sb = blk >> 2, q = blk & 3u;
    return ((uint64_t)tile * L.n_sb + sb) * 256u + (g * 16u + r) * 4u + q;
}

// Dword index holding the fields of weights 32g+16m .. +15 of block `blk`, row `row`.
OXB_HD uint64_t oxb_tq2_dword_index(const OxbLayout& L, uint32_t row, uint32_t blk, uint32_t g, uint32_t m) {
    uint32_t tile = row >> 4, r = row & 15u, sb = blk >> 2, q = blk & 3u;
    uint32_t half = q >> 1, e = q & 1u;
    return ((uint64_t)tile * L.n_sb + sb) * 512u + half * 256u + (g * 16u + r) * 4u + e * 2u + m;
}

// f16 index (within the scales section) of the scale of block `blk`, row `row`.
OXB_HD uint64_t oxb_scale_index(const OxbLayout& L, uint32_t row, uint32_t blk) {
    uint32_t tile = row >> 4, r = row & 15u, sb = blk >> 2, q = blk & 3u;
    return ((uint64_t)tile * L.n_sb + sb) * 64u + r * 4u + q;
}

// TQ2 field encoding: reference code (00 -> -1, 01 -> 0, 10 -> +1, 11 -> 0) to
// the stored field at in-dword position i, and back to the weight value.
OXB_HD uint32_t oxb_tq2_encode_field(uint32_t ref_code, uint32_t i) {
    int v = ref_code == 0u ? -1 : (ref_code == 2u ? 1 : 0);
    return (i & 3u) == 3u ? ((uint32_t)v & 3u) : (uint32_t)(v + 1);
}
OXB_HD int oxb_tq2_decode_field(uint32_t field, uint32_t i) {
    if ((i & 3u) == 3u) return field == 3u ? -1 : (field == 1u ? 1 : 0);
    return field == 0u ? -1 : (field == 2u ? 1 : 0);
}
