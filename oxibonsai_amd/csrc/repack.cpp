// repack.cpp — host-side AoS -> resident tiled-SoA repack (and its inverse).
//
// Replaces the reference's upload-time reformatters
//   reformat_q1_aos_to_soa        cuda_graph/cudagraph_reformat_q1_aos_to_soa_group.rs:21-41
//   reformat_tq2_blocks_to_soa    cuda_graph/cudagraph_reformat_tq2_blocks_to_soa_group.rs:16-27
// The TQ2 input is the block struct's own byte order [qs 32 B][d f16]
// (crates/oxibonsai-core/src/quant_ternary.rs:64-71), which is also what the
// model hands over as raw bytes (crates/oxibonsai-model/src/block/functions.rs:44-56).
#include "repack.h"

#include <algorithm>
#include <cstring>
#include <thread>
#include <vector>

namespace {

template <class F>
void parallel_tiles(uint32_t n_tiles, F&& fn) {
    unsigned hw = std::thread::hardware_concurrency();
    unsigned nt = std::max(1u, std::min(hw ? hw : 1u, 16u));
    if (n_tiles < 64 || nt == 1) {
        for (uint32_t t = 0; t < n_tiles; t++) fn(t);
        return;
    }
    std::vector<std::thread> th;
    for (unsigned w = 0; w < nt; w++)
        th.emplace_back([&, w] {
            for (uint32_t t = w; t < n_tiles; t += nt) fn(t);
        });
    for (auto& t : th) t.join();
}

inline uint32_t load_u32(const uint8_t* p) {
    uint32_t v;
    std::memcpy(&v, p, 4);
    return v;
}

}  // namespace

void oxb_repack_aos_to_tiled(const OxbLayout& L, const uint8_t* aos, uint32_t* codes, uint16_t* scales) {
    const uint32_t bpr = L.k / OXB_QK;
    std::memset(codes, 0, L.codes_bytes);
    std::memset(scales, 0, L.scales_bytes);
    parallel_tiles(L.n_tiles, [&](uint32_t tile) {
        for (uint32_t r = 0; r < 16; r++) {
            uint32_t row = tile * 16 + r;
            if (row >= L.n_rows) break;
            for (uint32_t blk = 0; blk < bpr; blk++) {
                if (L.fmt == OXB_FMT_Q1) {
                    const uint8_t* b = aos + ((size_t)row * bpr + blk) * OXB_Q1_AOS_BYTES;
                    scales[oxb_scale_index(L, row, blk)] = (uint16_t)(b[0] | (b[1] << 8));
                    for (uint32_t g = 0; g < 4; g++)
                        codes[oxb_q1_dword_index(L, row, blk, g)] = load_u32(b + 2 + 4 * g);
                } else {
                    const uint8_t* b = aos + ((size_t)row * bpr + blk) * OXB_TQ2_AOS_BYTES;
                    scales[oxb_scale_index(L, row, blk)] = (uint16_t)(b[32] | (b[33] << 8));
                    for (uint32_t dw = 0; dw < 8; dw++) {
                        uint32_t w = load_u32(b + 4 * dw), out = 0;
                        for (uint32_t i = 0; i < 16; i++)
                            out |= oxb_tq2_encode_field((w >> (2 * i)) & 3u, i) << (2 * i);
                        codes[oxb_tq2_dword_index(L, row, blk, dw >> 1, dw & 1u)] = out;
                    }
                }
            }
        }
    });
}

void oxb_repack_tiled_to_aos(const OxbLayout& L, const uint32_t* codes, const uint16_t* scales, uint8_t* aos) {
    const uint32_t bpr = L.k / OXB_QK;
    parallel_tiles(L.n_tiles, [&](uint32_t tile) {
        for (uint32_t r = 0; r < 16; r++) {
            uint32_t row = tile * 16 + r;
            if (row >= L.n_rows) break;
            for (uint32_t blk = 0; blk < bpr; blk++) {
                uint16_t d = scales[oxb_scale_index(L, row, blk)];
                if (L.fmt == OXB_FMT_Q1) {
                    uint8_t* b = aos + ((size_t)row * bpr + blk) * OXB_Q1_AOS_BYTES;
                    b[0] = (uint8_t)(d & 0xFF);
                    b[1] = (uint8_t)(d >> 8);
                    for (uint32_t g = 0; g < 4; g++) {
                        uint32_t w = codes[oxb_q1_dword_index(L, row, blk, g)];
                        std::memcpy(b + 2 + 4 * g, &w, 4);
                    }
                } else {
                    uint8_t* b = aos + ((size_t)row * bpr + blk) * OXB_TQ2_AOS_BYTES;
                    b[32] = (uint8_t)(d & 0xFF);
                    b[33] = (uint8_t)(d >> 8);
                    for (uint32_t dw = 0; dw < 8; dw++) {
                        uint32_t w = codes[oxb_tq2_dword_index(L, row, blk, dw >> 1, dw & 1u)], out = 0;
                        for (uint32_t i = 0; i < 16; i++) {
                            int v = oxb_tq2_decode_field((w >> (2 * i)) & 3u, i);
                            out |= (uint32_t)(v + 1) << (2 * i);  // canonical codes 00 / 01 / 10
                        }
                        std::memcpy(b + 4 * dw, &out, 4);
                    }
                }
            }
        }
    });
}
