// repack.h — host-side conversion between the reference's AoS blocks and the
// resident tiled-SoA layout described in layout.h.
#pragma once
#include "layout.h"

// aos: n_rows * (k/128) blocks in the reference's on-disk byte order.
// codes / scales: buffers of L.codes_bytes / L.scales_bytes.
void oxb_repack_aos_to_tiled(const OxbLayout& L, const uint8_t* aos, uint32_t* codes, uint16_t* scales);

// Inverse; TQ2 codes come back canonical (a reserved 0b11 input returns as 0b01,
// both decode to weight 0).
void oxb_repack_tiled_to_aos(const OxbLayout& L, const uint32_t* codes, const uint16_t* scales, uint8_t* aos);
