// gemv_kernels.hip — Q1_0_g128 / TQ2_0_g128 GEMV for gfx950 (MI355X).
//
// What it computes (reference: crates/oxibonsai-kernels/src/gemv.rs:60-84,
// gemv_ternary.rs:83-102):  y[row] = sum_blocks f16(d) * sum_128 code(w) * x.
//
// Why int8 MFMA and not per-weight VALU decode.  At 8 TB/s a Q1 stream delivers
// 64e12 weights/s, but the chip retires only ~39e12 non-packed VALU lane-ops/s
// (256 CU x 64 lanes x 2.4 GHz), so any scheme that spends >= 1 VALU op per
// weight is compute-bound at < 61 % of the HBM roofline.  Here a weight costs
// 1/4 VALU op: one AND with 0x01010101 << j (Q1) or 0x03030303 << 2jj (TQ2)
// turns a code dword into four int8 MFMA operands worth 2^j (4^jj) each, and the
// activation vector is pre-divided by the same power of two when it is
// quantised.  The fp32 activation is carried exactly: each x is scaled by a
// per-vector power of two to a 54-bit integer (every element within 2^22 of the
// largest one keeps all 24 mantissa bits) and split into eight balanced int8
// digits which occupy eight MFMA columns, so one 16x16x64 MFMA multiplies 16
// rows x 64 weights by all eight digits of up to two activation vectors.
// Block sums are exact integers; the per-block f16 scale is applied in fp32.
//
// Kernels:
//   quant_x_kernel   x[batch][k] fp32 -> int8 digit planes in MFMA B-operand order
//   gemv_mfma_kernel codes/scales (tiled SoA, see layout.h) x digit planes -> y
//   dequant_kernel   resident layout -> fp32 weights (bit-exactness check)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemv_kernels.h"
#include "layout.h"
#include "quant_device.h"


// The activation quantiser (quant_device.h) produces the MFMA B operands ("digit planes").
#define OXB_QUANT_THREADS 256

// Grid (vectors, parts): each workgroup takes whole exponent groups of one vector, finds their maxima and
// quantises them; no workgroup needs anything from another.
template <int FMT>
__global__ __launch_bounds__(OXB_QUANT_THREADS) void quant_x_kernel(const float* __restrict__ x, uint32_t k, uint32_t NC,
                                                                     uint32_t gsb, uint32_t n_groups,
                                                                     uint32_t* __restrict__ xq,
                                                                     int32_t* __restrict__ cneg,
                                                                     int32_t* __restrict__ xexp) {
    __shared__ uint32_t gstat[2 * OXB_XQ_MAX_GROUPS];
    const uint32_t n = blockIdx.x;
    const uint32_t per = (n_groups + gridDim.y - 1) / gridDim.y, g0 = blockIdx.y * per;
    const uint32_t g1 = g0 + per < n_groups ? g0 + per : n_groups;
    if (g0 >= g1) return;
    const float* xn = x + (size_t)n * k;
    gstat_scan(xn, k, gsb, g0, g1, gstat);
    quantise_groups<FMT>(xn, k, NC, n, gsb, n_groups, g0, g1, gstat, xq, cneg, xexp);
}

// ---------------------------------------------------------------------------
// GEMV.  One workgroup = S waves; wave s owns superblocks
// [sb_begin + s*NSBW, +NSBW) of every row tile the workgroup processes and keeps
// the matching slice of the digit planes in registers for the whole kernel, so
// the inner loop is: one coalesced 1 KiB code load per superblock, 4 ANDs + 1
// MFMA per 64 weights of 16 rows, 4 cvt + 4 fma per block for the scale.
// Partial row sums of the S waves meet in LDS; the last step weighs and adds the eight digit
// columns (DPP) and applies the epilogue (store / +=).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}

// Codes and scales of one row tile, restricted to this wave's K slice, as they wait in registers.
template <int FMT, int NSBW>
struct TileRegs {
    static constexpr int UNITS = (FMT == OXB_FMT_Q1) ? 1 : 2;  // 1 KiB code units per superblock
    v4i w[NSBW][UNITS];
    uint32_t sc[NSBW];  // lane (c, rg): f16 pair (c & 7) of row group rg, pair 2q+p = scales of block q, rows 2p, 2p+1
};

// `valid`, `tile` and the unit index are wave-uniform: they travel in scalar registers, the lane
// part of the address (lane_c, lane_s) is fixed for the whole kernel.
template <int FMT, int NSBW>
__device__ __forceinline__ void load_tile(TileRegs<FMT, NSBW>& t, __amdgpu_buffer_rsrc_t codes,
                                          __amdgpu_buffer_rsrc_t scales, uint32_t tile, bool valid, uint32_t n_sb,
                                          uint32_t sb0, int sb_lim, uint32_t lane_c, uint32_t lane_s) {
    constexpr int UNITS = TileRegs<FMT, NSBW>::UNITS;
#pragma unroll
    for (int i = 0; i < NSBW; i++) {
        const bool ok = valid && i < sb_lim;
        const uint32_t unit = __builtin_amdgcn_readfirstlane(tile * n_sb + sb0 + (uint32_t)i);
#pragma unroll
        for (int u = 0; u < UNITS; u++) t.w[i][u] = buf_load_b128(codes, ok ? lane_c : OXB_OOB, (unit * UNITS + u) * 1024u);
        t.sc[i] = buf_load_b32(scales, ok ? lane_s : OXB_OOB, unit * 128u);
    }
}

// One block: two MFMAs over its 128 weights, then the f16 scale in fp32.
template <int FMT, int Q>
__device__ __forceinline__ void block_mac(v4f& accf, uint32_t d0, uint32_t d1, const v4i& b0, const v4i& b1,
                                          const v4i& c4, uint32_t scdw) {
    v4i a0, a1;
    if (FMT == OXB_FMT_Q1) {  // d0 == d1: 32 sign bits
        a0 = (v4i){(int)(d0 & 0x01010101u), (int)(d0 & 0x02020202u), (int)(d0 & 0x04040404u), (int)(d0 & 0x08080808u)};
        a1 = (v4i){(int)(d0 & 0x10101010u), (int)(d0 & 0x20202020u), (int)(d0 & 0x40404040u), (int)(d0 & 0x80808080u)};
    } else {  // 16 two-bit fields each
        a0 = (v4i){(int)(d0 & 0x03030303u), (int)(d0 & 0x0C0C0C0Cu), (int)(d0 & 0x30303030u), (int)(d0 & 0xC0C0C0C0u)};
        a1 = (v4i){(int)(d1 & 0x03030303u), (int)(d1 & 0x0C0C0C0Cu), (int)(d1 & 0x30303030u), (int)(d1 & 0xC0C0C0C0u)};
    }
    v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b0, c4, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b1, acc, 0, 0, 0);
    const uint32_t p0 = dpp_u32<OXB_DPP_ROW_NEWBCAST(2 * Q)>(scdw);      // scales of rows 4g+0, 4g+1
    const uint32_t p1 = dpp_u32<OXB_DPP_ROW_NEWBCAST(2 * Q + 1)>(scdw);  // rows 4g+2, 4g+3
    accf[0] = fmaf((float)acc[0], f16_bits_to_f32(p0 & 0xFFFFu), accf[0]);
    accf[1] = fmaf((float)acc[1], f16_bits_to_f32(p0 >> 16), accf[1]);
    accf[2] = fmaf((float)acc[2], f16_bits_to_f32(p1 & 0xFFFFu), accf[2]);
    accf[3] = fmaf((float)acc[3], f16_bits_to_f32(p1 >> 16), accf[3]);
}

// Workgroup wg handles row tiles [wg * groups * TG, +groups * TG); TG tiles are in flight per
// wave at any time and are recombined together.  All control flow is uniform and branch-free
// inside a group, so the compiler can wait for exactly the tile it is about to use.
template <int FMT, int NSBW, int TG>
__global__ __launch_bounds__(512, (NSBW == 1 ? 4 : 2)) void gemv_mfma_kernel(const OxbGemvParams p) {
    extern __shared__ float part[];  // [2][TG][S][NC][16]
    constexpr int UNITS = TileRegs<FMT, NSBW>::UNITS;
    const uint32_t lane = threadIdx.x & 63u, s = threadIdx.x >> 6, S = blockDim.x >> 6;
    const uint32_t c = lane & 15u, g = lane >> 4;  // B operand: column c, k-group g; D: column c, rows 4g..4g+3
    const uint32_t NC = p.NC;
    const bool col_on = c < NC;

    const uint32_t lane_c = lane * 16u, lane_s = ((lane >> 4) * 8u + (lane & 7u)) * 4u;
    const uint32_t sb0 = __builtin_amdgcn_readfirstlane(p.sb_begin + s * NSBW);
    const int sb_lim = (int)(p.sb_begin + p.sb_count) - (int)sb0;  // superblocks of this wave's slice that exist

    const __amdgpu_buffer_rsrc_t r_codes = make_rsrc(p.codes, p.codes_bytes);
    const __amdgpu_buffer_rsrc_t r_scales = make_rsrc(p.scales, p.scales_bytes);
    const __amdgpu_buffer_rsrc_t r_xq = make_rsrc(p.xq, p.xq_bytes);
    const __amdgpu_buffer_rsrc_t r_cneg = make_rsrc(p.cneg, p.cneg_bytes);

    // Digit planes and accumulator start values of this wave's K slice (L2-resident), issued
    // first so that the weight stream behind them can be consumed tile by tile as it arrives.
    v4i B[NSBW][4][2];
    v4i C4[NSBW][4];
#pragma unroll
    for (int i = 0; i < NSBW; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const bool ok = col_on && i < sb_lim;
            const uint32_t blk = (sb0 + (uint32_t)i) * 4 + q;
            B[i][q][0] = buf_load_b128(r_xq, ok ? (((blk * 2 + 0) * 4 + g) * NC + c) * 16u : OXB_OOB);
            B[i][q][1] = buf_load_b128(r_xq, ok ? (((blk * 2 + 1) * 4 + g) * NC + c) * 16u : OXB_OOB);
            C4[i][q] = buf_load_b128(r_cneg, ok ? (blk * NC + c) * 16u : OXB_OOB);
        }
    // In the recombination, thread t handles column (t % NC): digit (t % 8) of vector (t % NC) / 8, and needs
    // the exponent of every wave's K slice (= exponent group) of that vector.
    __shared__ int xes[2 * 8];  // [vector][wave]; published by the first barrier of the tile loop
    if (threadIdx.x < 16) {
        const uint32_t vec = threadIdx.x >> 3, w = threadIdx.x & 7u;
        xes[threadIdx.x] = (vec * 8 < NC && w < S) ? p.xexp[vec * p.n_groups + p.sb_begin / NSBW + w] : 0;
    }
    const uint32_t my_vec = (threadIdx.x % NC) >> 3;

    const uint32_t tpw = p.groups * TG, t_begin = blockIdx.x * tpw;
    const uint32_t t_end = (t_begin + tpw) < p.n_tiles ? (t_begin + tpw) : p.n_tiles;

    // The scheduling barriers pin the issue order of the loads: memory returns in issue order, so
    // "tile t has arrived" is a wait for all but the loads issued after it.
    __builtin_amdgcn_sched_barrier(0);
    TileRegs<FMT, NSBW> ring[TG];
#pragma unroll
    for (int t = 0; t < TG; t++) {
        load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, t_begin + t, t_begin + t < t_end, p.n_sb, sb0, sb_lim, lane_c, lane_s);
        __builtin_amdgcn_sched_barrier(0);
    }

    for (uint32_t grp = 0; grp < p.groups; grp++) {
        float* buf = part + (size_t)(grp & 1u) * TG * S * NC * 16;
#pragma unroll
        for (int t = 0; t < TG; t++) {
            const uint32_t tile = t_begin + grp * TG + t;
            v4f accf = {0.f, 0.f, 0.f, 0.f};
            const TileRegs<FMT, NSBW>& r = ring[t];
#pragma unroll
            for (int i = 0; i < NSBW; i++) {
                if (FMT == OXB_FMT_Q1) {
                    block_mac<FMT, 0>(accf, r.w[i][0][0], r.w[i][0][0], B[i][0][0], B[i][0][1], C4[i][0], r.sc[i]);
                    block_mac<FMT, 1>(accf, r.w[i][0][1], r.w[i][0][1], B[i][1][0], B[i][1][1], C4[i][1], r.sc[i]);
                    block_mac<FMT, 2>(accf, r.w[i][0][2], r.w[i][0][2], B[i][2][0], B[i][2][1], C4[i][2], r.sc[i]);
                    block_mac<FMT, 3>(accf, r.w[i][0][3], r.w[i][0][3], B[i][3][0], B[i][3][1], C4[i][3], r.sc[i]);
                } else {
                    block_mac<FMT, 0>(accf, r.w[i][0][0], r.w[i][0][1], B[i][0][0], B[i][0][1], C4[i][0], r.sc[i]);
                    block_mac<FMT, 1>(accf, r.w[i][0][2], r.w[i][0][3], B[i][1][0], B[i][1][1], C4[i][1], r.sc[i]);
                    block_mac<FMT, 2>(accf, r.w[i][UNITS - 1][0], r.w[i][UNITS - 1][1], B[i][2][0], B[i][2][1], C4[i][2], r.sc[i]);
                    block_mac<FMT, 3>(accf, r.w[i][UNITS - 1][2], r.w[i][UNITS - 1][3], B[i][3][0], B[i][3][1], C4[i][3], r.sc[i]);
                }
            }
            // refill this ring slot with the tile TG ahead (reads nothing past the workgroup's range)
            load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile + TG, tile + TG < t_end, p.n_sb, sb0, sb_lim, lane_c, lane_s);
            __builtin_amdgcn_sched_barrier(0);
            if (col_on) *reinterpret_cast<v4f*>(&buf[(((size_t)t * S + s) * NC + c) * 16 + g * 4]) = accf;
        }
        lds_barrier();
        // thread -> (slot, row, column): add the S partial sums in a fixed order, weigh the digit
        // by 2^(8 digit + E - P), then add the eight digit columns of a vector across lanes.
        for (uint32_t idx = threadIdx.x; idx < (uint32_t)TG * 16 * NC; idx += blockDim.x) {
            const uint32_t cc = idx % NC, rr = (idx / NC) & 15u, slot = idx / (16 * NC);
            float v = 0.f;
            bool nan = false;
#pragma unroll
            for (int w = 0; w < 8; w++)
                if ((uint32_t)w < S) {
                    const int xe = xes[my_vec * 8 + w];
                    nan |= xe == INT32_MIN;
                    v += ldexpf(buf[(((size_t)slot * S + w) * NC + cc) * 16 + rr], xe + 8 * (int)(cc & 7u));
                }
            if (nan) v = __int_as_float(0x7FC00000);
            v += dpp_f32<OXB_DPP_ROW_SHR(1)>(v);
            v += dpp_f32<OXB_DPP_ROW_SHR(2)>(v);
            v += dpp_f32<OXB_DPP_ROW_SHR(4)>(v);
            const uint32_t tile = t_begin + grp * TG + slot, row = tile * 16 + rr;
            if ((cc & 7u) == 7u && tile < t_end && row < p.n_rows) {
                const size_t o = (size_t)(cc >> 3) * p.ldy + row;
                if (p.mode == OXB_GEMV_ACCUM) v += p.y[o];
                else if (p.mode == OXB_GEMV_RESIDUAL) v += p.residual[o];
                p.y[o] = v;
            }
        }
        // no second barrier: the next group writes the other half of `part`
    }
}

// ---------------------------------------------------------------------------
// Resident layout -> fp32 weights, row-major [n_rows][k]
// (reference: crates/oxibonsai-kernels/src/dequant.rs:15-37, dequant_ternary.rs:42-64).
// One thread per (row, block, 32-weight group).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dequant_kernel(OxbLayout L, const uint32_t* __restrict__ codes,
                                                       const uint16_t* __restrict__ scales, float* __restrict__ out) {
    const uint32_t bpr = L.k / OXB_QK;
    const uint64_t total = (uint64_t)L.n_rows * bpr * 4;
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= total) return;
    const uint32_t g = (uint32_t)(id & 3u);
    const uint32_t blk = (uint32_t)((id >> 2) % bpr), row = (uint32_t)((id >> 2) / bpr);
    const float d = f16_bits_to_f32(scales[oxb_scale_index(L, row, blk)]);
    float* o = out + (size_t)row * L.k + blk * 128 + g * 32;
    if (L.fmt == OXB_FMT_Q1) {
        const uint32_t w = codes[oxb_q1_dword_index(L, row, blk, g)];
        for (uint32_t i = 0; i < 32; i++) o[i] = ((w >> i) & 1u) ? d : -d;
    } else {
        for (uint32_t m = 0; m < 2; m++) {
            const uint32_t w = codes[oxb_tq2_dword_index(L, row, blk, g, m)];
            for (uint32_t i = 0; i < 16; i++) o[16 * m + i] = d * (float)oxb_tq2_decode_field((w >> (2 * i)) & 3u, i);
        }
    }
}

// ---------------------------------------------------------------------------
// Host-side launchers.
// ---------------------------------------------------------------------------
size_t oxb_xq_bytes(uint32_t k, uint32_t batch) {
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, NC = OXB_XQ_DIGITS * batch;
    return (size_t)nblk_pad * 8 * NC * 16;
}
size_t oxb_cneg_bytes(uint32_t k, uint32_t batch) {
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, NC = OXB_XQ_DIGITS * batch;
    return (size_t)nblk_pad * NC * 16;
}

hipError_t oxb_launch_quant_x(int fmt, const float* d_x, uint32_t k, uint32_t batch, uint32_t* d_xq, int32_t* d_cneg,
                              int32_t* d_xexp, hipStream_t st) {
    const uint32_t n_sb = (k + 511u) / 512u, NC = OXB_XQ_DIGITS * batch;
    const uint32_t gsb = oxb_xq_gsb(n_sb), n_groups = oxb_xq_groups(n_sb);
    if (n_groups > OXB_XQ_MAX_GROUPS) return hipErrorInvalidValue;
    const dim3 grid(batch, n_groups < 16 ? n_groups : 16);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL(quant_x_kernel<OXB_FMT_Q1>, grid, dim3(OXB_QUANT_THREADS), 0, st, d_x, k, NC, gsb, n_groups, d_xq, d_cneg,
                           d_xexp);
    else
        hipLaunchKernelGGL(quant_x_kernel<OXB_FMT_TQ2>, grid, dim3(OXB_QUANT_THREADS), 0, st, d_x, k, NC, gsb, n_groups, d_xq, d_cneg,
                           d_xexp);
    return hipGetLastError();
}

template <int FMT, int NSBW, int TG>
static hipError_t launch_gemv_t(OxbGemvParams p, uint32_t S, uint32_t grid, hipStream_t st) {
    const size_t shm = 2 * (size_t)TG * S * p.NC * 64u;
    hipLaunchKernelGGL((gemv_mfma_kernel<FMT, NSBW, TG>), dim3(grid), dim3(S * 64), shm, st, p);
    return hipGetLastError();
}

hipError_t oxb_launch_gemv(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st) {
    // K slice per wave = one exponent group of the quantised input: NSBW superblocks; S <= 8 waves per workgroup.
    const uint32_t nsbw = oxb_xq_gsb(p.n_sb);
    p.n_groups = oxb_xq_groups(p.n_sb);
    if (p.sb_count > 8 * nsbw || p.sb_begin % nsbw) return hipErrorInvalidValue;  // caller splits K into chunks of OXB_GEMV_MAX_SB superblocks
    const uint32_t S = (p.sb_count + nsbw - 1) / nsbw;
    if (p.n_tiles == 0) return hipSuccess;
    if (p.codes_bytes >= 0x7FFFFFFFull || p.xq_bytes >= 0x7FFFFFFFull) return hipErrorInvalidValue;
    // Choose workgroups per CU (j), tiles in flight per wave (TG) and groups of TG tiles per
    // workgroup so that the busiest CU computes the fewest tile slots; prefer more waves, then
    // a deeper ring.  The partial-sum buffers 2 x TG x S x NC x 64 B stay <= 64 KiB.
    const uint32_t units = fmt == OXB_FMT_Q1 ? 1u : 2u;
    const uint32_t occ = nsbw == 1 ? 2u : 1u;  // what the register budget of the variant allows
    uint32_t tg_max = nsbw == 1 ? 4u : (nsbw == 2 ? 4u / units : 1u);
    while (tg_max > 1 && 2u * tg_max * S * p.NC * 64u > 64u * 1024u) tg_max--;
    uint32_t best_cost = 0xFFFFFFFFu, tg = 1, grid = 1;
    for (uint32_t j = occ; j >= 1; j--)
        for (uint32_t t = tg_max; t >= 1; t--) {
            const uint32_t tpw0 = (p.n_tiles + n_cus * j - 1) / (n_cus * j);
            const uint32_t groups = (tpw0 + t - 1) / t, tpw = groups * t;
            const uint32_t g = (p.n_tiles + tpw - 1) / tpw;
            // tile slots of the busiest CU, weighted by how well a ring of t tiles hides the load latency
            // (measured on 14 MB and 87 MB matrices: one tile in flight costs about 30 %, two 8 %, three 3 %)
            static const uint32_t ring_weight[5] = {0, 130, 108, 103, 100};
            const uint32_t cost = ((g + n_cus - 1) / n_cus) * tpw * ring_weight[t];
            if (cost < best_cost || (cost == best_cost && g > grid)) {  // ties: more workgroups in flight
                best_cost = cost;
                tg = t;
                grid = g;
                p.groups = groups;
            }
        }
#define OXB_CASE(F, N, T)                                                \
    if (fmt == F && nsbw == N && tg == T) return launch_gemv_t<F, N, T>(p, S, grid, st);
    OXB_CASE(OXB_FMT_Q1, 1, 1) OXB_CASE(OXB_FMT_Q1, 1, 2) OXB_CASE(OXB_FMT_Q1, 1, 3) OXB_CASE(OXB_FMT_Q1, 1, 4)
    OXB_CASE(OXB_FMT_Q1, 2, 1) OXB_CASE(OXB_FMT_Q1, 2, 2) OXB_CASE(OXB_FMT_Q1, 2, 3) OXB_CASE(OXB_FMT_Q1, 2, 4)
    OXB_CASE(OXB_FMT_Q1, 3, 1)
    OXB_CASE(OXB_FMT_TQ2, 1, 1) OXB_CASE(OXB_FMT_TQ2, 1, 2) OXB_CASE(OXB_FMT_TQ2, 1, 3) OXB_CASE(OXB_FMT_TQ2, 1, 4)
    OXB_CASE(OXB_FMT_TQ2, 2, 1) OXB_CASE(OXB_FMT_TQ2, 2, 2)
    OXB_CASE(OXB_FMT_TQ2, 3, 1)
#undef OXB_CASE
    return hipErrorInvalidValue;
}

hipError_t oxb_launch_dequant(const OxbLayout& L, const uint32_t* d_codes, const uint16_t* d_scales, float* d_out,
                              hipStream_t st) {
    const uint64_t total = (uint64_t)L.n_rows * (L.k / OXB_QK) * 4;
    if (total == 0) return hipSuccess;
    const uint32_t grid = (uint32_t)((total + 255) / 256);
    hipLaunchKernelGGL(dequant_kernel, dim3(grid), dim3(256), 0, st, L, d_codes, d_scales, d_out);
    return hipGetLastError();
}
