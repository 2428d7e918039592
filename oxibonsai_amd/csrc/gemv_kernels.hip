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
// quantised.  The fp32 activation is carried exactly enough: each x is scaled by
// a per-vector power of two to a 30-bit integer and split into four balanced
// int8 digits which occupy four MFMA columns, so one 16x16x64 MFMA multiplies
// 16 rows x 64 weights by all four digits (and up to four batch columns).
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

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

#define OXB_XQ_P 29  // |x * 2^(P-E)| < 2^29, doubled values stay below 2^30

// ---------------------------------------------------------------------------
// Activation quantiser.
//
// Output, for vector n of the batch (NC = 4*batch columns, column c = 4n+digit):
//   xq  [((blk*2+m)*4+g)*NC + c][jj]  one dword = 4 int8 (bb = 0..3), the MFMA
//        B operand of lane (c,g), register jj, of MFMA m of block blk;
//        Q1 : element bb is digit(c%4) of  s_j * 2*r(k),  k = 128blk+32g+8bb+j, j = 4m+jj,
//             r(k) = rint(x[k] * 2^(P-E-j)),  s_j = -1 for j = 7 (0x80 is -128 as int8)
//        TQ2: element bb is digit(c%4) of  r(k) = rint(x[k] * 2^(P-E-2jj)), k = 128blk+32g+16m+4bb+jj
//   cneg[blk][c][0..3]  four copies of -C, C = the part of the block sum that the
//        biased encodings add (Q1: sum_k 2^j digit(r); TQ2: sum_{jj<3} 4^jj digit(r)),
//        used as the MFMA accumulator's start value;
//   xexp[n]  E - P, or INT_MIN when the vector holds a NaN or an infinity.
// ---------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(256) void quant_x_kernel(const float* __restrict__ x, uint32_t k, uint32_t nblk_pad,
                                                       uint32_t NC, uint32_t* __restrict__ xq,
                                                       int32_t* __restrict__ cneg, int32_t* __restrict__ xexp) {
    extern __shared__ int32_t csum[];  // [nblk_pad][4]
    __shared__ float red[256];
    __shared__ int bad_flag;
    const uint32_t n = blockIdx.x, tid = threadIdx.x;
    const float* xn = x + (size_t)n * k;

    if (tid == 0) bad_flag = 0;
    float mx = 0.0f;
    int bad = 0;
    for (uint32_t i = tid; i < k; i += 256) {
        float v = xn[i];
        bad |= !(fabsf(v) <= 3.402823466e38f);
        mx = fmaxf(mx, fabsf(v));
    }
    red[tid] = mx;
    for (uint32_t i = tid; i < nblk_pad * 4; i += 256) csum[i] = 0;
    __syncthreads();
    if (bad) bad_flag = 1;
    for (uint32_t s = 128; s > 0; s >>= 1) {
        if (tid < s) red[tid] = fmaxf(red[tid], red[tid + s]);
        __syncthreads();
    }
    mx = red[0];
    int E = 0;
    if (mx > 0.0f) (void)frexpf(mx, &E);  // mx = f * 2^E, f in [0.5, 1)
    const int base_shift = OXB_XQ_P - E;
    const uint32_t nblk = k / OXB_QK;

    for (uint32_t u = tid; u < nblk_pad * 32; u += 256) {
        const uint32_t blk = u >> 5, m = (u >> 4) & 1u, g = (u >> 2) & 3u, jj = u & 3u;
        uint32_t out[4] = {0, 0, 0, 0};
        if (blk < nblk && mx > 0.0f && !bad_flag) {
            int c0 = 0, c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
            for (uint32_t bb = 0; bb < 4; bb++) {
                int xi, cr, cmul;
                if (FMT == OXB_FMT_Q1) {
                    const uint32_t j = 4 * m + jj;
                    const float v = xn[blk * 128 + 32 * g + 8 * bb + j];
                    const int r = (int)rintf(ldexpf(v, base_shift - (int)j));
                    xi = (j == 7) ? -2 * r : 2 * r;
                    cr = r;
                    cmul = 1 << j;
                } else {
                    const float v = xn[blk * 128 + 32 * g + 16 * m + 4 * bb + jj];
                    xi = (int)rintf(ldexpf(v, base_shift - 2 * (int)jj));
                    cr = xi;
                    cmul = (jj < 3) ? (1 << (2 * jj)) : 0;
                }
                // balanced base-256 digits: byte d of t is the signed digit d
                const uint32_t t = ((uint32_t)xi + 0x00808080u) ^ 0x00808080u;
                out[0] |= ((t >> 0) & 0xFFu) << (8 * bb);
                out[1] |= ((t >> 8) & 0xFFu) << (8 * bb);
                out[2] |= ((t >> 16) & 0xFFu) << (8 * bb);
                out[3] |= ((t >> 24) & 0xFFu) << (8 * bb);
                const uint32_t tc = ((uint32_t)cr + 0x00808080u) ^ 0x00808080u;
                c0 += (int)(int8_t)(tc >> 0) * cmul;
                c1 += (int)(int8_t)(tc >> 8) * cmul;
                c2 += (int)(int8_t)(tc >> 16) * cmul;
                c3 += (int)(int8_t)(tc >> 24) * cmul;
            }
            atomicAdd(&csum[blk * 4 + 0], c0);
            atomicAdd(&csum[blk * 4 + 1], c1);
            atomicAdd(&csum[blk * 4 + 2], c2);
            atomicAdd(&csum[blk * 4 + 3], c3);
        }
        const size_t base = ((size_t)((blk * 2 + m) * 4 + g) * NC + 4 * n) * 4 + jj;
        xq[base + 0] = out[0];
        xq[base + 4] = out[1];
        xq[base + 8] = out[2];
        xq[base + 12] = out[3];
    }
    __syncthreads();
    for (uint32_t i = tid; i < nblk_pad * 4; i += 256) {
        const uint32_t blk = i >> 2, dgt = i & 3u;
        const int c = -csum[i];
        int4 v = make_int4(c, c, c, c);
        *reinterpret_cast<int4*>(cneg + ((size_t)blk * NC + 4 * n + dgt) * 4) = v;
    }
    if (tid == 0) xexp[n] = bad_flag ? INT32_MIN : (mx > 0.0f ? E - OXB_XQ_P : 0);
}

// ---------------------------------------------------------------------------
// GEMV.  One workgroup = S waves; wave s owns superblocks
// [sb_begin + s*NSBW, +NSBW) of every row tile the workgroup processes and keeps
// the matching slice of the digit planes in registers for the whole kernel, so
// the inner loop is: one coalesced 1 KiB code load per superblock, 4 ANDs + 1
// MFMA per 64 weights of 16 rows, 4 cvt + 4 fma per block for the scale.
// Partial row sums of the S waves meet in LDS; the last step recombines the
// four digit columns and applies the epilogue (store / += / SwiGLU).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}

template <int FMT, int NSBW, int SMAX>
__global__ __launch_bounds__(SMAX * 64) void gemv_mfma_kernel(const OxbGemvParams p) {
    extern __shared__ float part[];  // [slot][S][NC][16]
    const uint32_t lane = threadIdx.x & 63u, s = threadIdx.x >> 6, S = blockDim.x >> 6;
    const uint32_t c = lane & 15u, g = lane >> 4;  // B operand: column c, k-group g; D: column c, rows 4g..4g+3
    const uint32_t NC = p.NC;
    const bool col_on = c < NC;

    const int sb0 = (int)(p.sb_begin + s * NSBW);
    int nsb_w = (int)(p.sb_begin + p.sb_count) - sb0;
    nsb_w = nsb_w < 0 ? 0 : (nsb_w > NSBW ? NSBW : nsb_w);

    // Digit planes and accumulator start values of this wave's K slice.
    v4i B[NSBW][4][2];
    v4i C4[NSBW][4];
#pragma unroll
    for (int i = 0; i < NSBW; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            B[i][q][0] = B[i][q][1] = C4[i][q] = (v4i){0, 0, 0, 0};
            if (i < nsb_w && col_on) {
                const uint32_t blk = (uint32_t)(sb0 + i) * 4 + q;
                const v4i* xq4 = reinterpret_cast<const v4i*>(p.xq);
                B[i][q][0] = xq4[(size_t)((blk * 2 + 0) * 4 + g) * NC + c];
                B[i][q][1] = xq4[(size_t)((blk * 2 + 1) * 4 + g) * NC + c];
                C4[i][q] = reinterpret_cast<const v4i*>(p.cneg)[(size_t)blk * NC + c];
            }
        }

    // Contiguous range of row tiles for this workgroup.
    const uint32_t G = gridDim.x, wg = blockIdx.x;
    const uint32_t base_cnt = p.n_tiles / G, rem = p.n_tiles % G;
    const uint32_t t_begin = wg * base_cnt + (wg < rem ? wg : rem);
    const uint32_t t_count = base_cnt + (wg < rem ? 1u : 0u);
    const uint32_t max_count = base_cnt + (rem ? 1u : 0u);  // uniform barrier count across the grid is not needed,
                                                            // but it must be uniform inside the workgroup: it is.
    (void)max_count;

    const v4i* codes = reinterpret_cast<const v4i*>(p.codes);
    const v4i* scales = reinterpret_cast<const v4i*>(p.scales);
    constexpr int UNITS = (FMT == OXB_FMT_Q1) ? 1 : 2;  // 1 KiB code units per superblock

    for (uint32_t chunk0 = 0; chunk0 < t_count; chunk0 += p.slots) {
        const uint32_t chunk_n = (t_count - chunk0) < p.slots ? (t_count - chunk0) : p.slots;
        for (uint32_t sl = 0; sl < chunk_n; sl++) {
            const uint32_t tile = t_begin + chunk0 + sl;
            v4f accf = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NSBW; i++) {
                if (i < nsb_w) {
                    const size_t unit = (size_t)tile * p.n_sb + (uint32_t)(sb0 + i);
                    v4i w[UNITS];
#pragma unroll
                    for (int u = 0; u < UNITS; u++) w[u] = codes[(unit * UNITS + u) * 64 + lane];
                    const v4i sc0 = scales[(unit * 4 + g) * 2 + 0];  // f16 [q=0,1][v]
                    const v4i sc1 = scales[(unit * 4 + g) * 2 + 1];  // f16 [q=2,3][v]
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        v4i a0, a1;
                        if (FMT == OXB_FMT_Q1) {
                            const uint32_t wq = (uint32_t)w[0][q];
                            a0 = (v4i){(int)(wq & 0x01010101u), (int)(wq & 0x02020202u), (int)(wq & 0x04040404u),
                                       (int)(wq & 0x08080808u)};
                            a1 = (v4i){(int)(wq & 0x10101010u), (int)(wq & 0x20202020u), (int)(wq & 0x40404040u),
                                       (int)(wq & 0x80808080u)};
                        } else {
                            const uint32_t d0 = (uint32_t)w[q >> 1][(q & 1) * 2 + 0];
                            const uint32_t d1 = (uint32_t)w[q >> 1][(q & 1) * 2 + 1];
                            a0 = (v4i){(int)(d0 & 0x03030303u), (int)(d0 & 0x0C0C0C0Cu), (int)(d0 & 0x30303030u),
                                       (int)(d0 & 0xC0C0C0C0u)};
                            a1 = (v4i){(int)(d1 & 0x03030303u), (int)(d1 & 0x0C0C0C0Cu), (int)(d1 & 0x30303030u),
                                       (int)(d1 & 0xC0C0C0C0u)};
                        }
                        v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, B[i][q][0], C4[i][q], 0, 0, 0);
                        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, B[i][q][1], acc, 0, 0, 0);
                        const v4i sc = (q < 2) ? sc0 : sc1;
                        const uint32_t lo = (uint32_t)sc[(q & 1) * 2 + 0], hi = (uint32_t)sc[(q & 1) * 2 + 1];
                        accf[0] = fmaf((float)acc[0], f16_bits_to_f32(lo & 0xFFFFu), accf[0]);
                        accf[1] = fmaf((float)acc[1], f16_bits_to_f32(lo >> 16), accf[1]);
                        accf[2] = fmaf((float)acc[2], f16_bits_to_f32(hi & 0xFFFFu), accf[2]);
                        accf[3] = fmaf((float)acc[3], f16_bits_to_f32(hi >> 16), accf[3]);
                    }
                }
            }
            if (col_on) *reinterpret_cast<v4f*>(&part[(((size_t)sl * S + s) * NC + c) * 16 + g * 4]) = accf;
        }
        __syncthreads();
        // Recombine: thread -> (slot, batch column n, row); fixed summation order over waves.
        const uint32_t batch = NC >> 2;
        for (uint32_t idx = threadIdx.x; idx < chunk_n * batch * 16; idx += blockDim.x) {
            const uint32_t r = idx & 15u, n = (idx >> 4) % batch, sl = idx / (16 * batch);
            const uint32_t row = (t_begin + chunk0 + sl) * 16 + r;
            if (row >= p.n_rows) continue;
            float f[4];
#pragma unroll
            for (int dgt = 0; dgt < 4; dgt++) {
                float a = 0.f;
                for (uint32_t w = 0; w < S; w++) a += part[(((size_t)sl * S + w) * NC + 4 * n + dgt) * 16 + r];
                f[dgt] = a;
            }
            float v = fmaf(fmaf(fmaf(f[3], 256.f, f[2]), 256.f, f[1]), 256.f, f[0]);
            const int e = p.xexp[n];
            v = (e == INT32_MIN) ? __int_as_float(0x7FC00000) : ldexpf(v, e);
            const size_t o = (size_t)n * p.ldy + row;
            if (p.mode == OXB_GEMV_ACCUM) v += p.y[o];
            else if (p.mode == OXB_GEMV_RESIDUAL) v += p.residual[o];
            p.y[o] = v;
        }
        __syncthreads();
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
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, NC = 4 * batch;
    return (size_t)nblk_pad * 8 * NC * 16;
}
size_t oxb_cneg_bytes(uint32_t k, uint32_t batch) {
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, NC = 4 * batch;
    return (size_t)nblk_pad * NC * 16;
}

hipError_t oxb_launch_quant_x(int fmt, const float* d_x, uint32_t k, uint32_t batch, uint32_t* d_xq, int32_t* d_cneg,
                              int32_t* d_xexp, hipStream_t st) {
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, NC = 4 * batch;
    const size_t shm = (size_t)nblk_pad * 4 * sizeof(int32_t);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL(quant_x_kernel<OXB_FMT_Q1>, dim3(batch), dim3(256), shm, st, d_x, k, nblk_pad, NC, d_xq,
                           d_cneg, d_xexp);
    else
        hipLaunchKernelGGL(quant_x_kernel<OXB_FMT_TQ2>, dim3(batch), dim3(256), shm, st, d_x, k, nblk_pad, NC, d_xq,
                           d_cneg, d_xexp);
    return hipGetLastError();
}

template <int FMT, int NSBW, int SMAX>
static hipError_t launch_gemv_t(const OxbGemvParams& p, uint32_t S, uint32_t grid, size_t shm, hipStream_t st) {
    hipLaunchKernelGGL((gemv_mfma_kernel<FMT, NSBW, SMAX>), dim3(grid), dim3(S * 64), shm, st, p);
    return hipGetLastError();
}

hipError_t oxb_launch_gemv(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st) {
    // K slice per wave: NSBW superblocks; S waves per workgroup.
    uint32_t nsbw = (p.sb_count + 7u) / 8u;
    if (nsbw < 1) nsbw = 1;
    if (nsbw > 4) return hipErrorInvalidValue;  // caller splits K into chunks of <= 32 superblocks
    const uint32_t S = (p.sb_count + nsbw - 1) / nsbw;
    // Aim at 16 waves per CU.
    uint32_t wg_per_cu = 16u / S;
    if (wg_per_cu < 1) wg_per_cu = 1;
    uint32_t grid = n_cus * wg_per_cu;
    if (grid > p.n_tiles) grid = p.n_tiles;
    if (grid == 0) return hipSuccess;
    const uint32_t max_tiles = (p.n_tiles + grid - 1) / grid;
    uint32_t slots = (64u * 1024u) / (S * p.NC * 64u);
    if (slots > max_tiles) slots = max_tiles;
    if (slots < 1) slots = 1;
    p.slots = slots;
    const size_t shm = (size_t)slots * S * p.NC * 64u;
#define OXB_CASE(F, N, SM)                                                 \
    if (fmt == F && nsbw == N) return launch_gemv_t<F, N, SM>(p, S, grid, shm, st);
    OXB_CASE(OXB_FMT_Q1, 1, 8)
    OXB_CASE(OXB_FMT_Q1, 2, 8)
    OXB_CASE(OXB_FMT_Q1, 3, 8)
    OXB_CASE(OXB_FMT_Q1, 4, 8)
    OXB_CASE(OXB_FMT_TQ2, 1, 8)
    OXB_CASE(OXB_FMT_TQ2, 2, 8)
    OXB_CASE(OXB_FMT_TQ2, 3, 8)
    OXB_CASE(OXB_FMT_TQ2, 4, 8)
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
