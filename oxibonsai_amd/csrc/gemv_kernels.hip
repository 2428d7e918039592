// gemv_kernels.hip — Q1_0_g128 / TQ2_0_g128 GEMV for gfx950 (MI355X).
//
// What it computes (reference: crates/oxibonsai-kernels/src/gemv.rs:60-84,
// gemv_ternary.rs:83-102):  y[row] = sum_blocks f16(d) * sum_128 code(w) * x,
// optionally with RMSNorm in front (simd_float_ops.rs:204-215) and a residual add or SwiGLU
// (simd_float_ops.rs:217-236) behind it, as the reference's fused kernels gemv_*_residual and
// fused_gate_up_swiglu_q1 do (gpu_backend/cuda_kernels.rs:130-178, 456-543).
//
// Why int8 MFMA and not per-weight VALU decode.  At 8 TB/s a Q1 stream delivers 64e12 weights/s, but
// the chip retires about 33e12 VALU lane-operations/s, so any scheme that spends one VALU operation
// per weight is compute-bound far below the HBM roofline.  Here a weight costs 1/4 VALU operation: one
// AND with 0x01010101 << j (Q1) or 0x03030303 << 2jj (TQ2) turns a code dword into four int8 MFMA
// operands worth 2^j (4^jj) each, and the activation that meets them was divided by the same power of
// two when it was quantised.
//
// One kernel does everything.  The weights are the MFMA's B operand (16 weight rows = 16 columns), the
// activations its A operand: every activation is scaled by a power of two - one per K slice of a wave,
// 512 to 1536 values - to a 30-bit integer and cut into four balanced base-256 digits, which occupy four
// of the sixteen A rows, so up to four activation vectors share one pass over the weights.  A lane then
// holds the four digit sums of one (vector, weight row) pair: they are joined by two shift-adds, two
// conversions and one FMA, the fp16 block scale is applied by one mixed-precision FMA, the slice's power
// of two comes back with one ldexp per tile.  Block sums are exact integers; the rounding of the
// activations to 2^-26 .. 2^-30 of their slice's largest element is below what the fp32 sums of the
// reference lose (Q1 masks the high nibble of a code byte after a shift by 4, so that no operand byte
// is worth more than 8 and no activation gives up more than three bits to it).
// The quantisation happens in the kernel's prologue: the waves of a workgroup split K, and each wave
// quantises exactly the K slice it owns (the activations are requested before the weight stream, so
// they arrive while the first weight tiles are still on their way) - no quantiser kernel, no digit
// planes in memory.  Every workgroup repeats that work; it hides behind the first HBM round trip.
//
// Kernels:
//   gemv_kernel          codes/scales (tiled SoA, see layout.h) x fp32 activations -> y for two to four vectors
//                        (int8 matrix cores, described above)
//   gemv_f4_kernel       the same for one vector on the fp4 matrix-core instruction (described there)
//   stream_floor_kernel  the same loads and nothing else (measurement aid)
//   dequant_kernel       resident layout -> fp32 weights (bit-exactness check)
//   repack_kernel        the reference's block bytes (array of structs) -> resident layout, at upload
//   swiglu_kernel        silu(gate) * up on fp32 vectors (rows too long for one GEMV launch)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "gemv_kernels.h"
#include "gemv_pack_device.h"
#include "layout.h"

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
}

// Codes and scales of one row tile, restricted to this wave's K slice, as they wait in registers.
template <int FMT, int NSBW>
struct TileRegs {
    static constexpr int UNITS = (FMT == OXB_FMT_Q1) ? 1 : 2;  // 1 KiB code units per superblock
    v4i w[NSBW][UNITS];
    v2u sc[NSBW];  // the four f16 scales (blocks 0..3 of the superblock) of this lane's weight row
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
        t.sc[i] = __builtin_amdgcn_raw_buffer_load_b64(scales, (int)(ok ? lane_s : OXB_OOB), (int)(unit * 128u), 0);
    }
}

#define OXB_GEMV_META 4  // ints of per-block metadata a wave leaves in LDS: the four accumulator start values

// Dynamic LDS of a launch: [S][NSBW * 512] staging dwords | [S][NSBW * 4][META] | part [4][TG][S][64] floats | red [4][8] | flags [4]
__host__ __device__ inline size_t oxb_gemv_lds_bytes(uint32_t S, uint32_t nsbw, uint32_t tg) {
    return ((size_t)S * nsbw * 512 + (size_t)S * nsbw * 4 * OXB_GEMV_META + (size_t)4 * tg * S * 64 + 32 + 4) * 4;
}

// Workgroup wg handles tile slots [wg * tpw, +tpw) in groups of TG (TG tiles are in flight per wave).  For the SwiGLU
// epilogue the groups alternate between TG gate tiles and the TG up tiles of the same rows.  All control flow is
// uniform and branch-free inside a group, so the compiler waits for exactly the tile it is about to use.
template <int FMT, int NSBW, int TG, int PRO>
__global__ __launch_bounds__(512) void gemv_kernel(const OxbGemvParams p) {
    extern __shared__ uint32_t smem[];
    const uint32_t lane = threadIdx.x & 63u, s = threadIdx.x >> 6, S = blockDim.x >> 6;
    const uint32_t c = lane & 15u, g = lane >> 4;  // D: weight row c of the tile, activation vector g
    const uint32_t nvec = p.nvec;
    const bool swiglu = p.epi == OXB_GEMV_SWIGLU;
    uint32_t* stage = smem + (size_t)s * NSBW * 512;
    int* meta = (int*)(smem + (size_t)S * NSBW * 512) + (size_t)s * NSBW * 4 * OXB_GEMV_META;
    float* part = (float*)(smem + (size_t)S * NSBW * 512 + (size_t)S * NSBW * 4 * OXB_GEMV_META);
    float* red = part + (size_t)4 * TG * S * 64;
    int* flags = (int*)(red + 32);

    const uint32_t lane_c = lane * 16u, lane_s = c * 8u;
    const uint32_t sb0 = __builtin_amdgcn_readfirstlane(p.sb_begin + s * NSBW);
    const int sb_lim = (int)(p.sb_begin + p.sb_count) - (int)sb0;  // superblocks of this wave's slice that exist
    const __amdgpu_buffer_rsrc_t r_codes = make_rsrc(p.codes, p.codes_bytes);
    const __amdgpu_buffer_rsrc_t r_scales = make_rsrc(p.scales, p.scales_bytes);

    // slot (group, t) -> row tile
    const uint32_t half_tiles = p.n_tiles >> 1;
    const uint32_t n_units = swiglu ? half_tiles : p.n_tiles;                // gate tiles, or all tiles
    const uint32_t upw = swiglu ? (p.tpw >> 1) : p.tpw, u_begin = blockIdx.x * upw;
    const uint32_t groups = p.tpw / TG;
    auto unit_of = [&](uint32_t grp, uint32_t t) -> uint32_t { return u_begin + (swiglu ? (grp >> 1) : grp) * TG + t; };
    auto tile_of = [&](uint32_t grp, uint32_t t) -> uint32_t { return unit_of(grp, t) + ((swiglu && (grp & 1u)) ? half_tiles : 0u); };
    auto slot_ok = [&](uint32_t grp, uint32_t t) -> bool { return grp < groups && unit_of(grp, t) < n_units && unit_of(grp, t) < u_begin + upw; };

    // ---- prologue: this wave's K slice of every vector -> MFMA A operands ----
    // Loads complete in issue order, so the activations of the first vector are requested before the weight stream.
    constexpr uint32_t KS = FMT == OXB_FMT_Q1 ? 8 : 4;
    // lane -> (block of the superblock half, 32-weight group, bit position / field) of its four activations per pass:
    // Q1 k = 128 blk + 32 gg + 8 bb + j;  TQ2 k = 128 blk + 32 gg + 16 (j >> 2) + 4 bb + (j & 3),  bb = 0..3
    const uint32_t j = lane & 7u, gg = (lane >> 3) & 3u, blh = lane >> 5;
    const uint32_t koff = (FMT == OXB_FMT_Q1 ? 32 * gg + j : 32 * gg + 16 * (j >> 2) + (j & 3u)) * 4u;
    const int js = Fix<FMT>::shift_of(j);
    const __amdgpu_buffer_rsrc_t r_w = make_rsrc(p.norm_w, PRO == OXB_GEMV_PRO_RMSNORM ? p.k * 4u : 0u);
    float xe[NSBW][2][4], we[NSBW][2][4];
    // Only requests: nothing here waits for the values, so the weight stream can be requested right behind them.
    auto load_x = [&](uint32_t v) {
        const __amdgpu_buffer_rsrc_t r_x = make_rsrc(p.x + (size_t)v * p.ldx, p.k * 4u);
#pragma unroll
        for (int i = 0; i < NSBW; i++)
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const uint32_t blk = (sb0 + i) * 4 + pass * 2 + blh;
                const uint32_t off = i < sb_lim ? blk * 512u + koff : OXB_OOB;  // beyond k the buffer returns 0
#pragma unroll
                for (int bb = 0; bb < 4; bb++) {
                    xe[i][pass][bb] = __uint_as_float(buf_load_b32(r_x, off + KS * 4u * bb));
                    if (PRO == OXB_GEMV_PRO_RMSNORM) we[i][pass][bb] = __uint_as_float(buf_load_b32(r_w, off + KS * 4u * bb));
                }
            }
    };
    load_x(0);
    if (threadIdx.x < 4) flags[threadIdx.x] = 0;  // cleared for every wave once the barrier is passed
    // every wave's activation requests enter the CU's memory pipeline before any wave's weight requests
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
    TileRegs<FMT, NSBW> ring[TG];
#pragma unroll
    for (int t = 0; t < TG; t++) {
        load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(0, t), slot_ok(0, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
        __builtin_amdgcn_sched_barrier(0);
    }

    v4i A[NSBW][4][2];  // [superblock][block][MFMA]: digit d of vector v in lanes with c = 4 v + d
    v4i C4[NSBW][4];    // accumulator start values (they cancel the bias of the unsigned code encodings), lanes with g = v
    int EX = 0;         // E - P of this wave's K slice of vector g
#pragma unroll
    for (int i = 0; i < NSBW; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            A[i][q][0] = (v4i){0, 0, 0, 0};
            A[i][q][1] = (v4i){0, 0, 0, 0};
            C4[i][q] = (v4i){0, 0, 0, 0};
        }
    auto quantise_vector = [&](const uint32_t v) {
        uint32_t bad = 0;
        if (PRO == OXB_GEMV_PRO_RMSNORM) {
            // Sum of squares over the whole vector: every wave adds its own slice (in registers already); what the
            // waves of this launch do not cover between them is added by a strided loop.  The sums meet in LDS and
            // 1 / rms - a positive scalar, which does not change the slices' powers of two - is applied to the row
            // sums at the end, so the prologue neither waits for the other waves nor for a square root.
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < NSBW; i++)
#pragma unroll
                for (int pass = 0; pass < 2; pass++)
#pragma unroll
                    for (int bb = 0; bb < 4; bb++) {
                        ss = fmaf(xe[i][pass][bb], xe[i][pass][bb], ss);
                        xe[i][pass][bb] *= we[i][pass][bb];
                    }
            const uint32_t c0 = p.sb_begin * 512u, c1 = (p.sb_begin + S * NSBW) * 512u;
            if (c0 > 0 || c1 < p.k) {
                const float* xv = p.x + (size_t)v * p.ldx;
                for (uint32_t i = threadIdx.x; i < p.k; i += blockDim.x)
                    if (i < c0 || i >= c1) ss = fmaf(xv[i], xv[i], ss);
            }
            ss = wave_sum_f32(ss);
            if (lane == 0) red[v * 8 + s] = ss;
        }
        // exponent of the slice: |x| as integers are ordered like the floats, NaN and infinity on top
        uint32_t mxb = 0;
#pragma unroll
        for (int i = 0; i < NSBW; i++)
#pragma unroll
            for (int pass = 0; pass < 2; pass++)
#pragma unroll
                for (int bb = 0; bb < 4; bb++) {
                    mxb = max(mxb, __float_as_uint(xe[i][pass][bb]) & 0x7FFFFFFFu);
                }
        mxb = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_umax(mxb));
        bad |= mxb >= 0x7F800000u;
        const uint32_t be = mxb >> 23;
        const int E = (int)(be ? be : 1u) - 126;  // 2^E > max |x| (subnormal maxima share the smallest E)
        const int sh = Fix<FMT>::P - E - js;
#pragma unroll
        for (int i = 0; i < NSBW; i++) {
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const uint32_t bl = pass * 2 + blh;
                int r[4];
#pragma unroll
                for (int bb = 0; bb < 4; bb++) r[bb] = (int)rintf(ldexpf(xe[i][pass][bb], sh));
                uint32_t tb[4];
                // block sum of 2^js r, in two parts that cannot overflow (|r| <= 2^30)
                int cl = (r[0] & 0x7FFF) + (r[1] & 0x7FFF) + (r[2] & 0x7FFF) + (r[3] & 0x7FFF);
                int ch = (r[0] >> 15) + (r[1] >> 15) + (r[2] >> 15) + (r[3] >> 15);
                if (FMT == OXB_FMT_Q1) {
#pragma unroll
                    for (int bb = 0; bb < 4; bb++) tb[bb] = (((uint32_t)r[bb] << 1) + 0x00808080u) ^ 0x00808080u;
                } else {
#pragma unroll
                    for (int bb = 0; bb < 4; bb++) tb[bb] = ((uint32_t)r[bb] + 0x00808080u) ^ 0x00808080u;
                    if ((j & 3u) == 3u) cl = 0, ch = 0;  // field 3 is two's complement: no bias
                }
                cl = half_isum(cl << js), ch = half_isum(ch << js);
                uint32_t D[4];
                transpose_bytes4(tb, D);
                const uint32_t m = j >> 2, jj = j & 3u;
#pragma unroll
                for (int d = 0; d < 4; d++) stage[((((i * 4 + bl) * 2 + m) * 16 + gg * 4 + d) << 2) + jj] = D[d];
                if ((lane & 31u) == 0) {
                    const long long nc = -(((long long)ch << 15) + cl);  // as three balanced digits and a remainder
                    const unsigned long long t = ((unsigned long long)nc + 0x808080ull) ^ 0x808080ull;
                    *reinterpret_cast<v4i*>(meta + (i * 4 + bl) * OXB_GEMV_META) =
                        (v4i){(int)(signed char)(t & 0xFF), (int)(signed char)((t >> 8) & 0xFF), (int)(signed char)((t >> 16) & 0xFF),
                              (int)((long long)t >> 24)};
                }
            }
        }
        if (__builtin_amdgcn_ballot_w64(bad != 0) != 0 && lane == 0) atomicOr(&flags[v], 1);
        // the staging area is this wave's own: LDS operations of a wave execute in order
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if ((c >> 2) == v) {
#pragma unroll
            for (int i = 0; i < NSBW; i++)
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int m = 0; m < 2; m++)
                        A[i][q][m] = *reinterpret_cast<const v4i*>(&stage[(((i * 4 + q) * 2 + m) * 16 + g * 4 + (c & 3u)) << 2]);
        }
        if (g == v) {
#pragma unroll
            for (int i = 0; i < NSBW; i++)
#pragma unroll
                for (int q = 0; q < 4; q++) C4[i][q] = *reinterpret_cast<const v4i*>(meta + (i * 4 + q) * OXB_GEMV_META);
            EX = mxb ? E - Fix<FMT>::P : 0;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
    };
    quantise_vector(0);  // on the activations requested ahead of the weight stream
    for (uint32_t v = 1; v < nvec; v++) {
        load_x(v);
        quantise_vector(v);
    }

    // ---- main loop ----
    for (uint32_t grp = 0; grp < groups; grp++) {
        float* buf = part + (size_t)(grp & 3u) * TG * S * 64;
#pragma unroll
        for (int t = 0; t < TG; t++) {
            float accf = 0.f;
            const TileRegs<FMT, NSBW>& r = ring[t];
#pragma unroll
            for (int i = 0; i < NSBW; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    v4i b0, b1;
                    if (FMT == OXB_FMT_Q1) {  // 32 sign bits: low nibbles of the four bytes, then the high nibbles
                        const uint32_t d0 = (uint32_t)r.w[i][0][q], d1 = d0 >> 4;
                        b0 = (v4i){(int)(d0 & 0x01010101u), (int)(d0 & 0x02020202u), (int)(d0 & 0x04040404u), (int)(d0 & 0x08080808u)};
                        b1 = (v4i){(int)(d1 & 0x01010101u), (int)(d1 & 0x02020202u), (int)(d1 & 0x04040404u), (int)(d1 & 0x08080808u)};
                    } else {  // 16 two-bit fields each
                        const uint32_t d0 = (uint32_t)r.w[i][q >> 1][(q & 1) * 2], d1 = (uint32_t)r.w[i][q >> 1][(q & 1) * 2 + 1];
                        b0 = (v4i){(int)(d0 & 0x03030303u), (int)(d0 & 0x0C0C0C0Cu), (int)(d0 & 0x30303030u), (int)(d0 & 0xC0C0C0C0u)};
                        b1 = (v4i){(int)(d1 & 0x03030303u), (int)(d1 & 0x0C0C0C0Cu), (int)(d1 & 0x30303030u), (int)(d1 & 0xC0C0C0C0u)};
                    }
                    v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[i][q][0], b0, C4[i][q], 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[i][q][1], b1, acc, 0, 0, 0);
                    // four digit sums of (vector g, weight row c): sum_d 256^d acc[d], then the block scale
                    const int lo = acc[0] + (acc[1] << 8), hi = acc[2] + (acc[3] << 8);
                    const float val = fmaf((float)hi, 65536.0f, (float)lo);
                    const uint32_t scw = (q < 2) ? r.sc[i].x : r.sc[i].y;
                    accf = fmaf(val, f16_bits_to_f32((q & 1) ? scw >> 16 : scw & 0xFFFFu), accf);
                }
            }
            // refill this ring slot with the same slot of the next group (reads nothing past the workgroup's range)
            load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(grp + 1, t), slot_ok(grp + 1, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
            __builtin_amdgcn_sched_barrier(0);
            buf[((size_t)t * S + s) * 64 + lane] = ldexpf(accf, EX);  // the slice's 2^(E - P)
        }
        lds_barrier();
        if (swiglu && !(grp & 1u)) continue;  // the gate sums wait for the up sums of the same rows
        // thread -> (slot, vector, row): add the S partial sums in wave order, then the epilogue.  No second barrier:
        // the next groups write other quarters of `part`, and a quarter is reused only after two more barriers.
        const float* gbuf = part + (size_t)((grp - 1) & 3u) * TG * S * 64;
        for (uint32_t idx = threadIdx.x; idx < (uint32_t)TG * 64; idx += blockDim.x) {
            const uint32_t t = idx >> 6, ln = idx & 63u, cc = ln & 15u, vv = ln >> 4;
            if (vv >= nvec || !slot_ok(grp, t)) continue;
            float v0 = 0.f, v1 = 0.f;
            for (uint32_t w = 0; w < S; w++) v0 += buf[((size_t)t * S + w) * 64 + ln];
            if (swiglu)
                for (uint32_t w = 0; w < S; w++) v1 += gbuf[((size_t)t * S + w) * 64 + ln];
            if (PRO == OXB_GEMV_PRO_RMSNORM) {
                float tot = 0.f;
                for (uint32_t w = 0; w < S; w++) tot += red[vv * 8 + w];
                const float inv_rms = 1.0f / sqrtf(tot / (float)p.k + p.eps);
                if (!(fabsf(inv_rms) <= 3.402823466e38f)) v0 = __int_as_float(0x7FC00000);
                v0 *= inv_rms;
                v1 *= inv_rms;
            }
            if (flags[vv]) v0 = __int_as_float(0x7FC00000);
            const uint32_t row = unit_of(grp, t) * 16 + cc;
            if (row >= (swiglu ? (p.n_rows >> 1) : p.n_rows)) continue;
            const size_t o = (size_t)vv * p.ldy + row;
            if (swiglu) v0 = (v1 / (1.0f + expf(-v1))) * v0;  // v1 = gate, v0 = up
            else if (p.epi == OXB_GEMV_ACCUM) v0 += p.y[o];
            else if (p.epi == OXB_GEMV_RESIDUAL) v0 += p.residual[o];
            p.y[o] = v0;
        }
    }
}

// ---------------------------------------------------------------------------
// Five to eight activation vectors (and any count above one, where it is faster): quantised once, multiplied in one
// pass over the weights.
//
// gemv_kernel quantises every vector in every workgroup, which at eight vectors is three quarters of its instructions,
// and its sixteen A rows hold four vectors, so eight take two passes over the weights.  Here gemv_pack_kernel does the
// quantising once per GEMV - one wave per (superblock of K, vector), each superblock with a power of two of its own -
// and leaves, per group of four vectors and superblock, exactly what a wave of the GEMV holds in registers: the A
// operands of the eight MFMAs (lane l's 16 bytes at l * 16), the accumulator start values, the exponents and, for the
// RMSNorm prologue, the sums of squares.  gemv_packed_kernel loads them (L2 hits: 8.3 KB per superblock and group)
// instead of computing them, expands each code dword once and feeds it to the MFMAs of both vector groups.  Where a
// wave's K slice is too long for two groups' operands to stay in registers (more than one superblock per wave), the
// groups take turns on the tiles that wait in the ring, and the operands of one follow those of the other through the
// same registers.
// Packed layout, dwords, for n_sb superblocks and nvg groups, unit = vg * n_sb + sb:
//   A   [unit][q * 2 + m][lane][4]      C4 [unit][q][v][4]      EX [unit][v]      SS [unit][v]      CL [unit][q][v][2]
// (CL = the start values folded as the kernel joins the digit sums, d0 + 256 d1 and d2 + 256 d3: two registers per
// block instead of four, for the kernels whose K slice leaves no room for C4)
// ---------------------------------------------------------------------------
template <int FMT, int PRO>
__global__ __launch_bounds__(64) void gemv_pack_kernel(const float* __restrict__ x, uint32_t ldx, uint32_t nvec, uint32_t k,
                                                       const float* __restrict__ norm_w, uint32_t n_sb, uint32_t nvg,
                                                       uint32_t* __restrict__ out) {
    const uint32_t lane = threadIdx.x, sb = blockIdx.x, vec = blockIdx.y;
    // a vector beyond nvec reads as zeros: its operands are written all the same, so the GEMV needs no special case
    const __amdgpu_buffer_rsrc_t r_x = make_rsrc(x + (size_t)(vec < nvec ? vec : 0) * ldx, vec < nvec ? k * 4u : 0u);
    const __amdgpu_buffer_rsrc_t r_w = make_rsrc(norm_w, PRO == OXB_GEMV_PRO_RMSNORM ? k * 4u : 0u);
    float xe[2][4], we[2][4];
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
#pragma unroll
        for (int bb = 0; bb < 4; bb++) {
            const uint32_t off = (sb * 512u + gemv_pack_elem<FMT>(lane, pass, bb)) * 4u;  // beyond k the buffer returns 0
            xe[pass][bb] = __uint_as_float(buf_load_b32(r_x, off));
            if (PRO == OXB_GEMV_PRO_RMSNORM) we[pass][bb] = __uint_as_float(buf_load_b32(r_w, off));
        }
    }
    float ss = 0.f;
    if (PRO == OXB_GEMV_PRO_RMSNORM) {
#pragma unroll
        for (int pass = 0; pass < 2; pass++)
#pragma unroll
            for (int bb = 0; bb < 4; bb++) {
                ss = fmaf(xe[pass][bb], xe[pass][bb], ss);
                xe[pass][bb] *= we[pass][bb];
            }
        ss = wave_sum_f32(ss);
    }
    gemv_pack_write<FMT>(xe, ss, lane, sb, vec, n_sb, nvg, out);
}

// Dynamic LDS of a launch: part [4][NVG][TG][S][64] floats | flags [8] | inv_rms [8]
__host__ __device__ inline size_t oxb_gemv_packed_lds_bytes(uint32_t S, uint32_t tg, uint32_t nvg) {
    return ((size_t)4 * nvg * tg * S * 64 + 8 + 8) * 4;
}

// One 128-weight block of a waiting tile -> the two int8 B operands.  The code dword passes through an empty asm
// statement so that two expansions of the same dword (one per vector group) stay two: kept alive between the groups
// they would cost eight registers per block.
template <int FMT, int NSBW>
__device__ __forceinline__ void expand_block(const TileRegs<FMT, NSBW>& r, int i, int q, v4i& b0, v4i& b1) {
    if (FMT == OXB_FMT_Q1) {  // 32 sign bits: low nibbles of the four bytes, then the high nibbles
        uint32_t d0 = (uint32_t)r.w[i][0][q];
        asm volatile("" : "+v"(d0));
        const uint32_t d1 = d0 >> 4;
        b0 = (v4i){(int)(d0 & 0x01010101u), (int)(d0 & 0x02020202u), (int)(d0 & 0x04040404u), (int)(d0 & 0x08080808u)};
        b1 = (v4i){(int)(d1 & 0x01010101u), (int)(d1 & 0x02020202u), (int)(d1 & 0x04040404u), (int)(d1 & 0x08080808u)};
    } else {  // 16 two-bit fields each
        uint32_t d0 = (uint32_t)r.w[i][q >> 1][(q & 1) * 2], d1 = (uint32_t)r.w[i][q >> 1][(q & 1) * 2 + 1];
        asm volatile("" : "+v"(d0), "+v"(d1));
        b0 = (v4i){(int)(d0 & 0x03030303u), (int)(d0 & 0x0C0C0C0Cu), (int)(d0 & 0x30303030u), (int)(d0 & 0xC0C0C0C0u)};
        b1 = (v4i){(int)(d1 & 0x03030303u), (int)(d1 & 0x0C0C0C0Cu), (int)(d1 & 0x30303030u), (int)(d1 & 0xC0C0C0C0u)};
    }
}
template <int FMT, int NSBW>
__device__ __forceinline__ float block_scale(const TileRegs<FMT, NSBW>& r, int i, int q) {
    const uint32_t scw = (q < 2) ? r.sc[i].x : r.sc[i].y;
    return f16_bits_to_f32((q & 1) ? scw >> 16 : scw & 0xFFFFu);
}

// What the packer left for one (vector group, superblock): MFMA A operands, accumulator start values, exponent.
template <bool FOLDED>
struct PackedOps {
    v4i A[4][2];
    v4i C4[FOLDED ? 1 : 4];
    int CL[FOLDED ? 4 : 1][2];
    int EX;
};

// NVG = vector groups of the launch (1 or 2: up to eight vectors).  A wave's operands are NVG * NSBW (group,
// superblock) pairs; NSBW of them are in registers at a time: with a one-superblock slice and two groups both are
// resident and every expanded block feeds both groups' MFMAs; with longer slices the pairs of group 0 are replaced,
// as they are used up, by those of group 1 (and back, for the next tile group), so that the requests run NSBW - 1
// pairs ahead of their use.
// ONE: every workgroup has a single tile group (the launcher knows): no loop around the tile groups, nothing carried
// from one to the next - with long K slices that is what keeps the operands of two vector groups out of scratch memory.
template <int FMT, int NSBW, int TG, int NVG, bool ONE>
__global__ __launch_bounds__(512) void gemv_packed_kernel(const OxbGemvParams p) {
    extern __shared__ uint32_t smem[];
    constexpr bool SIDE = NSBW == 1 && NVG == 2;  // both groups resident, side by side
    constexpr int NOPS = SIDE ? 2 : NSBW, P = NVG * NSBW;
    constexpr bool FOLDED = NSBW >= 3;  // start values as two registers per block, added behind the MFMAs
    typedef PackedOps<FOLDED> Ops;
    const uint32_t lane = threadIdx.x & 63u, s = threadIdx.x >> 6, S = blockDim.x >> 6;
    const uint32_t c = lane & 15u, g = lane >> 4;  // D: weight row c of the tile, activation vector g of the group
    const bool swiglu = p.epi == OXB_GEMV_SWIGLU;
    float* part = (float*)smem;
    int* flags = (int*)(part + (size_t)4 * NVG * TG * S * 64);
    float* inv_rms_v = (float*)(flags + 8);  // 1 / rms of each vector (RMSNorm prologue)

    const uint32_t lane_c = lane * 16u, lane_s = c * 8u;
    const uint32_t sb0 = __builtin_amdgcn_readfirstlane(p.sb_begin + s * NSBW);
    const int sb_lim = (int)(p.sb_begin + p.sb_count) - (int)sb0;  // superblocks of this wave's slice that exist
    const __amdgpu_buffer_rsrc_t r_codes = make_rsrc(p.codes, p.codes_bytes);
    const __amdgpu_buffer_rsrc_t r_scales = make_rsrc(p.scales, p.scales_bytes);
    const __amdgpu_buffer_rsrc_t r_q = make_rsrc(p.xq, p.xq_bytes);

    const uint32_t half_tiles = p.n_tiles >> 1;
    const uint32_t n_units = swiglu ? half_tiles : p.n_tiles;
    const uint32_t upw = swiglu ? (p.tpw >> 1) : p.tpw, u_begin = blockIdx.x * upw;
    const uint32_t groups = ONE ? 1u : p.tpw / TG;
    auto unit_of = [&](uint32_t grp, uint32_t t) -> uint32_t { return u_begin + (swiglu ? (grp >> 1) : grp) * TG + t; };
    auto tile_of = [&](uint32_t grp, uint32_t t) -> uint32_t { return unit_of(grp, t) + ((swiglu && (grp & 1u)) ? half_tiles : 0u); };
    auto slot_ok = [&](uint32_t grp, uint32_t t) -> bool { return grp < groups && unit_of(grp, t) < n_units && unit_of(grp, t) < u_begin + upw; };

    // ---- prologue: requests for the first operands, then (behind a barrier) the weight ring ----
    const uint32_t q_units = NVG * p.n_sb;
    const uint32_t c4_base = q_units * 2048u * 4u, ex_base = q_units * (2048u + 64u) * 4u;
    Ops ops[NOPS];
    const uint32_t cl_base = q_units * (2048u + 64u + 8u) * 4u;
    auto load_ops = [&](Ops& o, int vgi, int i, bool wanted) {  // !wanted: zeros, and no data moves
        const bool ok = wanted && i < sb_lim;
        const uint32_t unit = __builtin_amdgcn_readfirstlane((uint32_t)vgi * p.n_sb + sb0 + (uint32_t)i);
#pragma unroll
        for (int q = 0; q < 4; q++) {
#pragma unroll
            for (int m = 0; m < 2; m++) o.A[q][m] = buf_load_b128(r_q, ok ? lane_c : OXB_OOB, unit * 8192u + (q * 2 + m) * 1024u);
            if (FOLDED) {
                const v2u cl = __builtin_amdgcn_raw_buffer_load_b64(r_q, (int)(ok ? g * 8u : OXB_OOB), (int)(cl_base + unit * 128u + q * 32u), 0);
                o.CL[q][0] = (int)cl.x;
                o.CL[q][1] = (int)cl.y;
            } else {
                o.C4[q] = buf_load_b128(r_q, ok ? g * 16u : OXB_OOB, c4_base + unit * 256u + q * 64u);
            }
        }
        o.EX = (int)buf_load_b32(r_q, ok ? g * 4u : OXB_OOB, ex_base + unit * 16u);
    };
    // pair n = (group n / NSBW, superblock n % NSBW) of the wave's slice lives in ops[n % NOPS]
#pragma unroll
    for (int n = 0; n < NOPS; n++) load_ops(ops[n], n / NSBW, n % NSBW, true);
    if (threadIdx.x < 8) flags[threadIdx.x] = 0;  // cleared for every wave once the barrier is passed
    // RMSNorm: the superblocks' sums of squares in order -> 1 / rms per vector, once per workgroup (the merge below
    // applies it to the row sums; it is first read behind the barrier that ends the first tile group)
    // (thread 4 g + v adds for vector v of group g; eight superblocks per round of requests, the first round issued
    // here with the operands, so that it is back long before the first weight tile)
    const bool norm_thread = p.pro == OXB_GEMV_PRO_RMSNORM && threadIdx.x < NVG * 4;
    const __amdgpu_buffer_rsrc_t r_ss = make_rsrc((const float*)p.xq + (size_t)NVG * p.n_sb * (2048 + 64 + 4), NVG * p.n_sb * 16u);
    auto ss_round = [&](uint32_t sb_first, float (&v)[8]) {
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) {
            const uint32_t sb = sb_first + i;
            v[i] = __uint_as_float(buf_load_b32(r_ss, norm_thread && sb < p.n_sb ? (((threadIdx.x >> 2) * p.n_sb + sb) * 4 + (threadIdx.x & 3u)) * 4u : OXB_OOB));
        }
    };
    float ss_first[8];
    ss_round(0, ss_first);
    // every wave's operand requests enter the CU's memory pipeline before any wave's weight requests
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
    TileRegs<FMT, NSBW> ring[TG];
#pragma unroll
    for (int t = 0; t < TG; t++) {
        load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(0, t), slot_ok(0, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (p.pro == OXB_GEMV_PRO_RMSNORM && s == 0) {  // wave-uniform: only the first wave has such threads
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) tot += ss_first[i];  // entries past the last superblock read as +0
        for (uint32_t sb = 8; sb < p.n_sb; sb += 8) {
            float more[8];
            ss_round(sb, more);
#pragma unroll
            for (int i = 0; i < 8; i++) tot += more[i];
        }
        if (norm_thread) inv_rms_v[threadIdx.x] = 1.0f / sqrtf(tot / (float)p.k + p.eps);
    }
    // a slice with an infinity or a NaN in it: every output of that vector becomes NaN
    auto take_ex = [&](Ops& o, int vgi) -> int {
        if (o.EX == OXB_GEMV_EX_BAD) {
            flags[vgi * 4 + g] = 1;
            return 0;
        }
        return o.EX;
    };

    // ---- main loop ----
    for (uint32_t grp = 0; grp < groups; grp++) {
        float* buf = part + (size_t)(grp & 3u) * NVG * TG * S * 64;
        float accf[NVG][TG];
#pragma unroll
        for (int vgi = 0; vgi < NVG; vgi++)
#pragma unroll
            for (int t = 0; t < TG; t++) accf[vgi][t] = 0.f;
        if (SIDE) {
            const int ex0 = take_ex(ops[0], 0), ex1 = take_ex(ops[NOPS - 1], 1);
#pragma unroll
            for (int t = 0; t < TG; t++) {
                float a0 = 0.f, a1 = 0.f;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    v4i b0, b1;
                    expand_block<FMT, NSBW>(ring[t], 0, q, b0, b1);
                    const float sc = block_scale<FMT, NSBW>(ring[t], 0, q);
                    v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ops[0].A[q][0], b0, ops[0].C4[q], 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ops[0].A[q][1], b1, acc, 0, 0, 0);
                    v4i bcc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ops[NOPS - 1].A[q][0], b0, ops[NOPS - 1].C4[q], 0, 0, 0);
                    bcc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ops[NOPS - 1].A[q][1], b1, bcc, 0, 0, 0);
                    a0 = fmaf(fmaf((float)(acc[2] + (acc[3] << 8)), 65536.0f, (float)(acc[0] + (acc[1] << 8))), sc, a0);
                    a1 = fmaf(fmaf((float)(bcc[2] + (bcc[3] << 8)), 65536.0f, (float)(bcc[0] + (bcc[1] << 8))), sc, a1);
                }
                load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(grp + 1, t), slot_ok(grp + 1, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
                __builtin_amdgcn_sched_barrier(0);
                accf[0][t] = ldexpf(a0, ex0);  // the superblock's 2^(E - P)
                accf[NVG - 1][t] = ldexpf(a1, ex1);
            }
        } else {
#pragma unroll
            for (int n = 0; n < P; n++) {
                const int vgi = n / NSBW, i = n % NSBW;
                Ops& o = ops[n % NOPS];
                const int ex = take_ex(o, vgi);
#pragma unroll
                for (int t = 0; t < TG; t++) {
                    float a0 = 0.f;
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        v4i b0, b1;
                        expand_block<FMT, NSBW>(ring[t], i, q, b0, b1);
                        v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.A[q][0], b0, FOLDED ? (v4i){0, 0, 0, 0} : o.C4[FOLDED ? 0 : q], 0, 0, 0);
                        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(o.A[q][1], b1, acc, 0, 0, 0);
                        int lo = acc[0] + (acc[1] << 8), hi = acc[2] + (acc[3] << 8);
                        if (FOLDED) lo += o.CL[FOLDED ? q : 0][0], hi += o.CL[FOLDED ? q : 0][1];
                        a0 = fmaf(fmaf((float)hi, 65536.0f, (float)lo), block_scale<FMT, NSBW>(ring[t], i, q), a0);
                    }
                    accf[vgi][t] += ldexpf(a0, ex);
                }
                // this pair's registers take the pair NSBW further on (of the next tile group, past the end)
                if (P > NOPS && !(ONE && n + NOPS >= P)) {  // unconditional requests (out of range when nothing follows): no second copy to select from
                    __builtin_amdgcn_sched_barrier(0);  // not above the pair's last use: the requests reuse its registers
                    load_ops(o, ((n + NOPS) % P) / NSBW, i, n + NOPS < P || grp + 1 < groups);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (!ONE) {
#pragma unroll
                for (int t = 0; t < TG; t++) {
                    load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(grp + 1, t), slot_ok(grp + 1, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
#pragma unroll
        for (int vgi = 0; vgi < NVG; vgi++)
#pragma unroll
            for (int t = 0; t < TG; t++) buf[(((size_t)vgi * TG + t) * S + s) * 64 + lane] = accf[vgi][t];
        lds_barrier();
        if (swiglu && !(grp & 1u)) continue;  // the gate sums wait for the up sums of the same rows
        // thread -> (vector group, slot, vector, row): add the S partial sums in wave order, then the epilogue.  No
        // second barrier: the next groups write other quarters of `part`, and a quarter is reused only after two more.
        const float* gbuf = part + (size_t)((grp - 1) & 3u) * NVG * TG * S * 64;
        for (uint32_t idx = threadIdx.x; idx < (uint32_t)NVG * TG * 64; idx += blockDim.x) {
            const uint32_t vgt = idx / ((uint32_t)TG * 64), rem = idx % ((uint32_t)TG * 64);
            const uint32_t t = rem >> 6, ln = rem & 63u, cc = ln & 15u, vv = vgt * 4 + (ln >> 4);
            if (vv >= p.nvec || !slot_ok(grp, t)) continue;
            const size_t o0 = (((size_t)vgt * TG + t) * S) * 64 + ln;
            float v0 = 0.f, v1 = 0.f;
            for (uint32_t w = 0; w < S; w++) v0 += buf[o0 + (size_t)w * 64];
            if (swiglu)
                for (uint32_t w = 0; w < S; w++) v1 += gbuf[o0 + (size_t)w * 64];
            if (p.pro == OXB_GEMV_PRO_RMSNORM) {  // 1 / rms on the row sums
                const float inv_rms = inv_rms_v[vv];
                if (!(fabsf(inv_rms) <= 3.402823466e38f)) v0 = __int_as_float(0x7FC00000);
                v0 *= inv_rms;
                v1 *= inv_rms;
            }
            if (flags[vv]) v0 = __int_as_float(0x7FC00000);
            const uint32_t row = unit_of(grp, t) * 16 + cc;
            if (row >= (swiglu ? (p.n_rows >> 1) : p.n_rows)) continue;
            const size_t o = (size_t)vv * p.ldy + row;
            if (swiglu) v0 = (v1 / (1.0f + expf(-v1))) * v0;  // v1 = gate, v0 = up
            else if (p.epi == OXB_GEMV_ACCUM) v0 += p.y[o];
            else if (p.epi == OXB_GEMV_RESIDUAL) v0 += p.residual[o];
            p.y[o] = v0;
        }
    }
}

// ---------------------------------------------------------------------------
// One activation vector, Q1 weights: the fp4 matrix-core route.
//
// v_mfma_scale_f32_16x16x128_f8f6f4 with both operands in fp4 (E2M1) multiplies a whole 128-weight block of 16 rows
// in one instruction that takes as long as one of the two int8 instructions above, and an fp4 operand is a nibble:
// the code dword of a lane ANDed with 0x11111111 << m is already four operands' worth - bit m of nibble i is weight
// 4 i + m of the lane's 32, and the nibbles 0001 / 0010 / 0100 read 0.5 / 1 / 2 as E2M1 numbers (m = 0, 1, 2), while
// (w & 0x88888888) | 0x22222222 reads -1 / +1 (m = 3).  So a block costs 3 ANDs and one AND-OR instead of 8 ANDs and a
// shift.  The activation meets them as sixteen base-4 digits of a 32-bit magnitude with the sign in every digit: digit j
// of all 128 activations is row j of the A operand, an E2M1 number d / 2 with d in 0..3.  |x| is scaled by a power of
// two - one per K slice of a wave, as above - so that x = 2^(E - 30) X with |X| < 2^30, and the integer that is cut into
// digits is X 2^(1 - s) for a weight whose set bit reads 2^s (the sum of b 2^s times it is twice the sum over the set
// bits; the accumulator starts at minus the sum over all of them, which one extra MFMA per block against constant
// operands computes in the prologue) and X with the opposite sign for m = 3.  Products and their sums over a block are
// small multiples of 1/8: every matrix-core result is exact.  A lane then holds the block sums of digits 4 g .. 4 g + 3
// for weight row c: four FMAs with the block's fp16 scale keep one fp32 accumulator per digit, four more per tile join
// them with the digits' powers of four, and two lane exchanges add the four lane groups before the wave leaves its
// sixteen row sums in LDS, where one wave per tile group (they take turns) adds the waves' sums and stores the rows.
// A block costs 8 vector instructions and one MFMA where the int8 route needs 15 and two.
// ---------------------------------------------------------------------------
typedef int v8i __attribute__((ext_vector_type(8)));
#define OXB_F4_P 30          // |x| < 2^E  ->  |X| < 2^30
#define OXB_F4_CELL 68       // dwords per (block, 32-weight group) cell of the staging area: 16 digits x 4 dwords + 4 of padding
#define OXB_F4_STAGE (16 * OXB_F4_CELL)

// Dynamic LDS of a launch: [S][OXB_F4_STAGE] staging dwords | part [4][TG][S][16] floats | red [16] | flags [4]
__host__ __device__ inline size_t oxb_gemv_f4_lds_bytes(uint32_t S, uint32_t tg) {
    return ((size_t)S * OXB_F4_STAGE + (size_t)4 * tg * S * 16 + 16 + 4) * 4;
}

__device__ __forceinline__ uint32_t bfi_u32(uint32_t mask, uint32_t a, uint32_t b) { return (a & mask) | (b & ~mask); }

__device__ __forceinline__ v4f mfma_f4(const v4i a, const v4i b, const v4f c) {
    const v8i a8 = {a[0], a[1], a[2], a[3], 0, 0, 0, 0}, b8 = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
    // formats 4 = fp4 for both operands; block scales 2^0 (E8M0 127)
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c, 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}
// the same with the B operand's block scale at 2^-1 (E8M0 126)
__device__ __forceinline__ v4f mfma_f4_half_b(const v4i a, const v4i b, const v4f c) {
    const v8i a8 = {a[0], a[1], a[2], a[3], 0, 0, 0, 0}, b8 = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c, 4, 4, 0, 0x7F7F7F7F, 0, 0x7E7E7E7E);
}

// the same with the B operand's block scale at 2^1 (E8M0 128)
__device__ __forceinline__ v4f mfma_f4_double_b(const v4i a, const v4i b, const v4f c) {
    const v8i a8 = {a[0], a[1], a[2], a[3], 0, 0, 0, 0}, b8 = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c, 4, 4, 0, 0x7F7F7F7F, 0, 0x80808080);
}

// TQ2 weights on the same route.  A stored field is value + 1 (0, 1, 2) and reads (value + 1) / 2 as an E2M1 nibble:
// the even fields of a code dword are in place after one AND with 0x33333333, the odd ones after a shift by two - and
// an add of 0x10101010 before the AND, which turns the two's-complement fields at in-byte position 3 into value + 1 like
// the others (the carry runs into bits that the AND drops).  The two dwords of a lane's 32 weights give the four operand
// registers: register j, nibble n is weight 2 n + (j & 1) + 16 (j >> 1) of the group, and the prologue's lane m = j
// quantises exactly those eight activations.  At a block scale of 2 the MFMA sums (value + 1) * digit / 2; the start
// value - the same digits against a constant -1 - takes the digit sums off again.  No shifts by bit position and no
// sign turns: every weight reads the same.  A block costs 8 + 4 vector instructions and one MFMA (the int8 route: 15
// and two).
template <int FMT, int NSBW, int TG, int PRO>
__global__ __launch_bounds__(512) void gemv_f4_kernel(const OxbGemvParams p) {
    extern __shared__ uint32_t smem[];
    const uint32_t lane = threadIdx.x & 63u, s = threadIdx.x >> 6, S = blockDim.x >> 6;
    const uint32_t c = lane & 15u, g = lane >> 4;  // D: weight row c of the tile, digits 4 g .. 4 g + 3
    const bool swiglu = p.epi == OXB_GEMV_SWIGLU;
    uint32_t* stage = smem + (size_t)s * OXB_F4_STAGE;
    float* part = (float*)(smem + (size_t)S * OXB_F4_STAGE);
    float* red = part + (size_t)4 * TG * S * 16;
    int* flags = (int*)(red + 16);

    const uint32_t lane_c = lane * 16u, lane_s = c * 8u;
    const uint32_t sb0 = __builtin_amdgcn_readfirstlane(p.sb_begin + s * NSBW);
    const int sb_lim = (int)(p.sb_begin + p.sb_count) - (int)sb0;
    const __amdgpu_buffer_rsrc_t r_codes = make_rsrc(p.codes, p.codes_bytes);
    const __amdgpu_buffer_rsrc_t r_scales = make_rsrc(p.scales, p.scales_bytes);

    const uint32_t half_tiles = p.n_tiles >> 1;
    const uint32_t n_units = swiglu ? half_tiles : p.n_tiles;
    const uint32_t upw = swiglu ? (p.tpw >> 1) : p.tpw, u_begin = blockIdx.x * upw;
    const uint32_t groups = p.tpw / TG;
    auto unit_of = [&](uint32_t grp, uint32_t t) -> uint32_t { return u_begin + (swiglu ? (grp >> 1) : grp) * TG + t; };
    auto tile_of = [&](uint32_t grp, uint32_t t) -> uint32_t { return unit_of(grp, t) + ((swiglu && (grp & 1u)) ? half_tiles : 0u); };
    auto slot_ok = [&](uint32_t grp, uint32_t t) -> bool { return grp < groups && unit_of(grp, t) < n_units && unit_of(grp, t) < u_begin + upw; };

    // ---- prologue ----
    // lane -> (block q of the superblock, 32-weight group gq, operand register m); its eight activations per superblock
    // are nibble i = 0 .. 7 of that register: Q1 the weights 4 i + m of the group (bit position m), TQ2 the weights
    // 2 i + (m & 1) + 16 (m >> 1).  Both load the Q1 set - the four lanes of a group take 16 consecutive bytes per
    // request - and TQ2 exchanges within the quad afterwards (requests of two 8-byte pieces per quad instead had the
    // activations arrive 0.5 us later: QKV 4096 x 2048 3.78 against 3.22 us).
    const uint32_t pq = lane >> 4, pg = (lane >> 2) & 3u, pm = lane & 3u;
    constexpr uint32_t XS = 16u;  // bytes between the lane's consecutive activations
    const uint32_t koff = (128u * pq + 32u * pg + pm) * 4u;
    const __amdgpu_buffer_rsrc_t r_x = make_rsrc(p.x, p.k * 4u);
    const __amdgpu_buffer_rsrc_t r_w = make_rsrc(p.norm_w, PRO == OXB_GEMV_PRO_RMSNORM ? p.k * 4u : 0u);
    float xe[NSBW][8], we[NSBW][8];
#pragma unroll
    for (int i = 0; i < NSBW; i++) {
        const uint32_t off = i < sb_lim ? (sb0 + i) * 2048u + koff : OXB_OOB;  // beyond k the buffer returns 0
#pragma unroll
        for (int e = 0; e < 8; e++) {
            xe[i][e] = __uint_as_float(buf_load_b32(r_x, off + XS * e));
            if (PRO == OXB_GEMV_PRO_RMSNORM) we[i][e] = __uint_as_float(buf_load_b32(r_w, off + XS * e));
        }
    }
    // Every wave's activation requests enter the CU's memory pipeline before any wave's weight requests: without
    // the barrier the activations of the waves that start last wait behind the weight tiles of the first ones, and
    // their whole prologue with them (gate||up 24576 x 4096: 6.5 -> 5.7 us).
    if (threadIdx.x == 0) flags[0] = 0;  // cleared for every wave once the barrier is passed
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
    TileRegs<FMT, NSBW> ring[TG];
#pragma unroll
    for (int t = 0; t < TG; t++) {
        load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(0, t), slot_ok(0, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
        __builtin_amdgcn_sched_barrier(0);
    }

    // RMSNorm: the weights are multiplied in here; the scalar 1 / rms is positive and the same for the whole vector, so
    // it does not change which power of two the slices get and is applied to the row sums at the end (the waves
    // leave their sums of squares in LDS and go on: no barrier, no wait for the other slices in the prologue).
    uint32_t bad = 0;
    if (PRO == OXB_GEMV_PRO_RMSNORM) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NSBW; i++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                ss = fmaf(xe[i][e], xe[i][e], ss);
                xe[i][e] *= we[i][e];
            }
        const uint32_t c0 = p.sb_begin * 512u, c1 = (p.sb_begin + S * NSBW) * 512u;
        if (c0 > 0 || c1 < p.k) {  // what the waves of this launch do not cover between them
            for (uint32_t i = threadIdx.x; i < p.k; i += blockDim.x)
                if (i < c0 || i >= c1) ss = fmaf(p.x[i], p.x[i], ss);
        }
        ss = wave_sum_f32(ss);
        if (lane == 0) red[s] = ss;
    }
    uint32_t mxb = 0;
#pragma unroll
    for (int i = 0; i < NSBW; i++)
#pragma unroll
        for (int e = 0; e < 8; e++) mxb = max(mxb, __float_as_uint(xe[i][e]) & 0x7FFFFFFFu);
    mxb = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_umax(mxb));
    bad |= mxb >= 0x7F800000u;
    if (__builtin_amdgcn_ballot_w64(bad != 0) != 0 && lane == 0) atomicOr(&flags[0], 1);
    const uint32_t be = mxb >> 23;
    const int E = (int)(be ? be : 1u) - 126;  // 2^E > max |x|
    const int sh = OXB_F4_P - E + (FMT == OXB_FMT_Q1 ? (pm == 0 ? 2 : (pm == 1 ? 1 : 0)) : 0);
    const uint32_t flip = (FMT == OXB_FMT_Q1 && pm == 3) ? 0x88888888u : 0u;  // Q1, m = 3: the operand reads -1 for a set bit, all eight signs turn

    if (FMT == OXB_FMT_TQ2) {
        // lane m holds the activations 4 e + m (what precedes does not depend on which lane holds which); it needs
        // 2 n + (m & 1) + 16 (m >> 1) = element (n >> 1) + 4 (m >> 1) of lane 2 (n & 1) + (m & 1) of its quad
#pragma unroll
        for (int i = 0; i < NSBW; i++) {
            float t[8];
#pragma unroll
            for (int n = 0; n < 8; n++) {
                const float lo = (n & 1) ? dpp_f32<0xEE>(xe[i][n >> 1]) : dpp_f32<0x44>(xe[i][n >> 1]);          // quad_perm [2,3,2,3] / [0,1,0,1]
                const float hi = (n & 1) ? dpp_f32<0xEE>(xe[i][4 + (n >> 1)]) : dpp_f32<0x44>(xe[i][4 + (n >> 1)]);
                t[n] = (pm >> 1) ? hi : lo;
            }
#pragma unroll
            for (int n = 0; n < 8; n++) xe[i][n] = t[n];
        }
    }
    v4i A[NSBW][4];   // [superblock][block]: digit c of the block's activations, group g
    v4f C4[NSBW][4];  // accumulator start values of digits 4 g .. 4 g + 3
#pragma unroll
    for (int i = 0; i < NSBW; i++) {
        uint32_t r[8], sg = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            r[e] = (uint32_t)rintf(ldexpf(fabsf(xe[i][e]), sh));
            sg |= (uint32_t)(__float_as_int(xe[i][e]) >> 31) & (8u << (4 * e));  // the sign into bit 3 of nibble e
        }
        sg ^= flip;
        // 8 x 8 nibble transpose: tr[n] nibble e = r[e] nibble n = digits 2 n and 2 n + 1 of activation e
        uint32_t lo[4], hi[4], tl[4], th[4];
#pragma unroll
        for (int a = 0; a < 4; a++) {
            lo[a] = bfi_u32(0x0F0F0F0Fu, r[2 * a], r[2 * a + 1] << 4);
            hi[a] = bfi_u32(0x0F0F0F0Fu, r[2 * a] >> 4, r[2 * a + 1]);
        }
        transpose_bytes4(lo, tl);
        transpose_bytes4(hi, th);
        uint32_t* cell = stage + (pq * 4 + pg) * OXB_F4_CELL + pm;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            cell[(4 * b + 0) * 4] = (tl[b] & 0x33333333u) | sg;          // digit 4 b
            cell[(4 * b + 1) * 4] = ((tl[b] >> 2) & 0x33333333u) | sg;   // digit 4 b + 1
            cell[(4 * b + 2) * 4] = (th[b] & 0x33333333u) | sg;          // digit 4 b + 2
            cell[(4 * b + 3) * 4] = ((th[b] >> 2) & 0x33333333u) | sg;   // digit 4 b + 3
        }
        // the staging area is this wave's own: LDS operations of a wave execute in order
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int q = 0; q < 4; q++) A[i][q] = *reinterpret_cast<const v4i*>(&stage[(q * 4 + g) * OXB_F4_CELL + c * 4]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int q = 0; q < 4; q++) {
            // Q1: minus the sum over the block of 2^(s - 1) a for m < 3: operands -0.5, -1, -2 at a block scale of 1/2;
            // TQ2: minus the sum of all digits
            if (FMT == OXB_FMT_Q1)
                C4[i][q] = mfma_f4_half_b(A[i][q], (v4i){(int)0x99999999u, (int)0xAAAAAAAAu, (int)0xCCCCCCCCu, 0}, (v4f){0.f, 0.f, 0.f, 0.f});
            else
                C4[i][q] = mfma_f4(A[i][q], (v4i){(int)0xAAAAAAAAu, (int)0xAAAAAAAAu, (int)0xAAAAAAAAu, (int)0xAAAAAAAAu}, (v4f){0.f, 0.f, 0.f, 0.f});
        }
    }
    // digit j of X is worth 2 * 4^j; the tile sums leave the wave as 2^-32 of that, and 2^(E - 30 + 32) follows
    float MQ[4];
#pragma unroll
    for (int jj = 0; jj < 4; jj++) MQ[jj] = ldexpf(1.0f, 2 * (int)(4 * g + jj) - 31);
    const int EX = mxb ? E - OXB_F4_P + 32 : 0;

    // ---- main loop ----
    for (uint32_t grp = 0; grp < groups; grp++) {
        float* buf = part + (size_t)(grp & 3u) * TG * S * 16;
#pragma unroll
        for (int t = 0; t < TG; t++) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            const TileRegs<FMT, NSBW>& r = ring[t];
#pragma unroll
            for (int i = 0; i < NSBW; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    v4f d;
                    if (FMT == OXB_FMT_Q1) {
                        const uint32_t w = (uint32_t)r.w[i][0][q];
                        const v4i b = {(int)(w & 0x11111111u), (int)(w & 0x22222222u), (int)(w & 0x44444444u),
                                       (int)((w & 0x88888888u) | 0x22222222u)};
                        d = mfma_f4(A[i][q], b, C4[i][q]);
                    } else {
                        const uint32_t lo = (uint32_t)r.w[i][FMT == OXB_FMT_Q1 ? 0 : q >> 1][2 * (q & 1)];
                        const uint32_t hi = (uint32_t)r.w[i][FMT == OXB_FMT_Q1 ? 0 : q >> 1][2 * (q & 1) + 1];
                        const v4i b = {(int)(lo & 0x33333333u), (int)(((lo >> 2) + 0x10101010u) & 0x33333333u),
                                       (int)(hi & 0x33333333u), (int)(((hi >> 2) + 0x10101010u) & 0x33333333u)};
                        d = mfma_f4_double_b(A[i][q], b, C4[i][q]);
                    }
                    const uint32_t scw = (q < 2) ? r.sc[i].x : r.sc[i].y;
                    const float sc = f16_bits_to_f32((q & 1) ? scw >> 16 : scw & 0xFFFFu);
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) acc[jj] = fmaf(d[jj], sc, acc[jj]);
                }
            }
            load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, tile_of(grp + 1, t), slot_ok(grp + 1, t), p.n_sb, sb0, sb_lim, lane_c, lane_s);
            __builtin_amdgcn_sched_barrier(0);
            float v = acc[0] * MQ[0];
            v = fmaf(acc[1], MQ[1], v);
            v = fmaf(acc[2], MQ[2], v);
            v = fmaf(acc[3], MQ[3], v);
            v = ldexpf(sum_rows4(v), EX);
            if (lane < 16) buf[((size_t)t * S + s) * 16 + lane] = v;
        }
        lds_barrier();
        if (swiglu && !(grp & 1u)) continue;  // the gate sums wait for the up sums of the same rows
        // One wave (they take turns) finishes the group: lane -> (tile t of the group, row c), the S sums of the
        // waves requested together and added in wave order, then the epilogue.  No second barrier: the next groups
        // write other quarters of `part`, and a quarter is reused only after two more barriers.
        if (s != (swiglu ? grp >> 1 : grp) % S) continue;
        const float* gbuf = part + (size_t)((grp - 1) & 3u) * TG * S * 16;
        const uint32_t t = lane >> 4;
        if (t >= (uint32_t)TG || !slot_ok(grp, t)) continue;
        float pv[8], pg[8];
#pragma unroll
        for (uint32_t w = 0; w < 8; w++) {
            const uint32_t wc = w < S ? w : S - 1;
            pv[w] = buf[((size_t)t * S + wc) * 16 + c];
            if (swiglu) pg[w] = gbuf[((size_t)t * S + wc) * 16 + c];
        }
        float rp[8];
        if (PRO == OXB_GEMV_PRO_RMSNORM) {
#pragma unroll
            for (uint32_t w = 0; w < 8; w++) rp[w] = red[w < S ? w : 0u];
        }
        int bad_in = flags[0];
        float v0 = 0.f, v1 = 0.f;
#pragma unroll
        for (uint32_t w = 0; w < 8; w++) {
            v0 += w < S ? pv[w] : 0.f;  // a wave that does not exist adds +0
            if (swiglu) v1 += w < S ? pg[w] : 0.f;
        }
        if (PRO == OXB_GEMV_PRO_RMSNORM) {  // the waves' sums of squares in wave order, then 1 / rms on the row sums
            float tot = 0.f;
#pragma unroll
            for (uint32_t w = 0; w < 8; w++) tot += w < S ? rp[w] : 0.f;
            const float inv_rms = 1.0f / sqrtf(tot / (float)p.k + p.eps);
            bad_in |= !(fabsf(inv_rms) <= 3.402823466e38f);
            v0 *= inv_rms;
            v1 *= inv_rms;
        }
        if (bad_in) v0 = __int_as_float(0x7FC00000);
        const uint32_t row = unit_of(grp, t) * 16 + c;
        if (row >= (swiglu ? (p.n_rows >> 1) : p.n_rows)) continue;
        if (swiglu) v0 = (v1 / (1.0f + expf(-v1))) * v0;  // v1 = gate, v0 = up
        else if (p.epi == OXB_GEMV_ACCUM) v0 += p.y[row];
        else if (p.epi == OXB_GEMV_RESIDUAL) v0 += p.residual[row];
        p.y[row] = v0;
    }
}

// The same grid, waves, ring and addresses as gemv_kernel, and no arithmetic beyond an OR.
template <int FMT, int NSBW, int TG>
__global__ __launch_bounds__(512) void stream_floor_kernel(const OxbGemvParams p) {
    const uint32_t lane = threadIdx.x & 63u, s = threadIdx.x >> 6;
    const uint32_t lane_c = lane * 16u, lane_s = (lane & 15u) * 8u;
    const uint32_t sb0 = __builtin_amdgcn_readfirstlane(p.sb_begin + s * NSBW);
    const int sb_lim = (int)(p.sb_begin + p.sb_count) - (int)sb0;
    const __amdgpu_buffer_rsrc_t r_codes = make_rsrc(p.codes, p.codes_bytes);
    const __amdgpu_buffer_rsrc_t r_scales = make_rsrc(p.scales, p.scales_bytes);
    const uint32_t t_begin = blockIdx.x * p.tpw;
    const uint32_t t_end = (t_begin + p.tpw) < p.n_tiles ? (t_begin + p.tpw) : p.n_tiles;
    TileRegs<FMT, NSBW> ring[TG];
#pragma unroll
    for (int t = 0; t < TG; t++) load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, t_begin + t, t_begin + t < t_end, p.n_sb, sb0, sb_lim, lane_c, lane_s);
    uint32_t acc = 0;
    for (uint32_t grp = 0; grp < p.tpw / TG; grp++) {
#pragma unroll
        for (int t = 0; t < TG; t++) {
            const uint32_t slot = t_begin + grp * TG + t;
#pragma unroll
            for (int i = 0; i < NSBW; i++) {
#pragma unroll
                for (int u = 0; u < TileRegs<FMT, NSBW>::UNITS; u++)
                    acc |= (uint32_t)(ring[t].w[i][u][0] | ring[t].w[i][u][1] | ring[t].w[i][u][2] | ring[t].w[i][u][3]);
                acc |= ring[t].sc[i].x | ring[t].sc[i].y;
            }
            load_tile<FMT, NSBW>(ring[t], r_codes, r_scales, slot + TG, slot + TG < t_end, p.n_sb, sb0, sb_lim, lane_c, lane_s);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (acc == 0x12345678u && p.y) p.y[threadIdx.x] = 1.f;  // practically never true; keeps the loads alive
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
// Upload-time repack on the device: the reference's blocks (Q1 18 B [d f16][qs 16], TQ2 34 B [qs 32][d f16], row
// after row) -> the resident codes and scales sections, padding included.  It writes what the host routine
// oxb_repack_aos_to_tiled writes (the reformatters cuda_graph/cudagraph_reformat_q1_aos_to_soa_group.rs:21-41 and
// cudagraph_reformat_tq2_blocks_to_soa_group.rs:16-27 are its counterparts).  One workgroup per (tile, superblock)
// unit, one thread per output dword: stores are contiguous, the 2-byte-aligned block bytes are read as halves.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void repack_kernel(OxbLayout L, const uint16_t* __restrict__ aos,
                                                     uint32_t* __restrict__ codes, uint16_t* __restrict__ scales) {
    const uint32_t bpr = L.k / OXB_QK;
    const uint32_t tile = blockIdx.x / L.n_sb, sb = blockIdx.x % L.n_sb;
    const uint32_t t = threadIdx.x;
    const uint32_t halves = L.fmt == OXB_FMT_Q1 ? OXB_Q1_AOS_BYTES / 2 : OXB_TQ2_AOS_BYTES / 2;
    if (t < 64) {  // scale [r][q]
        const uint32_t r = t >> 2, q = t & 3u, row = tile * 16 + r, blk = sb * 4 + q;
        uint16_t d = 0;
        if (row < L.n_rows && blk < bpr) {
            const uint16_t* b = aos + ((size_t)row * bpr + blk) * halves;
            d = L.fmt == OXB_FMT_Q1 ? b[0] : b[16];
        }
        scales[(size_t)blockIdx.x * 64 + t] = d;
    }
    for (uint32_t dwi = t; dwi < L.unit_dwords; dwi += 256) {
        uint32_t out = 0;
        if (L.fmt == OXB_FMT_Q1) {  // dword = lane * 4 + q, lane = g * 16 + r
            const uint32_t q = dwi & 3u, lane = dwi >> 2, r = lane & 15u, g = lane >> 4;
            const uint32_t row = tile * 16 + r, blk = sb * 4 + q;
            if (row < L.n_rows && blk < bpr) {
                const uint16_t* b = aos + ((size_t)row * bpr + blk) * halves + 1 + 2 * g;
                out = (uint32_t)b[0] | ((uint32_t)b[1] << 16);
            }
        } else {  // dword = half * 256 + lane * 4 + e * 2 + m
            const uint32_t half = dwi >> 8, lane = (dwi >> 2) & 63u, e = (dwi >> 1) & 1u, m = dwi & 1u;
            const uint32_t r = lane & 15u, g = lane >> 4;
            const uint32_t row = tile * 16 + r, blk = sb * 4 + half * 2 + e;
            if (row < L.n_rows && blk < bpr) {
                const uint16_t* b = aos + ((size_t)row * bpr + blk) * halves + 2 * (2 * g + m);
                const uint32_t w = (uint32_t)b[0] | ((uint32_t)b[1] << 16);
                for (uint32_t i = 0; i < 16; i++) out |= oxb_tq2_encode_field((w >> (2 * i)) & 3u, i) << (2 * i);
            }
        }
        codes[(size_t)blockIdx.x * L.unit_dwords + dwi] = out;
    }
}

// silu(gate) * up (simd_float_ops.rs:217-236) for rows whose GEMV took several launches.
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ gu, uint32_t inter, float* __restrict__ out, uint32_t ldo) {
    const uint32_t v = blockIdx.y, i = blockIdx.x * 256 + threadIdx.x;
    if (i >= inter) return;
    const float g = gu[(size_t)v * 2 * inter + i], u = gu[(size_t)v * 2 * inter + inter + i];
    out[(size_t)v * ldo + i] = (g / (1.0f + expf(-g))) * u;
}

// ---------------------------------------------------------------------------
// Host-side launchers.
// ---------------------------------------------------------------------------
struct GemvPlan {
    uint32_t nsbw, S, tg, tpw, grid;
};

// Waves split K (one to three superblocks each, eight waves at most); about one workgroup per CU, each taking whole
// groups of TG tiles.  TG is limited by the registers the ring needs; among the allowed values the one with the least
// padded work wins, weighted by how well a ring of that depth hides the load latency.
static bool plan_gemv(int fmt, const OxbGemvParams& p, uint32_t n_cus, GemvPlan* pl) {
    if (p.sb_count == 0 || p.sb_count > OXB_GEMV_MAX_SB) return false;
    pl->nsbw = (p.sb_count + 7u) / 8u;
    pl->S = (p.sb_count + pl->nsbw - 1) / pl->nsbw;
    const bool swiglu = p.epi == OXB_GEMV_SWIGLU;
    if (swiglu && ((p.n_tiles & 1u) || (p.n_rows & 31u))) return false;  // whole gate and up tiles
    const uint32_t units = swiglu ? p.n_tiles / 2 : p.n_tiles;
    uint32_t tg_max = 1;
    if (pl->nsbw == 1) tg_max = (fmt == OXB_FMT_Q1 && !(p.xq && p.nvg == 2)) ? 4u : 3u;  // (eight vectors x four tiles: 64 KB of partial sums)
    else if (pl->nsbw == 2) tg_max = fmt == OXB_FMT_Q1 ? 2u : 1u;
    const uint32_t per = (units + n_cus - 1) / n_cus;
    static const uint32_t ring_weight[5] = {0, 130, 108, 103, 100};
    uint32_t best = 0xFFFFFFFFu;
    for (uint32_t t = tg_max; t >= 1; t--) {
        const uint32_t padded = (per + t - 1) / t * t, cost = padded * ring_weight[t];
        if (cost < best) best = cost, pl->tg = t, pl->tpw = padded;
    }
    pl->grid = (units + pl->tpw - 1) / pl->tpw;
    if (swiglu) pl->tpw *= 2;
    return true;
}

template <int FMT, int NSBW, int TG>
static hipError_t launch_gemv_t(const OxbGemvParams& p, const GemvPlan& pl, hipStream_t st) {
    const size_t shm = oxb_gemv_lds_bytes(pl.S, NSBW, TG);
    if (p.pro == OXB_GEMV_PRO_RMSNORM)
        hipLaunchKernelGGL((gemv_kernel<FMT, NSBW, TG, OXB_GEMV_PRO_RMSNORM>), dim3(pl.grid), dim3(pl.S * 64), shm, st, p);
    else
        hipLaunchKernelGGL((gemv_kernel<FMT, NSBW, TG, OXB_GEMV_PRO_F32>), dim3(pl.grid), dim3(pl.S * 64), shm, st, p);
    return hipGetLastError();
}

template <int FMT, int NSBW, int TG>
static hipError_t launch_gemv_f4_t(const OxbGemvParams& p, const GemvPlan& pl, hipStream_t st) {
    const size_t shm = oxb_gemv_f4_lds_bytes(pl.S, TG);
    if (p.pro == OXB_GEMV_PRO_RMSNORM)
        hipLaunchKernelGGL((gemv_f4_kernel<FMT, NSBW, TG, OXB_GEMV_PRO_RMSNORM>), dim3(pl.grid), dim3(pl.S * 64), shm, st, p);
    else
        hipLaunchKernelGGL((gemv_f4_kernel<FMT, NSBW, TG, OXB_GEMV_PRO_F32>), dim3(pl.grid), dim3(pl.S * 64), shm, st, p);
    return hipGetLastError();
}

template <int FMT, int NSBW, int TG>
static hipError_t launch_floor_t(const OxbGemvParams& p, const GemvPlan& pl, hipStream_t st) {
    hipLaunchKernelGGL((stream_floor_kernel<FMT, NSBW, TG>), dim3(pl.grid), dim3(pl.S * 64), 0, st, p);
    return hipGetLastError();
}

template <int FMT, int NSBW, int TG, int NVG>
static hipError_t launch_gemv_packed_t(const OxbGemvParams& p, const GemvPlan& pl, hipStream_t st) {
    const size_t shm = oxb_gemv_packed_lds_bytes(pl.S, TG, NVG);
    if (NSBW >= 2 && p.epi != OXB_GEMV_SWIGLU && pl.tpw == (uint32_t)TG)
        hipLaunchKernelGGL((gemv_packed_kernel<FMT, NSBW, TG, NVG, NSBW >= 2>), dim3(pl.grid), dim3(pl.S * 64), shm, st, p);
    else
        hipLaunchKernelGGL((gemv_packed_kernel<FMT, NSBW, TG, NVG, false>), dim3(pl.grid), dim3(pl.S * 64), shm, st, p);
    return hipGetLastError();
}
template <int FMT, int NSBW, int TG>
static hipError_t launch_gemv_packed1_t(const OxbGemvParams& p, const GemvPlan& pl, hipStream_t st) {
    return launch_gemv_packed_t<FMT, NSBW, TG, 1>(p, pl, st);
}
template <int FMT, int NSBW, int TG>
static hipError_t launch_gemv_packed2_t(const OxbGemvParams& p, const GemvPlan& pl, hipStream_t st) {
    return launch_gemv_packed_t<FMT, NSBW, TG, 2>(p, pl, st);
}

#define OXB_GEMV_CASES(LAUNCH)                                                                                        \
    OXB_CASE(OXB_FMT_Q1, 1, 1, LAUNCH) OXB_CASE(OXB_FMT_Q1, 1, 2, LAUNCH) OXB_CASE(OXB_FMT_Q1, 1, 3, LAUNCH)         \
    OXB_CASE(OXB_FMT_Q1, 1, 4, LAUNCH) OXB_CASE(OXB_FMT_Q1, 2, 1, LAUNCH) OXB_CASE(OXB_FMT_Q1, 2, 2, LAUNCH)         \
    OXB_CASE(OXB_FMT_Q1, 3, 1, LAUNCH) OXB_CASE(OXB_FMT_TQ2, 1, 1, LAUNCH) OXB_CASE(OXB_FMT_TQ2, 1, 2, LAUNCH)       \
    OXB_CASE(OXB_FMT_TQ2, 1, 3, LAUNCH) OXB_CASE(OXB_FMT_TQ2, 2, 1, LAUNCH) OXB_CASE(OXB_FMT_TQ2, 3, 1, LAUNCH)
#define OXB_CASE(F, N, T, LAUNCH) \
    if (fmt == F && pl.nsbw == N && pl.tg == T) return LAUNCH<F, N, T>(p, pl, st);

static bool check_gemv_args(const OxbGemvParams& p) {
    if (p.nvec == 0 || p.nvec > (p.xq ? OXB_GEMV_PACKED_MAX_BATCH : OXB_GEMV_MAX_BATCH)) return false;
    if (p.xq && (p.nvg != (p.nvec + 3) / 4 || p.xq_bytes < oxb_gemv_pack_dwords(p.n_sb, p.nvg) * 4)) return false;
    if (p.codes_bytes >= 0x7FFFFFFFull || (uint64_t)p.k * 4 >= 0x7FFFFFFFull) return false;
    if (p.pro != OXB_GEMV_PRO_F32 && p.pro != OXB_GEMV_PRO_RMSNORM) return false;
    if (p.pro == OXB_GEMV_PRO_RMSNORM && !p.norm_w) return false;
    if (p.epi == OXB_GEMV_RESIDUAL && !p.residual) return false;
    if (p.epi == OXB_GEMV_SWIGLU && (p.sb_begin != 0 || p.sb_count != p.n_sb)) return false;  // needs the whole K
    return p.epi >= OXB_GEMV_STORE && p.epi <= OXB_GEMV_SWIGLU;
}

hipError_t oxb_launch_gemv(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st) {
    if (p.n_tiles == 0) return hipSuccess;
    GemvPlan pl;
    // The fp4 kernel's registers let two workgroups share a CU; that pays where a workgroup has many tiles to
    // spread its prologue over (the LM head: 18 -> 16.8 us), and costs where it has few (the second prologue).
    const bool many = p.epi != OXB_GEMV_SWIGLU && p.n_tiles >= 32u * n_cus;
    const bool f4 = p.nvec == 1 && !p.xq;
    if (f4 && many) n_cus *= 2;
    if (!check_gemv_args(p) || !plan_gemv(fmt, p, n_cus, &pl)) return hipErrorInvalidValue;
    p.tpw = pl.tpw;
    if (p.xq) {  // operands from the packer: one pass over the weights for up to eight vectors
        if (p.nvg == 1) {
            OXB_GEMV_CASES(launch_gemv_packed1_t)
        } else {
            OXB_GEMV_CASES(launch_gemv_packed2_t)
        }
        return hipErrorInvalidValue;
    }
    if (f4) {  // one vector, either format: the fp4 route
        OXB_GEMV_CASES(launch_gemv_f4_t)
    }
    OXB_GEMV_CASES(launch_gemv_t)
    return hipErrorInvalidValue;
}

size_t oxb_gemv_pack_bytes(uint32_t k, uint32_t nvec) {
    return oxb_gemv_pack_dwords((k / OXB_QK + 3) / 4, (nvec + 3) / 4) * 4;
}

hipError_t oxb_launch_gemv_pack(int fmt, int pro, const float* d_x, uint32_t ldx, uint32_t nvec, uint32_t k, const float* d_norm_w,
                                uint32_t* d_out, hipStream_t st) {
    const uint32_t n_sb = (k / OXB_QK + 3) / 4, nvg = (nvec + 3) / 4;
    if (nvec == 0 || nvg > OXB_GEMV_PACKED_MAX_BATCH / 4 || n_sb == 0 || (pro == OXB_GEMV_PRO_RMSNORM && !d_norm_w)) return hipErrorInvalidValue;
    const dim3 grid(n_sb, nvg * 4);
    if (fmt == OXB_FMT_Q1 && pro == OXB_GEMV_PRO_RMSNORM)
        hipLaunchKernelGGL((gemv_pack_kernel<OXB_FMT_Q1, OXB_GEMV_PRO_RMSNORM>), grid, dim3(64), 0, st, d_x, ldx, nvec, k, d_norm_w, n_sb, nvg, d_out);
    else if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL((gemv_pack_kernel<OXB_FMT_Q1, OXB_GEMV_PRO_F32>), grid, dim3(64), 0, st, d_x, ldx, nvec, k, d_norm_w, n_sb, nvg, d_out);
    else if (pro == OXB_GEMV_PRO_RMSNORM)
        hipLaunchKernelGGL((gemv_pack_kernel<OXB_FMT_TQ2, OXB_GEMV_PRO_RMSNORM>), grid, dim3(64), 0, st, d_x, ldx, nvec, k, d_norm_w, n_sb, nvg, d_out);
    else
        hipLaunchKernelGGL((gemv_pack_kernel<OXB_FMT_TQ2, OXB_GEMV_PRO_F32>), grid, dim3(64), 0, st, d_x, ldx, nvec, k, d_norm_w, n_sb, nvg, d_out);
    return hipGetLastError();
}

hipError_t oxb_launch_gemv_stream_floor(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st) {
    if (p.n_tiles == 0) return hipSuccess;
    GemvPlan pl;
    p.epi = OXB_GEMV_STORE;
    if (p.n_tiles >= 32u * n_cus) n_cus *= 2;  // as the single-vector route plans it 
    if (!plan_gemv(fmt, p, n_cus, &pl)) return hipErrorInvalidValue;
    p.tpw = pl.tpw;
    OXB_GEMV_CASES(launch_floor_t)
    return hipErrorInvalidValue;
}
#undef OXB_CASE

hipError_t oxb_launch_swiglu(const float* d_gu, uint32_t inter, uint32_t nvec, float* d_out, uint32_t ldo, hipStream_t st) {
    if (inter == 0 || nvec == 0) return hipSuccess;
    hipLaunchKernelGGL(swiglu_kernel, dim3((inter + 255) / 256, nvec), dim3(256), 0, st, d_gu, inter, d_out, ldo);
    return hipGetLastError();
}

hipError_t oxb_launch_dequant(const OxbLayout& L, const uint32_t* d_codes, const uint16_t* d_scales, float* d_out,
                              hipStream_t st) {
    const uint64_t total = (uint64_t)L.n_rows * (L.k / OXB_QK) * 4;
    if (total == 0) return hipSuccess;
    const uint32_t grid = (uint32_t)((total + 255) / 256);
    hipLaunchKernelGGL(dequant_kernel, dim3(grid), dim3(256), 0, st, L, d_codes, d_scales, d_out);
    return hipGetLastError();
}

hipError_t oxb_launch_repack(const OxbLayout& L, const uint8_t* d_aos, uint32_t* d_codes, uint16_t* d_scales, hipStream_t st) {
    const uint64_t units = (uint64_t)L.n_tiles * L.n_sb;
    if (units == 0) return hipSuccess;
    if (units > 0x7FFFFFFFull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(repack_kernel, dim3((uint32_t)units), dim3(256), 0, st, L, reinterpret_cast<const uint16_t*>(d_aos),
                       d_codes, d_scales);
    return hipGetLastError();
}
