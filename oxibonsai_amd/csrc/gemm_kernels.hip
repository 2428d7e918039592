// gemm_kernels.hip — prefill GEMM for Q1_0_g128 / TQ2_0_g128 weights on gfx950:
//     Y[m][n] = sum_k W[n][k] * X[m][k]      (X: M token rows, W: the resident quantised matrix)
// (reference semantics: crates/oxibonsai-kernels/src/gemm.rs:19-87, gemm_ternary.rs:35-69; the CUDA tier's
// scalar-FMA kernels gemm_q1_g128_v7 / gemm_tq2_g128_v7, gpu_backend/cuda_prefill_kernels.rs:74-140, 457-551).
//
// Arithmetic.  Weights +-d / 0 are exact in fp16 and so is every product with an fp16 activation in the fp32
// accumulator of v_mfma_f32_16x16x32_f16; the only rounding beyond fp32 summation is the activation's
// conversion to fp16 (relative 2^-11 per element), after scaling each token row by a power of two so the
// result does not depend on the row's magnitude.
//
// Data flow.  The weight side never touches LDS: the resident layout (layout.h) already hands lane (r, g) of a
// wave the code bits of row r, k-group g, which is the MFMA A-operand position, so each lane expands its own
// bits to fp16 +-d in registers.  Because the k order inside an MFMA is free as long as A and B agree, the
// expansion pairs weights whose codes lie 16 bits apart in a code dword (one shift + one mask builds two fp16
// values) and the activation packer writes X in exactly that order:
//   xh[(blk * 16 + 4g + s) * M_pad + m]  = 16 bytes = the 8 fp16 that lane (token m, k-group g) feeds to MFMA
//   step s of block blk;  element 2p+h  <->  k = 128 blk + 32 g + 4 s + p + 16 h            (Q1)
//                                             k = 128 blk + 32 g + 16 (s/2) + 4 (s%2) + p + 8 h   (TQ2)
// One workgroup = 4 waves stacked along the weight rows; they share one token tile of X that is staged per
// 128-weight block through double-buffered LDS.  Wave w owns up to RT row tiles (16 rows each) and CT token
// tiles (16 tokens each): RT*CT accumulator tiles, RT decoded A operands reused over CT B operands.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "gemm_kernels.h"
#include "layout.h"

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

#define OXB_GEMM_THREADS 256

// ---------------------------------------------------------------------------
// Activation packer, fused with the row-wise producer of the activations:
//   OXB_PACK_IDENT   a[m][k] = x[m][k]
//   OXB_PACK_RMSNORM a[m][k] = w[k] * x[m][k] / sqrt(mean_k x[m][k]^2 + eps)      (simd_float_ops.rs:204-215)
// Two kernels: row_stats (one workgroup per token row) finds the row's multiplier - the producer's scalar
// times the power of two that puts the row's largest |a| into [2^14, 2^15) - and the exponent that undoes the
// power of two; xh_pack (one workgroup = 16 token rows x a share of the blocks) recomputes a from x and writes
// fp16 in MFMA B-operand order.  The normalised activations never go to memory in fp32.  (SwiGLU is not a packer
// operation: the gate || up GEMM applies it in its epilogue, simd_float_ops.rs:217-236.)  A few token rows (decode batches)
// take both steps in one launch, xh_pack_rows, one workgroup per row.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    const v2h h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.0f + expf(-g))) * u; }

// Multiplier and exponent of one token row from the threads' partial results (sum of squares of x, largest |a|,
// non-finite seen); all 256 threads of the workgroup call it, thread 0 gets the result.
template <int OP>
__device__ __forceinline__ void row_finish(float ss, float mx, int bad, uint32_t k, float eps, float* red_s, float* red_m,
                                           int* red_b, float* mul_out, int32_t* xsh_out);

// The same with the pass over the row in front: a float4 per thread and step, in row order.
template <int OP>
__device__ __forceinline__ void row_stats(const float* __restrict__ xr, const float* __restrict__ w, uint32_t k, float eps,
                                          float* red_s, float* red_m, int* red_b, float* mul_out, int32_t* xsh_out) {
    const uint32_t tid = threadIdx.x;
    float ss = 0.f, mx = 0.f;
    int bad = 0;
    for (uint32_t i = tid * 4; i < k; i += 1024) {
        const float4 v = *reinterpret_cast<const float4*>(xr + i);
        float4 a = v;
        if (OP == OXB_PACK_RMSNORM) {
            const float4 g = *reinterpret_cast<const float4*>(w + i);
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
            a = make_float4(g.x * v.x, g.y * v.y, g.z * v.z, g.w * v.w);
        }
        bad |= !(fabsf(a.x) <= 3.402823466e38f) | !(fabsf(a.y) <= 3.402823466e38f) | !(fabsf(a.z) <= 3.402823466e38f) |
               !(fabsf(a.w) <= 3.402823466e38f);
        mx = fmaxf(fmaxf(mx, fmaxf(fabsf(a.x), fabsf(a.y))), fmaxf(fabsf(a.z), fabsf(a.w)));
    }
    row_finish<OP>(ss, mx, bad, k, eps, red_s, red_m, red_b, mul_out, xsh_out);
}

template <int OP>
__device__ __forceinline__ void row_finish(float ss, float mx, int bad, uint32_t k, float eps, float* red_s, float* red_m,
                                           int* red_b, float* mul_out, int32_t* xsh_out) {
    const uint32_t tid = threadIdx.x;
    ss = wave_sum_f32(ss);  // DPP and lane swaps: no trips through the LDS pipeline
    mx = wave_max_f32(mx);
    bad = __builtin_amdgcn_ballot_w64(bad != 0) != 0;
    if ((tid & 63u) == 0) red_s[tid >> 6] = ss, red_m[tid >> 6] = mx, red_b[tid >> 6] = bad;
    __syncthreads();
    if (tid == 0) {
        ss = red_s[0] + red_s[1] + red_s[2] + red_s[3];
        mx = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
        bad = red_b[0] | red_b[1] | red_b[2] | red_b[3];
        float scalar = 1.0f;
        if (OP == OXB_PACK_RMSNORM) {
            scalar = 1.0f / sqrtf(ss / (float)k + eps);
            mx *= scalar;
            bad |= !(fabsf(scalar) <= 3.402823466e38f) | !(fabsf(mx) <= 3.402823466e38f);
        }
        int E = 0;
        if (mx > 0.0f) (void)frexpf(mx, &E);  // mx = f * 2^E, f in [0.5, 1)
        const int shift = mx > 0.0f ? 15 - E : 0;
        *mul_out = bad ? 0.0f : ldexpf(scalar, shift);
        *xsh_out = bad ? INT32_MIN : -shift;
    }
}

template <int OP>
__global__ __launch_bounds__(256) void row_stats_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         uint32_t ldx, uint32_t k, float eps, float* __restrict__ rowmul,
                                                         int32_t* __restrict__ xsh) {
    __shared__ float red_s[4], red_m[4];
    __shared__ int red_b[4];
    const uint32_t m = blockIdx.x;
    float mul = 0.f;
    int32_t e = 0;
    row_stats<OP>(x + (size_t)m * ldx, w, k, eps, red_s, red_m, red_b, &mul, &e);
    if (threadIdx.x == 0) rowmul[m] = mul, xsh[m] = e;
}

// The eight activations of token row xr that chunk c = 4g + s of block blk holds, scaled by mul, as four fp16 pairs.
template <int FMT, int OP>
__device__ __forceinline__ uint4 pack_item(const float* __restrict__ xr, const float* __restrict__ w, uint32_t k, uint32_t blk,
                                           uint32_t c, float mul) {
    const uint32_t g = c >> 2, s = c & 3u;
    const uint32_t k0 = FMT == OXB_FMT_Q1 ? 32 * g + 4 * s : 32 * g + 16 * (s >> 1) + 4 * (s & 1u);
    const uint32_t k1 = k0 + (FMT == OXB_FMT_Q1 ? 16 : 8);
    const float* xb = xr + blk * 128;
    float4 a = *reinterpret_cast<const float4*>(xb + k0);
    float4 b = *reinterpret_cast<const float4*>(xb + k1);
    if (OP == OXB_PACK_RMSNORM) {
        const float4 wa = *reinterpret_cast<const float4*>(w + blk * 128 + k0), wb = *reinterpret_cast<const float4*>(w + blk * 128 + k1);
        a = make_float4(wa.x * a.x, wa.y * a.y, wa.z * a.z, wa.w * a.w);
        b = make_float4(wb.x * b.x, wb.y * b.y, wb.z * b.z, wb.w * b.w);
    }
    return make_uint4(pack_h2(a.x * mul, b.x * mul), pack_h2(a.y * mul, b.y * mul), pack_h2(a.z * mul, b.z * mul),
                      pack_h2(a.w * mul, b.w * mul));
}

// The two 16-byte pieces of token row xr behind chunk c = 4g + s of block blk (pack_item's loads).
template <int FMT>
__device__ __forceinline__ void item_offsets(uint32_t blk, uint32_t c, uint32_t* o0, uint32_t* o1) {
    const uint32_t g = c >> 2, s = c & 3u;
    const uint32_t k0 = FMT == OXB_FMT_Q1 ? 32 * g + 4 * s : 32 * g + 16 * (s >> 1) + 4 * (s & 1u);
    *o0 = blk * 128 + k0;
    *o1 = *o0 + (FMT == OXB_FMT_Q1 ? 16 : 8);
}

// Both steps in one launch for a few token rows (decode batches): one workgroup per token row, one pass over the row.
// A thread requests all of its items - the pieces it will pack, NI of them for rows of up to 2048 NI values - before
// it uses any, keeps them in registers while the workgroup finds the row's multiplier, and packs them from there;
// rows M .. M_pad - 1 are zero-filled.  With eight to thirty-two workgroups on the whole GPU the launch is as long
// as its chain of memory round trips: this way it is one for the row and one for the store.  (The sum of squares adds
// the row's values in another order than row_stats does: the multiplier may differ from the two-kernel route's in the
// last bit, within what fp16 activations already cost.)
template <int FMT, int OP, int NI>
__global__ __launch_bounds__(256) void xh_pack_rows_kernel(const float* __restrict__ x, const float* __restrict__ w, uint32_t ldx,
                                                            uint32_t k, float eps, uint32_t M, uint32_t M_pad, uint32_t nblk_pad,
                                                            int32_t* __restrict__ xsh, uint4* __restrict__ xh) {
    __shared__ float red_s[4], red_m[4];
    __shared__ int red_b[4];
    __shared__ float mul_s;
    const uint32_t m = blockIdx.x, tid = threadIdx.x, n_items = nblk_pad * 16;
    if (m >= M) {  // uniform over the workgroup
        for (uint32_t id = tid; id < n_items; id += 256) xh[(size_t)id * M_pad + m] = make_uint4(0, 0, 0, 0);
        return;
    }
    const float* xr = x + (size_t)m * ldx;
    float4 a[NI], b[NI], wa[NI], wb[NI];
#pragma unroll
    for (int it = 0; it < NI; it++) {
        const uint32_t id = it * 256 + tid;
        uint32_t o0, o1;
        item_offsets<FMT>(id >> 4, id & 15u, &o0, &o1);
        const bool ok = id < n_items && (id >> 4) * 128 < k;  // blocks past k are padding
        a[it] = ok ? *reinterpret_cast<const float4*>(xr + o0) : make_float4(0.f, 0.f, 0.f, 0.f);
        b[it] = ok ? *reinterpret_cast<const float4*>(xr + o1) : make_float4(0.f, 0.f, 0.f, 0.f);
        if (OP == OXB_PACK_RMSNORM) {
            wa[it] = ok ? *reinterpret_cast<const float4*>(w + o0) : make_float4(0.f, 0.f, 0.f, 0.f);
            wb[it] = ok ? *reinterpret_cast<const float4*>(w + o1) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    float ss = 0.f, mx = 0.f;
    int bad = 0;
#pragma unroll
    for (int it = 0; it < NI; it++) {
        float4& p = a[it];
        float4& q = b[it];
        if (OP == OXB_PACK_RMSNORM) {
            ss = fmaf(p.x, p.x, fmaf(p.y, p.y, fmaf(p.z, p.z, fmaf(p.w, p.w, ss))));
            ss = fmaf(q.x, q.x, fmaf(q.y, q.y, fmaf(q.z, q.z, fmaf(q.w, q.w, ss))));
            p = make_float4(wa[it].x * p.x, wa[it].y * p.y, wa[it].z * p.z, wa[it].w * p.w);
            q = make_float4(wb[it].x * q.x, wb[it].y * q.y, wb[it].z * q.z, wb[it].w * q.w);
        }
        const float v[8] = {p.x, p.y, p.z, p.w, q.x, q.y, q.z, q.w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            bad |= !(fabsf(v[e]) <= 3.402823466e38f);
            mx = fmaxf(mx, fabsf(v[e]));
        }
    }
    float mul = 0.f;
    int32_t e = 0;
    row_finish<OP>(ss, mx, bad, k, eps, red_s, red_m, red_b, &mul, &e);
    if (tid == 0) mul_s = mul, xsh[m] = e;
    __syncthreads();
    mul = mul_s;
#pragma unroll
    for (int it = 0; it < NI; it++) {
        const uint32_t id = it * 256 + tid;
        if (id >= n_items) continue;
        const float4 p = a[it], q = b[it];
        xh[(size_t)id * M_pad + m] = make_uint4(pack_h2(p.x * mul, q.x * mul), pack_h2(p.y * mul, q.y * mul),
                                                pack_h2(p.z * mul, q.z * mul), pack_h2(p.w * mul, q.w * mul));
    }
}

template <int FMT, int OP>
__global__ __launch_bounds__(256) void xh_pack_kernel(const float* __restrict__ x, const float* __restrict__ w, uint32_t ldx,
                                                       uint32_t k, uint32_t M, uint32_t M_pad, uint32_t nblk_pad,
                                                       const float* __restrict__ rowmul, uint4* __restrict__ xh) {
    const uint32_t tid = threadIdx.x, m0 = blockIdx.x * 16;
    const uint32_t j = tid & 15u, c = tid >> 4, m = m0 + j;
    const bool live = m < M;
    const float mul = live ? rowmul[m] : 0.0f;
    for (uint32_t blk = blockIdx.y; blk < nblk_pad; blk += gridDim.y) {
        uint4 o = make_uint4(0, 0, 0, 0);
        if (live && blk * 128 < k) o = pack_item<FMT, OP>(x + (size_t)m * ldx, w, k, blk, c, mul);
        xh[(size_t)(blk * 16 + c) * M_pad + m] = o;
    }
}

// ---------------------------------------------------------------------------
// GEMM.
// ---------------------------------------------------------------------------
// Codes and scales of one row tile for half a superblock (two 128-weight blocks), as loaded: the unit of the
// in-place register ring (half 0 is reloaded for the next superblock while half 1 is still being consumed).
template <int FMT>
struct HalfRegs {
    uint32_t c[FMT == OXB_FMT_Q1 ? 2 : 4];  // Q1: dword e = sign bits of block e; TQ2: dwords 2e, 2e+1 = fields of block e
    uint32_t d[2];                          // fp16 scale bits of blocks 0, 1 of the half (this lane's row)
};

template <int FMT>
__device__ __forceinline__ void load_half(HalfRegs<FMT>& H, __amdgpu_buffer_rsrc_t rc, __amdgpu_buffer_rsrc_t rs,
                                          uint32_t tile, bool ok, uint32_t n_sb, uint32_t sb, int half, uint32_t lane) {
    const uint32_t r = lane & 15u;
    const uint32_t unit = tile * n_sb + sb;  // wave-uniform
    ok = ok && sb < n_sb;
    if (FMT == OXB_FMT_Q1) {
        const v2u v = __builtin_amdgcn_raw_buffer_load_b64(rc, (int)(ok ? lane * 16u + half * 8u : OXB_OOB), (int)(unit * 1024u), 0);
        H.c[0] = v.x, H.c[1] = v.y;
    } else {
        const v4i v = buf_load_b128(rc, ok ? lane * 16u + half * 1024u : OXB_OOB, unit * 2048u);
        H.c[0] = (uint32_t)v.x, H.c[1] = (uint32_t)v.y, H.c[FMT == OXB_FMT_Q1 ? 0 : 2] = (uint32_t)v.z,
        H.c[FMT == OXB_FMT_Q1 ? 1 : 3] = (uint32_t)v.w;
    }
    // scales of blocks 2 * half and 2 * half + 1 of this lane's row lie side by side
    const uint32_t sv = __builtin_amdgcn_raw_buffer_load_b32(rs, (int)(ok ? r * 8u + half * 4u : OXB_OOB), (int)(unit * 128u), 0);
    H.d[0] = sv & 0xFFFFu;
    H.d[1] = sv >> 16;
}

// Per (row tile, block) state prepared once and used by the four MFMA steps of the block.
struct BlockDec {
    uint32_t w0, w1;  // Q1: w0 = inverted sign bits (xor the scale's sign); TQ2: fields of the 16-weight halves as value+1
    uint32_t d2;      // Q1: |d| in both halves of the dword; TQ2: d in both halves
};

template <int FMT>
__device__ __forceinline__ BlockDec prepare_block(const HalfRegs<FMT>& H, int e) {
    BlockDec B;
    const uint32_t dbits = H.d[e];
    const uint32_t dd = (dbits & 0xFFFFu) * 0x00010001u;
    if (FMT == OXB_FMT_Q1) {
        // weight = bit ? d : -d  ->  sign bit = ~bit ^ sign(d)
        const uint32_t flip = (uint32_t)((int32_t)(dbits << 16) >> 31);
        B.w0 = ~H.c[e] ^ flip;
        B.w1 = 0;
        B.d2 = dd & 0x7FFF7FFFu;
    } else {
        // fields at in-byte position 3 are 2-bit two's complement (3, 0, 1 for -1, 0, +1): adding 1 modulo 4
        // turns them into value+1 like the others
        const uint32_t a = H.c[FMT == OXB_FMT_Q1 ? 0 : 2 * e], b = H.c[FMT == OXB_FMT_Q1 ? 0 : 2 * e + 1];
        B.w0 = (a & 0x3F3F3F3Fu) | (((a & 0xC0C0C0C0u) + 0x40404040u) & 0xC0C0C0C0u);
        B.w1 = (b & 0x3F3F3F3Fu) | (((b & 0xC0C0C0C0u) + 0x40404040u) & 0xC0C0C0C0u);
        B.d2 = dd;
    }
    return B;
}

// The A operands of MFMA step s (0..3) of the block for all row tiles.  Written operation by operation across
// the RT x 4 independent dwords, so that consecutive VALU instructions do not depend on each other.
template <int FMT, int RT>
__device__ __forceinline__ void decode_step(const BlockDec (&B)[RT], int s, v8h (&A)[RT]) {
    uint32_t o[RT][4];
    // The masks live in registers (VOP3 encodings take no literal), opaque to the compiler so that
    // (x & mask) | y stays one v_and_or_b32.
    uint32_t kmask, kmagic;
    if (FMT == OXB_FMT_Q1) {
        asm volatile("s_mov_b32 %0, 0x80008000" : "=s"(kmask));
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) o[rt][p] = B[rt].w0 << (15 - (4 * s + p));
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) o[rt][p] = (o[rt][p] & kmask) | B[rt].d2;
    } else {
        asm volatile("s_mov_b32 %0, 0x00030003" : "=s"(kmask));
        asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(kmagic));
        const v2h bias = {(_Float16)1025.0f, (_Float16)1025.0f};
        v2h v[RT][4];
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) o[rt][p] = ((s >> 1) ? B[rt].w1 : B[rt].w0) >> (2 * (4 * (s & 1) + p));
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) o[rt][p] = (o[rt][p] & kmask) | kmagic;  // fp16 1024 + field
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) v[rt][p] = __builtin_bit_cast(v2h, o[rt][p]) - bias;  // exact: field - 1
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int rt = 0; rt < RT; rt++) o[rt][p] = __builtin_bit_cast(uint32_t, v[rt][p] * __builtin_bit_cast(v2h, B[rt].d2));
    }
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const v4u u = {o[rt][0], o[rt][1], o[rt][2], o[rt][3]};
        A[rt] = __builtin_bit_cast(v8h, u);
    }
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// One 128-weight block of the K loop: 4 MFMA steps over the staged token tile `xsb`.  The A operands of the
// step after the current one are expanded while the current step's MFMAs run (for the last step: the first
// step of the next block, from `bdn`), and each B operand is reloaded for the next step right after its last use.
template <int FMT, int RT, int CT>
__device__ __forceinline__ void block_steps(const v8h* __restrict__ xsb, v8h (&A)[RT], const BlockDec (&bd)[RT],
                                            const BlockDec (&bdn)[RT], v4f (&acc)[RT][CT], uint32_t boff) {
    constexpr int BM = 16 * CT;
    constexpr int NV = FMT == OXB_FMT_Q1 ? 1 : 2;  // VALU instructions issued after each MFMA
    v8h B[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) B[ct] = xsb[boff + ct * 16];
    // all B operands of the first step are requested at once, so their LDS latency is paid once per block
    __builtin_amdgcn_sched_group_barrier(0x100, CT, 0);
#pragma unroll
    for (int s = 0; s < 4; s++) {
        v8h An[RT];
        if (s < 3)
            decode_step<FMT, RT>(bd, s + 1, An);
        else
            decode_step<FMT, RT>(bdn, 0, An);
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
#pragma unroll
            for (int rt = 0; rt < RT; rt++)  // row tiles past the range hold zero weights
                acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[rt], B[ct], acc[rt][ct], 0, 0, 0);
            if (s < 3) B[ct] = xsb[boff + (s + 1) * BM + ct * 16];
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) A[rt] = An[rt];
        // issue order: one MFMA, then the VALU work that expands the next A operand, a B reload per token tile
#pragma unroll
        for (int i = 0; i < RT * CT; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            // (the first step also absorbs the per-block preparation of the next block's codes)
            if (s == 0)
                __builtin_amdgcn_sched_group_barrier(0x002, NV + 1, 0);
            else
                __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);
            if (s < 3 && i % RT == RT - 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);  // one scheduling region per step keeps compile time bounded
    }
}

template <int FMT, int RT, int CT>
__global__ __launch_bounds__(OXB_GEMM_THREADS, RT == 3 ? 2 : 1) void gemm_mfma_kernel(const OxbGemmParams p) {
    constexpr int BM = 16 * CT;
    // two stages of the token tile: [chunk 4g+s][token] x 16 bytes.  Separate arrays, so that loads in flight
    // into one stage do not make reads of the other wait.
    __shared__ __attribute__((aligned(16))) uint4 xs0[16 * BM];
    __shared__ __attribute__((aligned(16))) uint4 xs1[16 * BM];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, g = lane >> 4;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));  // keeps unit offsets in SGPRs
    const uint32_t m_t = blockIdx.x % p.n_mt, n_g = (blockIdx.x / p.n_mt) % p.n_ng, ks = blockIdx.x / (p.n_mt * p.n_ng);
    const uint32_t m0 = m_t * BM;
    // K slice of this workgroup, in superblocks
    const uint32_t sb0 = ks * p.sb_per_split, sb1 = min(sb0 + p.sb_per_split, p.n_sb);
    // row tiles: the workgroup's [wg_t0, wg_t1), split evenly over the four waves
    const uint32_t wg_t0 = n_g * p.tpw, wg_t1 = min(wg_t0 + p.tpw, p.n_tiles);
    // SWIGLU mode (the matrix is gate || up).  Even RT: the tile sequence interleaves gate tile j and up tile j, and
    // every wave starts on a gate tile (the launcher gives it an even count), so accumulators 2q and 2q+1 hold both
    // factors of 16 output rows.  Odd RT (three tiles per wave, the count that still runs two workgroups per CU): waves 0
    // and 1 take RT gate tiles each, waves 2 and 3 the up tiles of the same rows; the up factors cross over through the
    // LDS stages once the K loop is done.
    const bool sw = p.mode == OXB_GEMM_SWIGLU;
    constexpr bool SPLIT = RT == 3;  // (of the SWIGLU mode; other odd counts are never launched in it)
    auto tile_of = [&](uint32_t u) -> uint32_t { return sw ? ((u & 1u) ? p.n_tiles / 2 + (u >> 1) : (u >> 1)) : u; };
    uint32_t t0 = 0, n_valid = 0, up_base = 0;  // first tile index of this wave (an index into tile_of, or with SPLIT a gate tile)
    if (sw && SPLIT) {
        const uint32_t half_tiles = p.n_tiles / 2, g_first = n_g * (2 * RT) + (wave & 1u) * RT;
        t0 = g_first;
        n_valid = g_first < half_tiles ? min((uint32_t)RT, half_tiles - g_first) : 0u;
        up_base = (wave >> 1) ? half_tiles : 0u;
    } else {
        const uint32_t per = (p.tpw + 3u) / 4u;  // <= RT
        t0 = wg_t0 + wave * per;
        const uint32_t t1 = min(t0 + per, wg_t1);
        n_valid = t1 > t0 ? t1 - t0 : 0u;
    }
    auto tile_at = [&](uint32_t rt) -> uint32_t { return (sw && SPLIT) ? up_base + t0 + rt : tile_of(t0 + rt); };

    const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.codes, p.codes_bytes), rs = make_rsrc(p.scales, p.scales_bytes);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.xh, p.xh_bytes);

    v4f acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int ct = 0; ct < CT; ct++) acc[rt][ct] = (v4f){0.f, 0.f, 0.f, 0.f};

    // this thread's share of an X stage: CT items of 16 bytes; item id = it*256 + tid -> chunk id / BM, token id % BM.
    // The loads write LDS directly: lane l of a wave fills bytes [16 l, 16 l + 16) after the wave's base.
    uint32_t xoff[CT];
#pragma unroll
    for (int it = 0; it < CT; it++) {
        const uint32_t id = it * OXB_GEMM_THREADS + tid, c = id / BM, j = id % BM;
        xoff[it] = m0 + j < p.M_pad ? (c * p.M_pad + m0 + j) * 16u : OXB_OOB;
    }
    const uint32_t blk_stride = 16u * p.M_pad * 16u;  // bytes of xh per block
    const uint32_t nblk = p.n_sb * 4u;
    auto stage_x = [&](uint32_t blk, uint4* xs) {
        const uint32_t soff = (blk < nblk ? blk : nblk - 1) * blk_stride;  // past the end: restage the last block
#pragma unroll
        for (int it = 0; it < CT; it++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(xs + it * OXB_GEMM_THREADS + wave * 64), 16,
                                                     (int)xoff[it], (int)soff, 0, 0);
    };
    auto publish = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // In the blocks that also request the next superblock's weights, those 2 RT loads (codes and scales of each row
    // tile, load_half) are issued after the stage's loads (memory reads return in order) and stay in flight across
    // the barrier: they come from HBM and have until the end of the following block, instead of stalling the whole
    // workgroup at the end of this one.  The count must be exactly the weight loads: one more, and a piece of the
    // token-tile stage may still be on its way when the next block reads it.
    // Measured: three row tiles per wave gain 19 % from it (QKV 6144 x 4096 at 2048 tokens: 105 -> 85 us); with two, four
    // or five tiles the time does not change or gets 3 % worse, so those keep the plain wait.
    constexpr bool KEEP_W = RT == 3;
    auto publish_keep_weights = [&]() {
        if (KEEP_W)
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * RT) : "memory");
        else
            publish();
    };

    HalfRegs<FMT> H[RT][2];
    stage_x(sb0 * 4, xs0);
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        load_half<FMT>(H[rt][0], rc, rs, tile_at(rt), (uint32_t)rt < n_valid, p.n_sb, sb0, 0, lane);
        load_half<FMT>(H[rt][1], rc, rs, tile_at(rt), (uint32_t)rt < n_valid, p.n_sb, sb0, 1, lane);
    }
    publish();
    BlockDec bd[RT], bdn[RT];
    v8h A[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) bd[rt] = prepare_block<FMT>(H[rt][0], 0);
    decode_step<FMT, RT>(bd, 0, A);
    const uint32_t boff = g * 4 * BM + r;  // this lane's B operand of step s, token tile ct: xs[boff + s*BM + 16 ct]
    const v8h* x0 = reinterpret_cast<const v8h*>(xs0);
    const v8h* x1 = reinterpret_cast<const v8h*>(xs1);

    for (uint32_t sb = sb0; sb < sb1; sb++) {
        // block 0 of the superblock
        stage_x(sb * 4 + 1, xs1);
#pragma unroll
        for (int rt = 0; rt < RT; rt++) bdn[rt] = prepare_block<FMT>(H[rt][0], 1);
        block_steps<FMT, RT, CT>(x0, A, bd, bdn, acc, boff);
        publish();
        // block 1: half 0 is consumed; reload it for the next superblock
        stage_x(sb * 4 + 2, xs0);
        if (KEEP_W) __builtin_amdgcn_sched_barrier(0);  // the stage's loads first, then the weights (see publish_keep_weights)
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            bd[rt] = bdn[rt];
            bdn[rt] = prepare_block<FMT>(H[rt][1], 0);
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) load_half<FMT>(H[rt][0], rc, rs, tile_at(rt), (uint32_t)rt < n_valid, p.n_sb, sb + 1, 0, lane);
        if (KEEP_W) __builtin_amdgcn_sched_barrier(0);
        block_steps<FMT, RT, CT>(x1, A, bd, bdn, acc, boff);
        publish_keep_weights();
        // block 2
        stage_x(sb * 4 + 3, xs1);
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            bd[rt] = bdn[rt];
            bdn[rt] = prepare_block<FMT>(H[rt][1], 1);
        }
        block_steps<FMT, RT, CT>(x0, A, bd, bdn, acc, boff);
        publish();
        // block 3: half 1 is consumed; the next block is block 0 of the next superblock (half 0, already reloaded)
        stage_x(sb * 4 + 4, xs0);
        if (KEEP_W) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            bd[rt] = bdn[rt];
            bdn[rt] = prepare_block<FMT>(H[rt][0], 0);
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) load_half<FMT>(H[rt][1], rc, rs, tile_at(rt), (uint32_t)rt < n_valid, p.n_sb, sb + 1, 1, lane);
        if (KEEP_W) __builtin_amdgcn_sched_barrier(0);
        block_steps<FMT, RT, CT>(x1, A, bd, bdn, acc, boff);
        publish_keep_weights();
#pragma unroll
        for (int rt = 0; rt < RT; rt++) bd[rt] = bdn[rt];
    }

    // epilogue: lane holds rows 4g..4g+3 of the row tile for token 16ct + r
    const bool vec_ok = (p.ldy & 3u) == 0;
    if (sw && SPLIT) {
        // The K loop ended behind a barrier with no stage load in flight: both stages are free.  Up waves leave their
        // factors (already scaled back by the row's power of two) in the stage of their half, tile by tile as
        // [rt][ct][lane] float4; the gate waves of the same half pick them up.
        float4* ex = reinterpret_cast<float4*>((wave & 1u) ? xs1 : xs0);
        static_assert(!SPLIT || (size_t)RT * CT * 64 * 16 <= sizeof(xs0), "the up factors of a wave fit a stage");
        if (wave >> 1) {
#pragma unroll
            for (int ct = 0; ct < CT; ct++) {
                const uint32_t m = m0 + ct * 16 + r;
                const int e = m < p.M ? p.xsh[m] : 0;
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    float u[4];
#pragma unroll
                    for (int v = 0; v < 4; v++) u[v] = e == INT32_MIN ? __int_as_float(0x7FC00000) : ldexpf(acc[rt][ct][v], e);
                    ex[(rt * CT + ct) * 64 + lane] = make_float4(u[0], u[1], u[2], u[3]);
                }
            }
        }
        __syncthreads();
        if (wave >> 1) return;
#pragma unroll
        for (int ct = 0; ct < CT; ct++) {
            const uint32_t m = m0 + ct * 16 + r;
            if (m >= p.M) continue;
            const int e = p.xsh[m];
            float* yr = p.y + (size_t)m * p.ldy;
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                if ((uint32_t)rt >= n_valid) continue;
                const uint32_t n = (t0 + rt) * 16 + 4 * g, n_lim = p.n_rows / 2;
                const float4 u = ex[(rt * CT + ct) * 64 + lane];
                const float uu[4] = {u.x, u.y, u.z, u.w};
                float o[4];
#pragma unroll
                for (int v = 0; v < 4; v++)
                    o[v] = silu_mul(e == INT32_MIN ? __int_as_float(0x7FC00000) : ldexpf(acc[rt][ct][v], e), uu[v]);
                if (vec_ok && n + 3 < n_lim) {
                    *reinterpret_cast<float4*>(yr + n) = make_float4(o[0], o[1], o[2], o[3]);
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++)
                        if (n + v < n_lim) yr[n + v] = o[v];
                }
            }
        }
        return;
    }
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
        const uint32_t m = m0 + ct * 16 + r;
        if (m >= p.M) continue;
        const int e = p.xsh[m];
        // with K split over workgroups, slice ks writes its partial sums to plane ks of the workspace
        float* yr = p.ksplit > 1 ? p.part + ((size_t)ks * p.M + m) * p.ldy : p.y + (size_t)m * p.ldy;
        const float* rr = (p.mode == OXB_GEMM_RESIDUAL && p.ksplit == 1) ? p.residual + (size_t)m * p.ldy : nullptr;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            if ((uint32_t)rt >= n_valid) continue;
            if (sw && (rt & 1)) continue;  // the up factor: consumed with its gate tile
            const uint32_t n = sw ? ((t0 + rt) >> 1) * 16 + 4 * g : (t0 + rt) * 16 + 4 * g;
            const uint32_t n_lim = sw ? p.n_rows / 2 : p.n_rows;
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; v++) o[v] = e == INT32_MIN ? __int_as_float(0x7FC00000) : ldexpf(acc[rt][ct][v], e);
            if (sw) {
                constexpr int ru = RT > 1 ? 1 : 0;  // (RT = 1 is never launched in this mode)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float u = e == INT32_MIN ? __int_as_float(0x7FC00000) : ldexpf(acc[rt + ru < RT ? rt + ru : rt][ct][v], e);
                    o[v] = silu_mul(o[v], u);
                }
            }
            if (vec_ok && n + 3 < n_lim) {
                if (rr) {
                    const float4 q4 = *reinterpret_cast<const float4*>(rr + n);
                    o[0] += q4.x, o[1] += q4.y, o[2] += q4.z, o[3] += q4.w;
                }
                *reinterpret_cast<float4*>(yr + n) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (n + v < n_lim) yr[n + v] = rr ? rr[n + v] + o[v] : o[v];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// GEMM for a few token rows (M <= 32: decode batches).  The wide kernel above would spend its time on barriers
// and on MFMAs over padding; here the weights stream once at GEMV-like rates.  A workgroup = 8 waves owns RT row
// tiles; the waves split K (contiguous runs of superblocks), each expands its weights and multiplies them with
// B operands read straight from the packed activations (they stay in L2, no LDS stage, no barrier in the loop),
// prefetched one block ahead; the eight partial sums meet in LDS and are added in wave order.
// ---------------------------------------------------------------------------
#define OXB_GEMM_NARROW_THREADS 512

template <int FMT, int RT, int CT>
__global__ __launch_bounds__(OXB_GEMM_NARROW_THREADS) void gemm_narrow_kernel(const OxbGemmParams p) {
    // The partial sums meet in LDS in passes of PT row tiles (all of them up to four; pairs beyond, so that the
    // array stays within 64 KB): in SWIGLU mode a pass holds gate tiles and the up tiles of the same rows.
    constexpr int PT = RT <= 4 ? RT : 2, NPASS = RT / PT;
    static_assert(RT % PT == 0, "row tiles per pass");
    __shared__ float red[8][PT * CT * 4][64];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, r = lane & 15u, g = lane >> 4;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    // Row tiles of this workgroup.  Plain modes: RT consecutive tiles.  SWIGLU mode (the matrix is gate || up,
    // RT even): RT/2 consecutive gate tiles and the up tiles of the same rows, so the epilogue holds both factors.
    const bool sw = p.mode == OXB_GEMM_SWIGLU;
    constexpr uint32_t HP = RT > 1 ? RT / 2 : 1;
    const uint32_t t0 = sw ? blockIdx.x * HP : blockIdx.x * RT;
    const uint32_t t_lim = sw ? p.n_tiles / 2 : p.n_tiles;
    auto tile_of = [&](int rt) -> uint32_t { return sw ? ((uint32_t)rt < HP ? t0 + rt : p.n_tiles / 2 + t0 + rt - HP) : t0 + rt; };
    auto valid = [&](int rt) -> bool { return sw ? t0 + ((uint32_t)rt % HP) < t_lim : t0 + rt < t_lim; };
    const uint32_t per = (p.n_sb + 7u) / 8u, sb0 = wave * per, sb1 = min(sb0 + per, p.n_sb);
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.codes, p.codes_bytes), rs = make_rsrc(p.scales, p.scales_bytes);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.xh, p.xh_bytes);

    v4f acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int ct = 0; ct < CT; ct++) acc[rt][ct] = (v4f){0.f, 0.f, 0.f, 0.f};

    if (sb0 < sb1) {
        const uint32_t blk_stride = 16u * p.M_pad * 16u;  // bytes of xh per block
        const uint32_t blk_end = sb1 * 4u;
        // B operand of step s, token tile ct of a block: chunk 4g + s, token 16 ct + r
        v8h B[2][4][CT];
        auto load_b = [&](uint32_t blk, v8h (&dst)[4][CT]) {
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int ct = 0; ct < CT; ct++) {
                    const uint32_t off = ((4u * g + s) * p.M_pad + ct * 16u + r) * 16u;
                    dst[s][ct] = __builtin_bit_cast(v8h, buf_load_b128(rx, blk < blk_end ? off : OXB_OOB, blk * blk_stride));
                }
        };
        // RING: the next superblock's weights wait in a second register set; with more than four row tiles there
        // is no room for one, and a half is requested again in place once its second block has been prepared.
        constexpr bool RING = RT <= 4;
        HalfRegs<FMT> H[RT][2], Hn[RING ? RT : 1][2];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            load_half<FMT>(H[rt][0], rc, rs, tile_of(rt), valid(rt), p.n_sb, sb0, 0, lane);
            load_half<FMT>(H[rt][1], rc, rs, tile_of(rt), valid(rt), p.n_sb, sb0, 1, lane);
        }
        load_b(sb0 * 4u, B[0]);
        for (uint32_t sb = sb0; sb < sb1; sb++) {
            // next superblock's weights (all zero past the slice: never used)
            if (RING) {
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    load_half<FMT>(Hn[RING ? rt : 0][0], rc, rs, tile_of(rt), valid(rt) && sb + 1 < sb1, p.n_sb, sb + 1, 0, lane);
                    load_half<FMT>(Hn[RING ? rt : 0][1], rc, rs, tile_of(rt), valid(rt) && sb + 1 < sb1, p.n_sb, sb + 1, 1, lane);
                }
            }
#pragma unroll
            for (int bi = 0; bi < 4; bi++) {
                load_b(sb * 4u + bi + 1, B[(bi + 1) & 1]);
                BlockDec bd[RT];
#pragma unroll
                for (int rt = 0; rt < RT; rt++) bd[rt] = prepare_block<FMT>(H[rt][bi >> 1], bi & 1);
                if (!RING && (bi & 1) && sb + 1 < sb1) {  // (wave-uniform) both blocks of the half are in bd now
#pragma unroll
                    for (int rt = 0; rt < RT; rt++) load_half<FMT>(H[rt][bi >> 1], rc, rs, tile_of(rt), valid(rt), p.n_sb, sb + 1, bi >> 1, lane);
                }
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    v8h A[RT];
                    decode_step<FMT, RT>(bd, s, A);
#pragma unroll
                    for (int ct = 0; ct < CT; ct++)
#pragma unroll
                        for (int rt = 0; rt < RT; rt++)  // row tiles past the range hold zero weights
                            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[rt], B[bi & 1][s][ct], acc[rt][ct], 0, 0, 0);
                }
            }
            if (RING) {
#pragma unroll
                for (int rt = 0; rt < RT; rt++) H[rt][0] = Hn[RING ? rt : 0][0], H[rt][1] = Hn[RING ? rt : 0][1];
            }
        }
    }
    // row tile behind slot q of pass ps: all tiles in order with a single pass; with pairs, SWIGLU mode takes a gate
    // tile and the up tile of the same rows, the plain modes two neighbours
    auto pass_rt = [&](int ps, int q) -> int { return NPASS == 1 ? q : (sw ? ps + q * (int)HP : ps * PT + q); };
#pragma unroll
    for (int ps = 0; ps < NPASS; ps++) {
    if (ps) __syncthreads();  // the last pass has been read
#pragma unroll
    for (int q = 0; q < PT; q++)
#pragma unroll
        for (int ct = 0; ct < CT; ct++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                // (constant register indices in both arms: the choice is a select, not an indexed array)
                const int rt_sw = NPASS == 1 ? q : ps + q * (int)HP, rt_pl = NPASS == 1 ? q : ps * PT + q;
                red[wave][(q * CT + ct) * 4 + v][lane] = sw ? acc[rt_sw < RT ? rt_sw : 0][ct][v] : acc[rt_pl][ct][v];
            }
    __syncthreads();
    // wave w finishes the accumulator tiles w, w + 8, ...: lane holds rows 4g..4g+3 of row tile rt for token 16ct + r
    const bool vec_ok = (p.ldy & 3u) == 0;
    auto total = [&](uint32_t idx, float (&o)[4], int e) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            float a = red[0][idx * 4 + v][lane];
#pragma unroll
            for (int w = 1; w < 8; w++) a += red[w][idx * 4 + v][lane];
            o[v] = e == INT32_MIN ? __int_as_float(0x7FC00000) : ldexpf(a, e);
        }
    };
    // slots of a pass that hold output rows: all of them; in SWIGLU mode the gate slots (half of a single pass, slot 0 of a pair)
    const uint32_t q_out = sw ? (NPASS == 1 ? HP : 1u) : (uint32_t)PT, q_up = NPASS == 1 ? HP : 1u;
    for (uint32_t idx = wave; idx < q_out * CT; idx += 8) {
        const uint32_t q = idx / CT, ct = idx % CT, m = ct * 16 + r;
        const uint32_t rt = (uint32_t)pass_rt(ps, (int)q);
        if (!valid((int)rt) || m >= p.M) continue;
        const int e = p.xsh[m];
        float o[4];
        total(idx, o, e);
        if (sw) {  // y[m][row] = silu(gate) * up, rows counted within the gate half
            float u[4];
            total((q + q_up) * CT + ct, u, e);
#pragma unroll
            for (int v = 0; v < 4; v++) o[v] = silu_mul(o[v], u[v]);
        }
        float* yr = p.y + (size_t)m * p.ldy;
        const float* rr = p.mode == OXB_GEMM_RESIDUAL ? p.residual + (size_t)m * p.ldy : nullptr;
        const uint32_t n = (t0 + rt) * 16 + 4 * g, n_lim = sw ? p.n_rows / 2 : p.n_rows;
        if (vec_ok && n + 3 < n_lim) {
            if (rr) {
                const float4 q4 = *reinterpret_cast<const float4*>(rr + n);
                o[0] += q4.x, o[1] += q4.y, o[2] += q4.z, o[3] += q4.w;
            }
            *reinterpret_cast<float4*>(yr + n) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (n + v < n_lim) yr[n + v] = rr ? rr[n + v] + o[v] : o[v];
        }
    }
    }
}

// y = (residual +) the K slices' partial sums, added in slice order (deterministic).
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part, uint32_t ksplit, size_t plane,
                                                                  const float* __restrict__ residual, float* __restrict__ y,
                                                                  size_t n4) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    float4 a = reinterpret_cast<const float4*>(part)[i];
    for (uint32_t s = 1; s < ksplit; s++) {
        const float4 b = reinterpret_cast<const float4*>(part + s * plane)[i];
        a.x += b.x, a.y += b.y, a.z += b.z, a.w += b.w;
    }
    if (residual) {
        const float4 r = reinterpret_cast<const float4*>(residual)[i];
        a.x += r.x, a.y += r.y, a.z += r.z, a.w += r.w;
    }
    reinterpret_cast<float4*>(y)[i] = a;
}

// ---------------------------------------------------------------------------
// Host-side launchers.
// ---------------------------------------------------------------------------
size_t oxb_xh_bytes(uint32_t k, uint32_t M) {
    const size_t nblk_pad = ((k + 511u) / 512u) * 4u, M_pad = (M + 15u) / 16u * 16u;
    return nblk_pad * 16 * M_pad * 16;
}

#define OXB_PACK_ROWS_MAX 64  // up to this many token rows (of at most 16384 values) the one-launch packer is used

template <int OP>
static void launch_pack_op(int fmt, const float* d_x, const float* d_w, uint32_t ldx, uint32_t k, uint32_t M, uint32_t M_pad,
                           uint32_t nblk_pad, float eps, float* d_rowmul, uint32_t* d_xh, int32_t* d_xsh, hipStream_t st) {
    const uint32_t per_thread = (nblk_pad * 16 + 255) / 256;  // items of a row per thread of the one-launch packer
    if (M <= OXB_PACK_ROWS_MAX && per_thread <= 8) {
#define OXB_ROWS_CASE(NI)                                                                                                      \
    if (per_thread <= NI) {                                                                                                    \
        if (fmt == OXB_FMT_Q1)                                                                                                 \
            hipLaunchKernelGGL((xh_pack_rows_kernel<OXB_FMT_Q1, OP, NI>), dim3(M_pad), dim3(256), 0, st, d_x, d_w, ldx, k, eps, M, \
                               M_pad, nblk_pad, d_xsh, reinterpret_cast<uint4*>(d_xh));                                        \
        else                                                                                                                   \
            hipLaunchKernelGGL((xh_pack_rows_kernel<OXB_FMT_TQ2, OP, NI>), dim3(M_pad), dim3(256), 0, st, d_x, d_w, ldx, k, eps, M, \
                               M_pad, nblk_pad, d_xsh, reinterpret_cast<uint4*>(d_xh));                                        \
        return;                                                                                                                \
    }
        OXB_ROWS_CASE(1) OXB_ROWS_CASE(2) OXB_ROWS_CASE(4) OXB_ROWS_CASE(6) OXB_ROWS_CASE(8)
#undef OXB_ROWS_CASE
    }
    hipLaunchKernelGGL(row_stats_kernel<OP>, dim3(M), dim3(256), 0, st, d_x, d_w, ldx, k, eps, d_rowmul, d_xsh);
    const dim3 grid(M_pad / 16, nblk_pad < 16 ? nblk_pad : 16);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL((xh_pack_kernel<OXB_FMT_Q1, OP>), grid, dim3(256), 0, st, d_x, d_w, ldx, k, M, M_pad, nblk_pad, d_rowmul,
                           reinterpret_cast<uint4*>(d_xh));
    else
        hipLaunchKernelGGL((xh_pack_kernel<OXB_FMT_TQ2, OP>), grid, dim3(256), 0, st, d_x, d_w, ldx, k, M, M_pad, nblk_pad, d_rowmul,
                           reinterpret_cast<uint4*>(d_xh));
}

hipError_t oxb_launch_xh_pack(int fmt, int op, const float* d_x, const float* d_w, uint32_t ldx, uint32_t k, float eps,
                              uint32_t M, float* d_rowmul, uint32_t* d_xh, int32_t* d_xsh, hipStream_t st) {
    if (M == 0 || k == 0 || (k % OXB_QK) != 0 || (ldx & 3u) != 0) return hipErrorInvalidValue;
    if (op == OXB_PACK_RMSNORM && !d_w) return hipErrorInvalidValue;
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, M_pad = (M + 15u) / 16u * 16u;
    if (oxb_xh_bytes(k, M) >= 0xFFFFFFF0ull) return hipErrorInvalidValue;
    switch (op) {
        case OXB_PACK_IDENT: launch_pack_op<OXB_PACK_IDENT>(fmt, d_x, d_w, ldx, k, M, M_pad, nblk_pad, eps, d_rowmul, d_xh, d_xsh, st); break;
        case OXB_PACK_RMSNORM: launch_pack_op<OXB_PACK_RMSNORM>(fmt, d_x, d_w, ldx, k, M, M_pad, nblk_pad, eps, d_rowmul, d_xh, d_xsh, st); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <int FMT, int RT, int CT>
static hipError_t launch_gemm_case(const OxbGemmParams& p, uint32_t grid, hipStream_t st) {
    hipLaunchKernelGGL((gemm_mfma_kernel<FMT, RT, CT>), dim3(grid), dim3(OXB_GEMM_THREADS), 0, st, p);
    return hipGetLastError();
}

struct GemmPlan { uint32_t rt, tpw, ksplit, sb_per_split, ct; };

// Row tiles per workgroup and K slices: minimise (rounds of workgroups over the CUs) x (time of one workgroup),
// where a workgroup costs, per superblock of its K slice, its row tiles per wave plus about one more for staging,
// barriers and operand latency, plus a fixed part for its start and epilogue.  Splitting K adds a pass over the
// output per slice (the partial sums are written, then added in slice order).  Ties go to the larger tile.
static GemmPlan plan_gemm(const OxbGemmParams& p, uint32_t n_cus) {
    constexpr uint32_t BM = 128;
    const uint32_t n_mt = (p.M + BM - 1) / BM;
    static const uint32_t rts[] = {5, 4, 3, 2, 1};
    GemmPlan best = {1, 4, 1, p.n_sb, 8};
    if (p.mode == OXB_GEMM_SWIGLU) best = {2, 8, 1, p.n_sb, 8};
    uint64_t best_cost = ~0ull;
    const bool sw = p.mode == OXB_GEMM_SWIGLU;  // even tile counts per wave, no K split (the epilogue is not linear)
    const bool can_split = (p.ldy & 3u) == 0 && !sw;
    for (uint32_t ks = 1; ks <= (can_split ? 8u : 1u) && ks <= p.n_sb; ks++) {
        const uint32_t spk = (p.n_sb + ks - 1) / ks;
        if (ks > 1 && (p.n_sb + spk - 1) / spk != ks) continue;  // same slices as a smaller count
        for (uint32_t rt : rts) {
            // SWIGLU: a wave takes gate and up tiles in pairs.  One pair per wave (164 registers: two workgroups per
            // CU, whose starts and epilogues overlap) measured faster than two pairs (308 registers, one workgroup per
            // CU) on both quoted gate || up shapes at 2048 tokens: 24576 x 4096 357 against 368 us, 12288 x 2048 109
            // against 121 us.
            if (sw && rt != 2) continue;  // (three tiles per wave are considered below)
            for (uint32_t tpw = 4 * rt; tpw > (sw ? 4 * rt - 1 : 4 * rt - 4); tpw--) {
                const uint32_t groups = (p.n_tiles + tpw - 1) / tpw;
                const uint64_t wgs = (uint64_t)groups * n_mt * ks;
                uint64_t cost = ((wgs + n_cus - 1) / n_cus) * ((uint64_t)spk * (rt + 1) + 2 * rt + 2);
                if (ks > 1) cost += (uint64_t)ks * 2 + 4;  // the reduction pass
                if (cost < best_cost) best_cost = cost, best = {rt, tpw, ks, spk, 8};
            }
        }
    }
    // Small matrices leave the 128-token tile short of workgroups (one or two row tiles per wave and still fewer
    // workgroups than CUs): there a 64-token tile with one row tile per wave doubles their number.  Measured at 512
    // tokens: 4096 x 4096 26.2 -> 23.0 us, 6144 x 4096 37.0 -> 33.2, 5120 x 2560 (TQ2) 26.6 -> 24.6, 4096 x 2048 17.5 ->
    // 15.8, 2048 x 2048 14.9 -> 11.4; with more workgroups to begin with the wider tile wins.
    if (!sw && best.ksplit == 1 && best.rt <= 2) {
        const uint64_t wgs = (uint64_t)((p.n_tiles + best.tpw - 1) / best.tpw) * n_mt;
        if (best.rt == 1 || wgs < n_cus) best = {1, 4, 1, p.n_sb, 4};
    }
    // gate || up with three tiles per wave (two gate waves, two up waves; still two workgroups per CU): fewer LDS reads
    // per MFMA than with two.  Measured at 2048 tokens (plain stores): 24576 x 4096 310 against 343 us, 19456 x 2560
    // (TQ2) 181 against 193, 12288 x 2048 (TQ2) 92 against 101; taken where its workgroups still cover the CUs.
    if (sw && (uint64_t)((p.n_tiles / 2 + 5) / 6) * n_mt >= n_cus) best = {3, 12, 1, p.n_sb, 8};
    return best;
}

template <int FMT, int RT, int CT>
static hipError_t launch_narrow_case(const OxbGemmParams& p, hipStream_t st) {
    const uint32_t grid = p.mode == OXB_GEMM_SWIGLU ? (p.n_tiles / 2 + RT / 2 - 1) / (RT > 1 ? RT / 2 : 1) : (p.n_tiles + RT - 1) / RT;
    hipLaunchKernelGGL((gemm_narrow_kernel<FMT, RT, CT>), dim3(grid), dim3(OXB_GEMM_NARROW_THREADS), 0, st, p);
    return hipGetLastError();
}

// Row tiles per workgroup (1, 2, 4 or - Q1 - 6): the count that minimises (rounds of workgroups over the CUs) x (row tiles + 2 - a
// workgroup's time grows with its tiles on top of a fixed part: its start, the K-split sum and the epilogue).  What
// counts is the last round: 384 workgroups of one tile leave half the CUs with two and the launch as long as those
// (QKV 6144 x 4096, 8 rows: 5.5 us against 4.7 us as 192 workgroups of two tiles; 32 rows: 8.2 against 6.1).  A tie
// goes to the larger workgroups (every workgroup reads all of the packed activations); 8B-shape decode with this rule
// against "as many tiles as leave a workgroup per CU": +2 % at 8 and at 32 sequences.  Six tiles (three gate and three up
// tiles in SWIGLU mode) make gate || up 24576 x 4096 one workgroup per CU: at four, the 384 workgroups - one resident per
// CU at their register count - ran in two rounds (32 rows: 17.4 -> 13.0 us per launch, the LM head 78 -> 74 us).
static hipError_t launch_gemm_narrow(int fmt, OxbGemmParams p, uint32_t n_cus, hipStream_t st) {
    p.ksplit = 1;
    p.sb_per_split = p.n_sb;
    const bool sw = p.mode == OXB_GEMM_SWIGLU;
    if (sw && (p.n_rows & 31u) != 0) return hipErrorInvalidValue;  // gate and up halves of whole row tiles
    const uint32_t ct = p.M_pad / 16;
    uint32_t rt = sw ? 2 : 1;
    uint64_t best_cost = ~0ull;
    static const uint32_t choices[4] = {1, 2, 4, 6};
    for (uint32_t ci = sw ? 1 : 0; ci < (fmt == OXB_FMT_Q1 ? 4u : 3u); ci++) {  // (six tiles: Q1 only - the ternary decoder's registers do not fit)
        const uint32_t r = choices[ci];
        const uint32_t wgs = sw ? (p.n_tiles / 2 + r / 2 - 1) / (r / 2) : (p.n_tiles + r - 1) / r;
        const uint64_t cost = (uint64_t)((wgs + n_cus - 1) / n_cus) * (r + 2);
        if (cost <= best_cost) best_cost = cost, rt = r;
    }
#define OXB_NARROW_CASE(F, R, C) \
    if (fmt == F && rt == R && ct == C) return launch_narrow_case<F, R, C>(p, st);
    OXB_NARROW_CASE(OXB_FMT_Q1, 1, 1) OXB_NARROW_CASE(OXB_FMT_Q1, 2, 1) OXB_NARROW_CASE(OXB_FMT_Q1, 4, 1)
    OXB_NARROW_CASE(OXB_FMT_Q1, 1, 2) OXB_NARROW_CASE(OXB_FMT_Q1, 2, 2) OXB_NARROW_CASE(OXB_FMT_Q1, 4, 2)
    OXB_NARROW_CASE(OXB_FMT_Q1, 6, 1) OXB_NARROW_CASE(OXB_FMT_Q1, 6, 2)
    OXB_NARROW_CASE(OXB_FMT_TQ2, 1, 1) OXB_NARROW_CASE(OXB_FMT_TQ2, 2, 1) OXB_NARROW_CASE(OXB_FMT_TQ2, 4, 1)
    OXB_NARROW_CASE(OXB_FMT_TQ2, 1, 2) OXB_NARROW_CASE(OXB_FMT_TQ2, 2, 2) OXB_NARROW_CASE(OXB_FMT_TQ2, 4, 2)
#undef OXB_NARROW_CASE
    return hipErrorInvalidValue;
}


uint32_t oxb_gemm_ksplit(const OxbGemmParams& p, uint32_t n_cus) {
    if (p.M == 0 || p.n_rows == 0 || p.n_sb == 0 || p.M <= OXB_GEMM_NARROW_MAX_M) return 1;
    return plan_gemm(p, n_cus).ksplit;
}

hipError_t oxb_launch_gemm(int fmt, OxbGemmParams p, uint32_t n_cus, hipStream_t st) {
    if (p.M == 0 || p.n_rows == 0) return hipSuccess;
    if (p.n_sb == 0 || (uint64_t)p.n_tiles * p.n_sb * 2048ull >= 0xFFFFFFF0ull) return hipErrorInvalidValue;
    p.M_pad = (p.M + 15u) / 16u * 16u;
    if (p.M <= OXB_GEMM_NARROW_MAX_M) return launch_gemm_narrow(fmt, p, n_cus, st);
    if (p.mode == OXB_GEMM_SWIGLU && (p.n_rows & 31u) != 0) return hipErrorInvalidValue;  // whole gate and up row tiles
    const GemmPlan plan = plan_gemm(p, n_cus);
    const uint32_t BM = 16 * plan.ct;  // tokens per workgroup tile
    p.n_mt = (p.M + BM - 1) / BM;
    const uint32_t best_rt = plan.rt, best_tpw = plan.tpw;
    p.ksplit = plan.ksplit;
    p.sb_per_split = plan.sb_per_split;
    if (p.ksplit > 1 && !p.part) return hipErrorInvalidValue;
    p.tpw = best_tpw;
    p.n_ng = (p.n_tiles + p.tpw - 1) / p.tpw;
    const uint32_t grid = p.n_ng * p.n_mt * p.ksplit;
    hipError_t err = hipErrorInvalidValue;
#define OXB_GEMM_CASE(F, R) \
    if (fmt == F && best_rt == R && plan.ct == 8) err = launch_gemm_case<F, R, 8>(p, grid, st);
    OXB_GEMM_CASE(OXB_FMT_Q1, 1)
    OXB_GEMM_CASE(OXB_FMT_Q1, 2)
    OXB_GEMM_CASE(OXB_FMT_Q1, 3)
    OXB_GEMM_CASE(OXB_FMT_Q1, 4)
    OXB_GEMM_CASE(OXB_FMT_Q1, 5)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 1)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 2)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 3)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 4)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 5)
#undef OXB_GEMM_CASE
    if (plan.ct == 4 && best_rt == 1) err = fmt == OXB_FMT_Q1 ? launch_gemm_case<OXB_FMT_Q1, 1, 4>(p, grid, st) : launch_gemm_case<OXB_FMT_TQ2, 1, 4>(p, grid, st);
    if (err != hipSuccess || p.ksplit == 1) return err;
    const size_t plane = (size_t)p.M * p.ldy, n4 = plane / 4;
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((uint32_t)((n4 + 255) / 256)), dim3(256), 0, st, p.part, p.ksplit, plane,
                       p.mode == OXB_GEMM_RESIDUAL ? p.residual : nullptr, p.y, n4);
    return hipGetLastError();
}
