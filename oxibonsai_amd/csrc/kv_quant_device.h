// kv_quant_device.h — quantised KV-cache rows on the device: one row = the head_dim values of one position of one
// kv head, stored as head_dim one-byte codes plus one f32 scale.
//
//   OXB_KV_I8        code = round(x / scale) clamped to +-127 (half away from zero), scale = max(max|x| / 127, eps)
//                    (quantize_row_i8, crates/oxibonsai-model/src/kv_cache_quant.rs:46-62)
//   OXB_KV_FP8_E4M3  code = E4M3FN(x / scale), round to nearest even, saturating at +-448, scale = max(max|x| / 448, eps)
//                    (quantize_row_fp8, kv_cache_quant.rs:519-540; fp8_e4m3_encode, crates/oxibonsai-core/src/quant_fp8.rs:47-160)
// Reading back is code * scale (kv_cache_quant.rs:69-71, 545-556).  The attention kernels never form that product
// per element: the codes go to the matrix cores as exact fp16 numbers and the row scale multiplies the score (K)
// or the probability (V).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define OXB_KV_F16 0
#define OXB_KV_I8 1
#define OXB_KV_FP8_E4M3 2

// Where the rows of a KV cache lie.  Contiguous: [sequence][layer][kv_head][row_stride] rows (row_stride = the context
// rounded up to a whole number of 128-position attention chunks).  Paged (PagedKvCache / BlockTable,
// crates/oxibonsai-model/src/paged_kv_cache.rs:187-236, 294-345): a pool of n_pages pages of 2^page_shift positions
// each, [layer][kv_head][page][position in page] rows - the pages of one (layer, head) lie side by side, so a walk
// over a sequence stays inside n_pages * page bytes of address space, as it does in the contiguous cache - and per
// sequence a table of physical page numbers indexed by position >> page_shift.  A row index addresses both the data
// (row * head_dim elements) and the row scales.
struct OxbKvLayout {
    const uint32_t* page_table;  // null: contiguous
    uint32_t page_shift, table_stride, n_pages;
    uint32_t n_layers, nkv, row_stride;
};
#if defined(__HIPCC__)
__device__ __forceinline__ size_t kv_row(const OxbKvLayout& L, uint32_t seq, uint32_t layer, uint32_t kvh, uint32_t pos) {
    if (L.page_table) {
        const uint32_t page = L.page_table[(size_t)seq * L.table_stride + (pos >> L.page_shift)];
        return ((((size_t)layer * L.nkv + kvh) * L.n_pages + page) << L.page_shift) + (pos & ((1u << L.page_shift) - 1u));
    }
    return (((size_t)seq * L.n_layers + layer) * L.nkv + kvh) * L.row_stride + pos;
}
#endif

typedef _Float16 kvh2_t __attribute__((ext_vector_type(2)));
typedef _Float16 kvh8_t __attribute__((ext_vector_type(8)));
typedef int kvi2_t __attribute__((ext_vector_type(2)));

template <int KVM>
__device__ __forceinline__ float kv_row_scale(float max_abs) {
    const float s = max_abs / (KVM == OXB_KV_I8 ? 127.0f : 448.0f);
    return s >= 1.1920929e-07f ? s : 1.1920929e-07f;  // f32::EPSILON
}

// E4M3FN code of t: s eeee mmm, bias 7, no infinity, NaN = 0x7f.
__device__ __forceinline__ uint32_t kv_e4m3_encode(float t) {
    const uint32_t bits = __float_as_uint(t), sign = (bits >> 24) & 0x80u, mag = bits & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return 0x7fu;
    if (mag >= 0x43E00000u) return sign | 0x7eu;  // |t| >= 448 (and infinity) saturates
    const int e = (int)(mag >> 23) - 120;         // biased exponent in the target format
    uint32_t code;
    if (e >= 1) {
        const uint32_t man = mag & 0x7FFFFFu, rem = man & 0xFFFFFu;
        code = ((uint32_t)e << 3) | (man >> 20);
        code += (rem > 0x80000u || (rem == 0x80000u && (code & 1u))) ? 1u : 0u;  // ties to even; a carry runs into the exponent
    } else {
        code = (uint32_t)__builtin_rintf(__uint_as_float(mag) * 512.0f);  // multiples of 2^-9; 8 = the smallest normal value
    }
    return sign | code;
}

template <int KVM>
__device__ __forceinline__ uint32_t kv_encode(float x, float scale) {
    const float t = x / scale;
    if (KVM == OXB_KV_I8) {
        float r = roundf(t);
        r = r < -127.0f ? -127.0f : (r > 127.0f ? 127.0f : r);
        return (uint32_t)(int)r & 0xFFu;
    }
    return kv_e4m3_encode(t);
}

// Four codes (one dword, lowest byte first) -> four exact fp16 values in two dwords.
template <int KVM>
__device__ __forceinline__ void kv_dec4(uint32_t w, uint32_t& lo, uint32_t& hi) {
    if (KVM == OXB_KV_I8) {
        // byte b -> the fp16 number 0x6400 | (b ^ 0x80) = 1024 + 128 + b; subtracting 1152 is exact
        const uint32_t x = w ^ 0x80808080u;
        const kvh2_t off = {(_Float16)1152.0f, (_Float16)1152.0f};
        const kvh2_t a = __builtin_bit_cast(kvh2_t, __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u)) - off;
        const kvh2_t b = __builtin_bit_cast(kvh2_t, __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u)) - off;
        lo = __builtin_bit_cast(uint32_t, a);
        hi = __builtin_bit_cast(uint32_t, b);
    } else {
        // the conversion instruction of gfx950 (OCP E4M3: the format of fp8_e4m3_encode) widens two codes at a time,
        // exactly: every E4M3 value, subnormal codes included, is an fp16 number
        lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));  // bytes 0, 1
        hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));   // bytes 2, 3
    }
}

// Eight codes -> one MFMA operand of eight fp16 values (element e = byte e).
template <int KVM>
__device__ __forceinline__ kvh8_t kv_dec8(kvi2_t raw) {
    uint32_t d[4];
    kv_dec4<KVM>((uint32_t)raw.x, d[0], d[1]);
    kv_dec4<KVM>((uint32_t)raw.y, d[2], d[3]);
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    return __builtin_bit_cast(kvh8_t, (u4){d[0], d[1], d[2], d[3]});
}
