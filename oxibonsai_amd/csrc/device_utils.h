// device_utils.h — small device-side helpers shared by the kernels: DPP lane moves, buffer-resource
// loads with hardware bounds checking, and a barrier that leaves global loads in flight.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// DPP moves: lanes that would read outside their 16-lane row get 0.
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// Reductions over the 64 lanes of a wave, result in every lane, without a trip through the LDS pipeline: four DPP
// steps inside every 16-lane row (quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror, row_mirror), then the four rows as
// (r0 + r1) + (r2 + r3): v_permlane16_swap exchanges the odd rows of its first operand with the even rows of its
// second, v_permlane32_swap the upper half of the first with the lower half of the second; on two copies of one value
// each leaves the two addends of a pair side by side.
__device__ __forceinline__ float sum_rows4(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
__device__ __forceinline__ float max_rows4(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float wave_sum_f32(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    return sum_rows4(v);
}
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    return max_rows4(v);
}
#define OXB_DPP_ROW_SHR(n) (0x110 + (n))
#define OXB_DPP_ROW_NEWBCAST(n) (0x150 + (n))  // lane n of each 16-lane row to the whole row

// Buffer resources: a load whose byte offset lies outside the buffer returns 0 and moves no
// data, which replaces every "is this tile / superblock / column in range" branch below.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
#define OXB_OOB 0xFFFFFFF0u
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
// voff is per lane and is what the range check sees; soff is wave-uniform (an SGPR) and is not checked.
__device__ __forceinline__ v4i buf_load_b128(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff = 0) {
    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
    return (v4i){(int)v.x, (int)v.y, (int)v.z, (int)v.w};
}
__device__ __forceinline__ uint32_t buf_load_b32(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff = 0) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0);
}
// Workgroup barrier that orders LDS traffic only: global loads already in flight (the
// prefetched weight tiles) stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ds_read_b64_tr_b16, the transposing LDS read of gfx950: each lane gives the address of four consecutive halves;
// within every block of 16 lanes these are the rows of a 4 x 16 tile (lane i: row i / 4, columns 4 (i % 4) .. + 3),
// and lane j receives column j of the tile (rows 0 .. 3).  It turns a row-major [key][d] block into the matrix cores'
// operand layout (k = key contiguous per lane) without 2-byte gathers.
typedef _Float16 v4h_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ v4h_t lds_read_tr16(const _Float16* q) {
    typedef short v4s_t __attribute__((ext_vector_type(4)));
    return __builtin_bit_cast(v4h_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s_t*)q));
}


// Agent-coherent accesses (the sc1 cache-policy bit): the store is written through to memory, the load is served from
// memory and not from this CU's L1 or this XCD's L2.  Data that other workgroups of the same launch produce and
// consume goes through these, with a counter in between, instead of through whole-cache write-backs and invalidates.
#define OXB_AUX_SC1 16
__device__ __forceinline__ void buf_store_b32_coherent(__amdgpu_buffer_rsrc_t r, uint32_t voff, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, (int)voff, 0, OXB_AUX_SC1);
}
__device__ __forceinline__ v4f buf_load_f128_coherent(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, 0, OXB_AUX_SC1);
    return (v4f){__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
}
__device__ __forceinline__ float buf_load_f32_coherent(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, 0, OXB_AUX_SC1));
}
