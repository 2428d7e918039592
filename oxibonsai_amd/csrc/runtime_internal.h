// runtime_internal.h — state shared by the translation units of the library.
#pragma once
#include <hip/hip_runtime.h>

#include <exception>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>

#include "layout.h"

namespace oxb {

struct DevBuf {  // grow-only device scratch
    void* ptr = nullptr;
    size_t cap = 0;
    bool fixed = false;  // a view of memory owned elsewhere: never grown, never freed
    int ensure(size_t bytes);
    void release();
};

// Scratch of one GEMM call: packed fp16 activations, per-row exponents and multipliers, and the partial sums of
// the K slices when K is split over workgroups.  A sequence of calls captured into a graph needs buffers of its
// own that never move.
struct GemmWorkspace {
    DevBuf xh, xsh, rowmul, part;
    void release() { xh.release(); xsh.release(); rowmul.release(); part.release(); }
};

// One resident matrix: [codes section][scales section].  A weight uploaded as bytes alone (the reference's
// upload_weights_raw / upload_weights_ternary carry no shape) waits as a device copy of those bytes, d_raw, with
// L.n_rows == 0, until the first call that names (n_rows, k) binds the shape and repacks it on the device.
struct Weight {
    OxbLayout L;
    void* d_base = nullptr;
    uint32_t* d_codes = nullptr;
    uint16_t* d_scales = nullptr;
    void* d_raw = nullptr;
    size_t raw_blocks = 0;
};

struct Vector {  // a resident fp32 vector (norm weights)
    float* d = nullptr;
    size_t n = 0;
    float absmax = 0.f;  // max |value|, the RMSNorm kernel's bound for its output range
};

struct Runtime {
    bool ready = false;
    int device = -1;
    uint32_t n_cus = 0;
    char name[256] = {0};
    hipStream_t own_stream = nullptr, stream = nullptr;
    std::unordered_map<uint64_t, Weight> weights;
    std::unordered_map<uint64_t, Vector> vectors;
    uint64_t next_id = 1ull << 40;  // library-allocated handles stay clear of caller-chosen ids
    // Counts every free or replacement of a resident matrix or vector.  A captured decode graph holds their device
    // pointers; a model compares the count it captured under with this one and captures again when they differ.
    uint64_t weights_gen = 0;
    DevBuf ws_x, ws_y, ws_aux;
    DevBuf gemv_pack;  // quantised activation vectors of one GEMV call (gemv_launch with pack_ws)
    void* static_scratch = nullptr;  // device address of the library's file-scope scratch array on g_rt.device
    GemmWorkspace gemm_ws;  // shared by every GEMM call that does not bring its own
};

extern Runtime g_rt;
extern std::recursive_mutex g_mu;

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char* what);
int ensure_init();
Weight* find_weight(uint64_t id);
int upload_weight(uint64_t* id, int fmt, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k);
// Holds the weight to (n_rows, k): binds and repacks one that has no shape yet (never inside a stream capture), else
// compares.
int bind_shape(Weight& w, uint32_t n_rows, uint32_t k);
int gemv_device(const Weight& w, const float* d_x, float* d_y, uint32_t batch, uint32_t ldy, int mode,
                const float* d_residual);
// nvec <= OXB_GEMV_MAX_BATCH vectors x [nvec][ldx] through one pass over the weights: pro / epi are OXB_GEMV_PRO_* /
// OXB_GEMV_* (RMSNorm with d_norm_w and eps in front; store, residual add or SwiGLU behind).
// With pack_ws the vectors (up to OXB_GEMV_PACKED_MAX_BATCH) are quantised by a launch of their own into that buffer
// (grown on demand: never inside a stream capture) and the GEMV loads its operands from there; with `prepacked` the
// buffer already holds them (left there by the kernel that produced the vectors) and no pack launch is made.
int gemv_launch(const Weight& w, const float* d_x, uint32_t ldx, uint32_t nvec, float* d_y, uint32_t ldy, int pro,
                const float* d_norm_w, float eps, int epi, const float* d_residual, DevBuf* pack_ws = nullptr, bool prepacked = false);
uint32_t gemv_packed_min_batch(uint32_t k);
// x (device, [m][ldx]) -> y (device, [m][ldy]) through the fp16 packer + MFMA GEMM.  pack_op (OXB_PACK_*) names the
// row-wise producer fused into the packer: RMSNorm with weights d_pack_w and eps, or SwiGLU of x = [gate | up].
// ws = nullptr uses (and may grow) the runtime's shared workspace.
int gemm_device(const Weight& w, const float* d_x, uint32_t ldx, float* d_y, uint32_t m, uint32_t ldy, int mode,
                const float* d_residual, int pack_op, const float* d_pack_w, float eps, GemmWorkspace* ws = nullptr);
void shutdown_models();

// Every `int` entry point of the C ABI runs its body between these two, so that no C++ exception (a failed host
// allocation in a std container, above all) unwinds into the caller.
#define OXB_API_BEGIN try {
#define OXB_API_END                                                                                          \
    }                                                                                                        \
    catch (const std::bad_alloc&) { return oxb::fail(OXB_HIP_OUT_OF_MEMORY, "out of host memory"); }        \
    catch (const std::exception& e_) { return oxb::fail(OXB_HIP_INVALID_ARGUMENT, "internal error: %s", e_.what()); } \
    catch (...) { return oxb::fail(OXB_HIP_INVALID_ARGUMENT, "internal error: unknown C++ exception"); }

}  // namespace oxb
