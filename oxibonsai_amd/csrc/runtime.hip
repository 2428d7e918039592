// runtime.hip — the C ABI of the native-hip tier: device/stream ownership, the
// weight handle table, workspaces, validation and error reporting.
//
// Host-side counterpart of the reference's CudaGraph singleton and
// NativeCudaBackend (crates/oxibonsai-kernels/src/gpu_backend/cuda_graph/
// cudagraph_type.rs:18-32, nativecudabackend_traits.rs:29-188): one device, one
// stream, a process-wide map u64 -> resident weight, every call under a mutex.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/oxb_hip.h"
#include "../../include/oxb_hip_measure.h"
#include "gemm_kernels.h"
#include "gemv_kernels.h"
#include "layout.h"
#include "repack.h"
#include "runtime_internal.h"

namespace oxb {

thread_local std::string t_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    t_last_error = buf;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    int code = (e == hipErrorOutOfMemory) ? OXB_HIP_OUT_OF_MEMORY : OXB_HIP_KERNEL_LAUNCH;
    return fail(code, "%s: %s", what, hipGetErrorString(e));
}

Runtime g_rt;
std::recursive_mutex g_mu;

// Scratch of the allocation-free GEMM entry point (oxb_hip_gemm_dev_static): packed fp16 activations, per-row
// exponents and multipliers, and the partial sums of a K split.  It lives in the code object, so the GPU the library
// runs on holds it from the first use of the library until the process ends.  In host code the array's name only
// stands for the symbol; its device address is looked up once in oxb_hip_init and kept in g_rt.static_scratch.
#define OXB_STATIC_SCRATCH_BYTES (32u << 20)
static __device__ __align__(256) unsigned char oxb_static_scratch[OXB_STATIC_SCRATCH_BYTES];

int DevBuf::ensure(size_t bytes) {
    if (bytes <= cap) return OXB_HIP_OK;
    if (fixed) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %zu bytes of scratch needed, the fixed buffer holds %zu", bytes, cap);
    // Growing means hipFree + hipMalloc, which a stream capture in progress cannot take: every buffer a captured
    // sequence uses is sized before the capture begins, so this is a bug if it ever triggers - fail, do not allocate.
    hipStreamCaptureStatus cap_status = hipStreamCaptureStatusNone;
    if (g_rt.stream && hipStreamIsCapturing(g_rt.stream, &cap_status) == hipSuccess && cap_status != hipStreamCaptureStatusNone)
        return fail(OXB_HIP_KERNEL_LAUNCH, "internal error: a workspace of %zu bytes would have to grow to %zu inside a stream capture", cap, bytes);
    if (ptr) (void)hipFree(ptr);
    ptr = nullptr;
    cap = 0;
    size_t want = bytes + (bytes >> 2);
    want = (want + 255) & ~(size_t)255;
    hipError_t e = hipMalloc(&ptr, want);
    if (e != hipSuccess) {
        ptr = nullptr;
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", want, g_rt.device);
    }
    cap = want;
    return OXB_HIP_OK;
}

void DevBuf::release() {
    if (ptr && !fixed) (void)hipFree(ptr);
    ptr = nullptr;
    cap = 0;
}

int ensure_init() {
    if (g_rt.ready) return OXB_HIP_OK;
    return oxb_hip_init(g_rt.device < 0 ? 0 : g_rt.device);
}

Weight* find_weight(uint64_t id) {
    auto it = g_rt.weights.find(id);
    return it == g_rt.weights.end() ? nullptr : &it->second;
}

static void free_weight_mem(Weight& w) {
    if (w.d_base) (void)hipFree(w.d_base);
    if (w.d_raw) (void)hipFree(w.d_raw);
    w.d_base = nullptr;
    w.d_raw = nullptr;
}

// Block bytes -> a device copy, shape still open.  Nothing in the handle table changes here.
static int make_weight_bytes(int fmt, const uint8_t* aos, size_t n_bytes, Weight* out) {
    const size_t bb = fmt == OXB_FMT_Q1 ? OXB_Q1_AOS_BYTES : OXB_TQ2_AOS_BYTES;
    if (!aos || n_bytes == 0 || n_bytes % bb != 0)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight buffer of %zu bytes is not a whole number of %zu-byte blocks",
                    n_bytes, bb);
    int rc = ensure_init();
    if (rc) return rc;
    Weight w;
    w.L = oxb_make_layout((uint32_t)fmt, 0, 0);
    w.raw_blocks = n_bytes / bb;
    hipError_t e = hipMalloc(&w.d_raw, n_bytes);
    if (e != hipSuccess)
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", n_bytes, g_rt.device);
    e = hipMemcpy(w.d_raw, aos, n_bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(w.d_raw);
        return hip_fail(e, "weight upload");
    }
    *out = w;
    return OXB_HIP_OK;
}

// A finished weight takes its place in the handle table; the one it replaces (a caller-chosen id may name one) is
// freed only now, when the new copy is complete, so a failed upload leaves the old weight in use.
static void store_weight(uint64_t* id, const Weight& w) {
    if (*id == 0) *id = g_rt.next_id++;
    if (Weight* old = find_weight(*id)) {
        (void)hipStreamSynchronize(g_rt.stream);  // a launch in flight may still read the old copy
        free_weight_mem(*old);
        g_rt.weights_gen++;
    }
    g_rt.weights[*id] = w;
}

static int upload_weight_bytes(uint64_t* id, int fmt, const uint8_t* aos, size_t n_bytes) {
    if (!id) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: id pointer is null");
    Weight w;
    int rc = make_weight_bytes(fmt, aos, n_bytes, &w);
    if (rc) return rc;
    store_weight(id, w);
    return OXB_HIP_OK;
}

int bind_shape(Weight& w, uint32_t n_rows, uint32_t k) {
    if (k == 0 || k % OXB_QK != 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: k=%u is not a multiple of 128", k);
    if (!w.d_raw) {
        if (w.L.n_rows != n_rows || w.L.k != k)
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight is %ux%u, call asks for %ux%u", w.L.n_rows,
                        w.L.k, n_rows, k);
        return OXB_HIP_OK;
    }
    const size_t need = (size_t)n_rows * (k / OXB_QK);
    if (n_rows == 0 || need != w.raw_blocks)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight holds %zu blocks, %ux%u needs %zu", w.raw_blocks,
                    n_rows, k, need);
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(g_rt.stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
        return fail(OXB_HIP_INVALID_ARGUMENT,
                    "invalid argument: a weight uploaded without a shape cannot be bound inside a stream capture; call once before capturing");
    const OxbLayout L = oxb_make_layout(w.L.fmt, n_rows, k);
    const size_t total = L.codes_bytes + L.scales_bytes;
    void* base = nullptr;
    hipError_t e = hipMalloc(&base, total);
    if (e != hipSuccess)
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", total, g_rt.device);
    uint32_t* codes = reinterpret_cast<uint32_t*>(base);
    uint16_t* scales = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(base) + L.codes_bytes);
    e = oxb_launch_repack(L, reinterpret_cast<const uint8_t*>(w.d_raw), codes, scales, g_rt.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_rt.stream);
    if (e != hipSuccess) {
        (void)hipFree(base);
        return hip_fail(e, "kernel launch failed: repack");
    }
    (void)hipFree(w.d_raw);
    w.d_raw = nullptr;
    w.L = L;
    w.d_base = base;
    w.d_codes = codes;
    w.d_scales = scales;
    return OXB_HIP_OK;
}

int upload_weight(uint64_t* id, int fmt, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k) {
    if (!id) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: id pointer is null");
    if (k == 0 || k % OXB_QK != 0)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: k=%u is not a multiple of 128", k);
    if (n_rows == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: n_rows is 0");
    const size_t bb = fmt == OXB_FMT_Q1 ? OXB_Q1_AOS_BYTES : OXB_TQ2_AOS_BYTES;
    const size_t need = (size_t)n_rows * (k / OXB_QK) * bb;
    if (!aos || n_bytes < need)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight buffer holds %zu bytes, %zu needed", n_bytes, need);
    Weight w;  // raw copy, then the repack; the handle table is touched only when both have succeeded
    int rc = make_weight_bytes(fmt, aos, need, &w);
    if (rc) return rc;
    rc = bind_shape(w, n_rows, k);
    if (rc) {
        free_weight_mem(w);
        return rc;
    }
    store_weight(id, w);
    return OXB_HIP_OK;
}

// One GEMV over resident weights, any K: launches of at most OXB_GEMV_MAX_SB superblocks, the first with the wanted
// epilogue, the rest accumulating.  nvec <= OXB_GEMV_MAX_BATCH vectors share each pass over the weights.
int gemv_launch(const Weight& w, const float* d_x, uint32_t ldx, uint32_t nvec, float* d_y, uint32_t ldy, int pro,
                const float* d_norm_w, float eps, int epi, const float* d_residual, DevBuf* pack_ws, bool prepacked) {
    OxbGemvParams p;
    memset(&p, 0, sizeof p);
    if (pack_ws) {  // quantise the vectors once, in a launch of its own; the GEMV then loads its operands
        const size_t need = oxb_gemv_pack_bytes(w.L.k, nvec);
        if (prepacked) {  // (the kernel that produced the vectors has left them quantised in pack_ws)
            if (pro != OXB_GEMV_PRO_F32) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: operands packed ahead carry no RMSNorm");
            if (pack_ws->cap < need) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: packed operands of %zu bytes, %zu needed", pack_ws->cap, need);
        } else {
            int rc = pack_ws->ensure(need);
            if (rc) return rc;
            hipError_t e = oxb_launch_gemv_pack((int)w.L.fmt, pro, d_x, ldx, nvec, w.L.k, d_norm_w, (uint32_t*)pack_ws->ptr, g_rt.stream);
            if (e != hipSuccess) return hip_fail(e, "kernel launch failed: gemv_pack");
        }
        p.xq = (const uint32_t*)pack_ws->ptr;
        p.xq_bytes = (uint32_t)need;
        p.nvg = (nvec + 3) / 4;
    }
    p.codes = w.d_codes;
    p.scales = w.d_scales;
    p.x = d_x;
    p.norm_w = d_norm_w;
    p.eps = eps;
    p.y = d_y;
    p.residual = d_residual;
    p.n_rows = w.L.n_rows;
    p.n_tiles = w.L.n_tiles;
    p.n_sb = w.L.n_sb;
    p.k = w.L.k;
    p.nvec = nvec;
    p.ldx = ldx;
    p.ldy = ldy;
    p.codes_bytes = (uint32_t)w.L.codes_bytes;
    p.scales_bytes = (uint32_t)w.L.scales_bytes;
    p.pro = pro;
    for (uint32_t sb = 0; sb < w.L.n_sb; sb += OXB_GEMV_MAX_SB) {
        p.sb_begin = sb;
        p.sb_count = (w.L.n_sb - sb) < OXB_GEMV_MAX_SB ? (w.L.n_sb - sb) : OXB_GEMV_MAX_SB;
        p.epi = sb == 0 ? epi : OXB_GEMV_ACCUM;
        hipError_t e = oxb_launch_gemv((int)w.L.fmt, p, g_rt.n_cus, g_rt.stream);
        if (e != hipSuccess) return hip_fail(e, "kernel launch failed: gemv");
    }
    return OXB_HIP_OK;
}

// Vectors from which a GEMV quantises its activations in a launch of its own (then up to eight share one pass over
// the weights) instead of in every workgroup's prologue (four per pass).
// 1 = by shape (the default), 0 = never, n >= 2 = from n vectors on.  By shape: five vectors and more always; two to
// four where a wave's K slice is longer than one superblock (K above 4096), because there the prologue that every
// workgroup repeats costs more than the extra launch (measured at K = 6144 and 12288 against 2048 and 4096).
static uint32_t g_packed_min_batch = 1;
uint32_t gemv_packed_min_batch(uint32_t k) {
    if (g_packed_min_batch == 0) return 0xFFFFFFFFu;
    if (g_packed_min_batch >= 2) return g_packed_min_batch;
    return k > 4096 ? 2u : 5u;
}

// x (device, [batch][k]) -> y (device, [batch][ldy]): up to eight vectors per pass over the weights (four, and the
// quantisation in the kernel itself, for what is left below gemv_packed_min_batch(k)).
int gemv_device(const Weight& w, const float* d_x, float* d_y, uint32_t batch, uint32_t ldy, int mode,
                const float* d_residual) {
    const uint32_t k = w.L.k;
    for (uint32_t b0 = 0; b0 < batch;) {
        const uint32_t left = batch - b0;
        const bool packed = left >= gemv_packed_min_batch(k);
        const uint32_t cap = packed ? OXB_GEMV_PACKED_MAX_BATCH : OXB_GEMV_MAX_BATCH, nb = left < cap ? left : cap;
        int rc = gemv_launch(w, d_x + (size_t)b0 * k, k, nb, d_y + (size_t)b0 * ldy, ldy, OXB_GEMV_PRO_F32, nullptr, 0.f, mode,
                             d_residual ? d_residual + (size_t)b0 * ldy : nullptr, packed ? &g_rt.gemv_pack : nullptr);
        if (rc) return rc;
        b0 += nb;
    }
    return OXB_HIP_OK;
}

int gemm_device(const Weight& w, const float* d_x, uint32_t ldx, float* d_y, uint32_t m, uint32_t ldy, int mode,
                const float* d_residual, int pack_op, const float* d_pack_w, float eps, GemmWorkspace* ws) {
    if (!ws) ws = &g_rt.gemm_ws;
    const uint32_t k = w.L.k;
    if ((uint64_t)m * k >= (1ull << 31))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %u rows of %u activations exceed one GEMM call", m, k);
    int rc;
    if ((rc = ws->xh.ensure(oxb_xh_bytes(k, m)))) return rc;
    if ((rc = ws->xsh.ensure(((size_t)m + 16) * sizeof(int32_t)))) return rc;
    if ((rc = ws->rowmul.ensure(((size_t)m + 16) * sizeof(float)))) return rc;
    hipError_t e = oxb_launch_xh_pack((int)w.L.fmt, pack_op, d_x, d_pack_w, ldx, k, eps, m, (float*)ws->rowmul.ptr,
                                      (uint32_t*)ws->xh.ptr, (int32_t*)ws->xsh.ptr, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "kernel launch failed: xh_pack");
    OxbGemmParams p;
    memset(&p, 0, sizeof p);
    p.codes = w.d_codes;
    p.scales = w.d_scales;
    p.xh = (const uint32_t*)ws->xh.ptr;
    p.xsh = (const int32_t*)ws->xsh.ptr;
    p.y = d_y;
    p.residual = d_residual;
    p.n_rows = w.L.n_rows;
    p.n_tiles = w.L.n_tiles;
    p.n_sb = w.L.n_sb;
    p.M = m;
    p.ldy = ldy;
    p.codes_bytes = (uint32_t)w.L.codes_bytes;
    p.scales_bytes = (uint32_t)w.L.scales_bytes;
    p.xh_bytes = (uint32_t)oxb_xh_bytes(k, m);
    p.mode = mode;
    const uint32_t ksplit = oxb_gemm_ksplit(p, g_rt.n_cus);
    if (ksplit > 1) {
        if ((rc = ws->part.ensure((size_t)ksplit * m * ldy * sizeof(float)))) return rc;
        p.part = (float*)ws->part.ptr;
    }
    e = oxb_launch_gemm((int)w.L.fmt, p, g_rt.n_cus, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "kernel launch failed: gemm");
    return OXB_HIP_OK;
}

static int sync_stream(const char* what) {
    hipError_t e = hipStreamSynchronize(g_rt.stream);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: %s: %s", what, hipGetErrorString(e));
    return OXB_HIP_OK;
}

static int oneshot_gemv(int fmt, const uint8_t* aos, size_t n_bytes, const float* x, size_t x_len, float* y,
                        size_t y_len, uint32_t n_rows, uint32_t k) {
    // Validation order of the scalar kernels (gemv.rs:32-58 / gemv_ternary.rs:55-81).
    if (k % OXB_QK != 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: k=%u is not a multiple of 128", k);
    if (x_len < k) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: input holds %zu values, %u needed", x_len, k);
    if (y_len < n_rows) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: output holds %zu values, %u needed", y_len, n_rows);
    if (n_rows == 0) return OXB_HIP_OK;
    uint64_t id = 0;
    int rc = upload_weight(&id, fmt, aos, n_bytes, n_rows, k);
    if (rc) return rc;
    rc = oxb_hip_gemv(id, x, y, n_rows, k, 1);
    int rc2 = oxb_hip_free_weight(id);
    return rc ? rc : rc2;
}

}  // namespace oxb

using namespace oxb;

extern "C" {

const char* oxb_hip_last_error(void) { return t_last_error.c_str(); }

int oxb_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int oxb_hip_init(int device_ordinal) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (g_rt.ready) {
        if (device_ordinal != g_rt.device)
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: already initialised on device %d", g_rt.device);
        return OXB_HIP_OK;
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) return fail(OXB_HIP_NOT_AVAILABLE, "GPU not available: no HIP device");
    if (device_ordinal < 0 || device_ordinal >= n)
        return fail(OXB_HIP_NOT_AVAILABLE, "GPU not available: device %d of %d", device_ordinal, n);
    if ((e = hipSetDevice(device_ordinal)) != hipSuccess) return fail(OXB_HIP_NOT_AVAILABLE, "GPU not available: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    if ((e = hipGetDeviceProperties(&prop, device_ordinal)) != hipSuccess)
        return fail(OXB_HIP_NOT_AVAILABLE, "GPU not available: %s", hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(OXB_HIP_NOT_AVAILABLE, "GPU not available: kernels are built for gfx950, device is %s", prop.gcnArchName);
    void* scratch_addr = nullptr;
    if ((e = hipGetSymbolAddress(&scratch_addr, HIP_SYMBOL(oxb_static_scratch))) != hipSuccess || !scratch_addr)
        return hip_fail(e, "static scratch lookup");
    g_rt.static_scratch = scratch_addr;
    if ((e = hipStreamCreateWithFlags(&g_rt.own_stream, hipStreamNonBlocking)) != hipSuccess)
        return hip_fail(e, "stream creation");
    g_rt.stream = g_rt.own_stream;
    g_rt.device = device_ordinal;
    g_rt.n_cus = (uint32_t)prop.multiProcessorCount;
    snprintf(g_rt.name, sizeof g_rt.name, "%s (%s)", prop.name, prop.gcnArchName);
    // The pack buffer of the batched GEMV exists from the start (eight vectors of K = 32768 fit: 1.1 MB), so that a
    // caller who captures oxb_hip_gemv_dev into a graph of its own needs no warm-up call for it to grow.
    const int rc_pack = g_rt.gemv_pack.ensure(oxb_gemv_pack_bytes(32768, OXB_GEMV_PACKED_MAX_BATCH));
    if (rc_pack) {
        (void)hipStreamDestroy(g_rt.own_stream);
        g_rt.own_stream = g_rt.stream = nullptr;
        return rc_pack;
    }
    g_rt.ready = true;
    return OXB_HIP_OK;
    OXB_API_END
}

void oxb_hip_shutdown(void) {
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!g_rt.ready) return;
    (void)hipStreamSynchronize(g_rt.stream);
    shutdown_models();
    for (auto& kv : g_rt.weights) free_weight_mem(kv.second);
    g_rt.weights.clear();
    for (auto& kv : g_rt.vectors) (void)hipFree(kv.second.d);
    g_rt.vectors.clear();
    g_rt.ws_x.release();
    g_rt.ws_y.release();
    g_rt.ws_aux.release();
    g_rt.gemv_pack.release();
    g_rt.gemm_ws.release();
    (void)hipStreamDestroy(g_rt.own_stream);
    g_rt.static_scratch = nullptr;
    g_rt.own_stream = nullptr;
    g_rt.stream = nullptr;
    g_rt.ready = false;
}

int oxb_hip_device_info(char* name, size_t name_cap, size_t* free_bytes, size_t* total_bytes) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    int rc = ensure_init();
    if (rc) return rc;
    if (name && name_cap) snprintf(name, name_cap, "%s", g_rt.name);
    size_t f = 0, t = 0;
    hipError_t e = hipMemGetInfo(&f, &t);
    if (e != hipSuccess) return hip_fail(e, "memory info");
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_synchronize(void) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    int rc = ensure_init();
    if (rc) return rc;
    return sync_stream("synchronize");
    OXB_API_END
}

int oxb_hip_set_stream(void* hip_stream) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    int rc = ensure_init();
    if (rc) return rc;
    g_rt.stream = hip_stream ? (hipStream_t)hip_stream : g_rt.own_stream;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_upload_q1(uint64_t* id, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    return upload_weight(id, OXB_FMT_Q1, aos, n_bytes, n_rows, k);
    OXB_API_END
}

int oxb_hip_upload_tq2(uint64_t* id, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    return upload_weight(id, OXB_FMT_TQ2, aos, n_bytes, n_rows, k);
    OXB_API_END
}

int oxb_hip_upload_q1_raw(uint64_t* id, const uint8_t* aos, size_t n_bytes) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    return upload_weight_bytes(id, OXB_FMT_Q1, aos, n_bytes);
    OXB_API_END
}

int oxb_hip_upload_tq2_raw(uint64_t* id, const uint8_t* aos, size_t n_bytes) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    return upload_weight_bytes(id, OXB_FMT_TQ2, aos, n_bytes);
    OXB_API_END
}

int oxb_hip_free_weight(uint64_t id) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    if (g_rt.ready) (void)hipStreamSynchronize(g_rt.stream);
    free_weight_mem(*w);
    g_rt.weights.erase(id);
    g_rt.weights_gen++;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_weight_info(uint64_t id, int* fmt, uint32_t* n_rows, uint32_t* k, size_t* resident_bytes) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    if (fmt) *fmt = (int)w->L.fmt;
    if (n_rows) *n_rows = w->L.n_rows;
    if (k) *k = w->L.k;
    if (resident_bytes)
        *resident_bytes = w->d_raw ? w->raw_blocks * (w->L.fmt == OXB_FMT_Q1 ? OXB_Q1_AOS_BYTES : OXB_TQ2_AOS_BYTES)
                                   : w->L.codes_bytes + w->L.scales_bytes;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_dequant(uint64_t id, float* out, size_t out_len) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    if (w->d_raw)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight %llu was uploaded without a shape and no call has named one yet",
                    (unsigned long long)id);
    const size_t n = (size_t)w->L.n_rows * w->L.k;
    if (!out || out_len < n) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: output holds %zu values, %zu needed", out_len, n);
    int rc = g_rt.ws_y.ensure(n * sizeof(float));
    if (rc) return rc;
    hipError_t e = oxb_launch_dequant(w->L, w->d_codes, w->d_scales, (float*)g_rt.ws_y.ptr, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "kernel launch failed: dequant");
    e = hipMemcpyAsync(out, g_rt.ws_y.ptr, n * sizeof(float), hipMemcpyDeviceToHost, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "dequant download");
    return sync_stream("dequant");
    OXB_API_END
}

int oxb_hip_gemv_dev(uint64_t id, const float* d_x, float* d_y, uint32_t n_rows, uint32_t k, uint32_t batch) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    int rc = bind_shape(*w, n_rows, k);
    if (rc) return rc;
    if (!d_x || !d_y || batch == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or batch 0");
    return gemv_device(*w, d_x, d_y, batch, n_rows, OXB_GEMV_STORE, nullptr);
    OXB_API_END
}

static int profile_gemv_impl(bool floor_only, const uint64_t* ids, uint32_t n_ids, const float* d_x, float* d_y, uint32_t n_rows,
                             uint32_t k, uint32_t warmup, uint32_t iters, float* avg_us) {
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!ids || n_ids == 0 || (!floor_only && (!d_x || !d_y)) || !avg_us || iters == 0)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or zero count");
    std::vector<const Weight*> ws;
    for (uint32_t i = 0; i < n_ids; i++) {
        Weight* w = find_weight(ids[i]);
        if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)ids[i]);
        int rc = bind_shape(*w, n_rows, k);
        if (rc) return rc;
        if (!ws.empty() && w->L.fmt != ws[0]->L.fmt)
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weights differ in format");
        ws.push_back(w);
    }
    if (ws[0]->L.n_sb > OXB_GEMV_MAX_SB) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: k too large for a single launch");
    const int fmt = (int)ws[0]->L.fmt;
    OxbGemvParams p;
    memset(&p, 0, sizeof p);
    p.x = d_x;
    p.y = d_y;
    p.n_rows = n_rows;
    p.n_tiles = ws[0]->L.n_tiles;
    p.n_sb = ws[0]->L.n_sb;
    p.k = k;
    p.sb_begin = 0;
    p.sb_count = p.n_sb;
    p.nvec = 1;
    p.ldx = k;
    p.ldy = n_rows;
    p.pro = OXB_GEMV_PRO_F32;
    p.epi = OXB_GEMV_STORE;
    hipEvent_t ev0, ev1;
    hipError_t e;
    if ((e = hipEventCreate(&ev0)) != hipSuccess) return hip_fail(e, "event creation");
    if ((e = hipEventCreate(&ev1)) != hipSuccess) { (void)hipEventDestroy(ev0); return hip_fail(e, "event creation"); }
    int rc = OXB_HIP_OK;
    for (uint32_t i = 0; i < warmup + iters && rc == OXB_HIP_OK; i++) {
        if (i == warmup) (void)hipEventRecord(ev0, g_rt.stream);
        const Weight* w = ws[i % n_ids];
        p.codes = w->d_codes;
        p.scales = w->d_scales;
        p.codes_bytes = (uint32_t)w->L.codes_bytes;
        p.scales_bytes = (uint32_t)w->L.scales_bytes;
        e = floor_only ? oxb_launch_gemv_stream_floor(fmt, p, g_rt.n_cus, g_rt.stream) : oxb_launch_gemv(fmt, p, g_rt.n_cus, g_rt.stream);
        if (e != hipSuccess) rc = hip_fail(e, "kernel launch failed: gemv");
    }
    (void)hipEventRecord(ev1, g_rt.stream);
    if (rc == OXB_HIP_OK) {
        e = hipEventSynchronize(ev1);
        if (e != hipSuccess) rc = fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: %s", hipGetErrorString(e));
    }
    if (rc == OXB_HIP_OK) {
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, ev0, ev1);
        *avg_us = ms * 1000.0f / (float)iters;
    }
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    return rc;
}

int oxb_hip_set_gemv_packed_min_batch(uint32_t n) {
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    g_packed_min_batch = n;
    return OXB_HIP_OK;
}

int oxb_hip_profile_gemv(const uint64_t* ids, uint32_t n_ids, const float* d_x, float* d_y, uint32_t n_rows,
                         uint32_t k, uint32_t warmup, uint32_t iters, float* avg_us) {
    OXB_API_BEGIN
    return profile_gemv_impl(false, ids, n_ids, d_x, d_y, n_rows, k, warmup, iters, avg_us);
    OXB_API_END
}

int oxb_hip_profile_gemv_floor(const uint64_t* ids, uint32_t n_ids, uint32_t n_rows, uint32_t k, uint32_t warmup,
                               uint32_t iters, float* avg_us) {
    OXB_API_BEGIN
    return profile_gemv_impl(true, ids, n_ids, nullptr, nullptr, n_rows, k, warmup, iters, avg_us);
    OXB_API_END
}

int oxb_hip_gemm_dev(uint64_t id, const float* d_x, float* d_y, uint32_t m, uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    int rc = bind_shape(*w, n_rows, k);
    if (rc) return rc;
    if (!d_x || !d_y || m == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or m = 0");
    return gemm_device(*w, d_x, k, d_y, m, n_rows, OXB_GEMM_STORE, nullptr, OXB_PACK_IDENT, nullptr, 0.f);
    OXB_API_END
}

int oxb_hip_gemm_dev_static(uint64_t id, const float* d_x, float* d_y, uint32_t m, uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    if (w->d_raw)  // binding a shape allocates the resident copy: not in this entry point
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight %llu was uploaded without a shape; name its shape in another call first",
                    (unsigned long long)id);
    int rc = bind_shape(*w, n_rows, k);
    if (rc) return rc;
    if (!d_x || !d_y || m == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or m = 0");
    if (!g_rt.ready || !g_rt.static_scratch) return fail(OXB_HIP_NOT_AVAILABLE, "GPU not available: the library is not initialised");
    // Carve the file-scope array into the four buffers of a GEMM call.  Every byte the kernels read from them is
    // written earlier in the same call (the packer fills its padding rows and blocks with zeros, every K slice
    // writes all of its partial sums), so nothing needs clearing between calls.
    OxbGemmParams gp;
    memset(&gp, 0, sizeof gp);
    gp.n_rows = n_rows, gp.n_tiles = w->L.n_tiles, gp.n_sb = w->L.n_sb, gp.M = m, gp.ldy = n_rows;
    const uint32_t ksplit = oxb_gemm_ksplit(gp, g_rt.n_cus);
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t need[4] = {up(oxb_xh_bytes(k, m)), up(((size_t)m + 16) * sizeof(int32_t)), up(((size_t)m + 16) * sizeof(float)),
                            ksplit > 1 ? up((size_t)ksplit * m * n_rows * sizeof(float)) : 0};
    const size_t total = need[0] + need[1] + need[2] + need[3];
    if (total > OXB_STATIC_SCRATCH_BYTES)
        return fail(OXB_HIP_INVALID_ARGUMENT,
                    "invalid argument: a GEMM of %u rows x %u x %u needs %zu bytes of scratch, the allocation-free entry point holds %u",
                    m, n_rows, k, total, OXB_STATIC_SCRATCH_BYTES);
    GemmWorkspace ws;
    DevBuf* bufs[4] = {&ws.xh, &ws.xsh, &ws.rowmul, &ws.part};
    size_t off = 0;
    for (int i = 0; i < 4; i++) {
        bufs[i]->ptr = need[i] ? (unsigned char*)g_rt.static_scratch + off : nullptr;
        bufs[i]->cap = need[i];
        bufs[i]->fixed = true;
        off += need[i];
    }
    return gemm_device(*w, d_x, k, d_y, m, n_rows, OXB_GEMM_STORE, nullptr, OXB_PACK_IDENT, nullptr, 0.f, &ws);
    OXB_API_END
}

int oxb_hip_gemm(uint64_t id, const float* x, float* y, uint32_t m, uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    int rc = bind_shape(*w, n_rows, k);
    if (rc) return rc;
    if (!x || !y || m == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or m = 0");
    const size_t xb = (size_t)m * k * sizeof(float), yb = (size_t)m * n_rows * sizeof(float);
    if ((rc = g_rt.ws_x.ensure(xb))) return rc;
    if ((rc = g_rt.ws_y.ensure(yb))) return rc;
    hipError_t e = hipMemcpyAsync(g_rt.ws_x.ptr, x, xb, hipMemcpyHostToDevice, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "input upload");
    rc = gemm_device(*w, (const float*)g_rt.ws_x.ptr, k, (float*)g_rt.ws_y.ptr, m, n_rows, OXB_GEMM_STORE, nullptr, OXB_PACK_IDENT, nullptr, 0.f);
    if (rc) return rc;
    e = hipMemcpyAsync(y, g_rt.ws_y.ptr, yb, hipMemcpyDeviceToHost, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "output download");
    return sync_stream("gemm");
    OXB_API_END
}

int oxb_hip_profile_gemm(uint64_t id, const float* d_x, float* d_y, uint32_t m, uint32_t n_rows, uint32_t k,
                         uint32_t warmup, uint32_t iters, float* avg_us) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    int rc = bind_shape(*w, n_rows, k);
    if (rc) return rc;
    if (!d_x || !d_y || !avg_us || m == 0 || iters == 0)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or zero count");
    if ((rc = gemm_device(*w, d_x, k, d_y, m, n_rows, OXB_GEMM_STORE, nullptr, OXB_PACK_IDENT, nullptr, 0.f))) return rc;  // packs x, warms up
    OxbGemmParams p;
    memset(&p, 0, sizeof p);
    p.codes = w->d_codes;
    p.scales = w->d_scales;
    p.xh = (const uint32_t*)g_rt.gemm_ws.xh.ptr;
    p.xsh = (const int32_t*)g_rt.gemm_ws.xsh.ptr;
    p.y = d_y;
    p.n_rows = n_rows;
    p.n_tiles = w->L.n_tiles;
    p.n_sb = w->L.n_sb;
    p.M = m;
    p.ldy = n_rows;
    p.codes_bytes = (uint32_t)w->L.codes_bytes;
    p.scales_bytes = (uint32_t)w->L.scales_bytes;
    p.xh_bytes = (uint32_t)oxb_xh_bytes(k, m);
    p.mode = OXB_GEMM_STORE;
    p.part = (float*)g_rt.gemm_ws.part.ptr;  // sized by the gemm_device call above
    hipEvent_t ev0, ev1;
    hipError_t e;
    if ((e = hipEventCreate(&ev0)) != hipSuccess) return hip_fail(e, "event creation");
    if ((e = hipEventCreate(&ev1)) != hipSuccess) { (void)hipEventDestroy(ev0); return hip_fail(e, "event creation"); }
    for (uint32_t i = 0; i < warmup + iters && rc == OXB_HIP_OK; i++) {
        if (i == warmup) (void)hipEventRecord(ev0, g_rt.stream);
        e = oxb_launch_gemm((int)w->L.fmt, p, g_rt.n_cus, g_rt.stream);
        if (e != hipSuccess) rc = hip_fail(e, "kernel launch failed: gemm");
    }
    (void)hipEventRecord(ev1, g_rt.stream);
    if (rc == OXB_HIP_OK) {
        e = hipEventSynchronize(ev1);
        if (e != hipSuccess) rc = fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: %s", hipGetErrorString(e));
    }
    if (rc == OXB_HIP_OK) {
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, ev0, ev1);
        *avg_us = ms * 1000.0f / (float)iters;
    }
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    return rc;
    OXB_API_END
}

int oxb_hip_gemv(uint64_t id, const float* x, float* y, uint32_t n_rows, uint32_t k, uint32_t batch) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Weight* w = find_weight(id);
    if (!w) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    int rc = bind_shape(*w, n_rows, k);
    if (rc) return rc;
    if (!x || !y || batch == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer or batch 0");
    const size_t xb = (size_t)batch * k * sizeof(float), yb = (size_t)batch * n_rows * sizeof(float);
    if ((rc = g_rt.ws_x.ensure(xb))) return rc;
    if ((rc = g_rt.ws_y.ensure(yb))) return rc;
    hipError_t e = hipMemcpyAsync(g_rt.ws_x.ptr, x, xb, hipMemcpyHostToDevice, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "input upload");
    rc = gemv_device(*w, (const float*)g_rt.ws_x.ptr, (float*)g_rt.ws_y.ptr, batch, n_rows, OXB_GEMV_STORE, nullptr);
    if (rc) return rc;
    e = hipMemcpyAsync(y, g_rt.ws_y.ptr, yb, hipMemcpyDeviceToHost, g_rt.stream);
    if (e != hipSuccess) return hip_fail(e, "output download");
    return sync_stream("gemv");
    OXB_API_END
}

int oxb_hip_gemv_q1_g128(const uint8_t* aos, size_t n_bytes, const float* x, size_t x_len, float* y, size_t y_len,
                         uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    return oneshot_gemv(OXB_FMT_Q1, aos, n_bytes, x, x_len, y, y_len, n_rows, k);
    OXB_API_END
}

int oxb_hip_gemv_tq2_g128(const uint8_t* aos, size_t n_bytes, const float* x, size_t x_len, float* y, size_t y_len,
                          uint32_t n_rows, uint32_t k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    return oneshot_gemv(OXB_FMT_TQ2, aos, n_bytes, x, x_len, y, y_len, n_rows, k);
    OXB_API_END
}

// ---- host-only repack helpers -------------------------------------------------
static int repack_args(int fmt, uint32_t n_rows, uint32_t k) {
    if (fmt != OXB_FMT_Q1 && fmt != OXB_FMT_TQ2) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown format %d", fmt);
    if (k == 0 || k % OXB_QK != 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: k=%u is not a multiple of 128", k);
    if (n_rows == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: n_rows is 0");
    return OXB_HIP_OK;
}

int oxb_hip_repack_sizes(int fmt, uint32_t n_rows, uint32_t k, size_t* codes_bytes, size_t* scales_bytes) {
    OXB_API_BEGIN
    int rc = repack_args(fmt, n_rows, k);
    if (rc) return rc;
    OxbLayout L = oxb_make_layout((uint32_t)fmt, n_rows, k);
    if (codes_bytes) *codes_bytes = L.codes_bytes;
    if (scales_bytes) *scales_bytes = L.scales_bytes;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_repack(int fmt, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k, uint8_t* codes,
                   size_t codes_cap, uint8_t* scales, size_t scales_cap) {
    OXB_API_BEGIN
    int rc = repack_args(fmt, n_rows, k);
    if (rc) return rc;
    OxbLayout L = oxb_make_layout((uint32_t)fmt, n_rows, k);
    const size_t need = (size_t)n_rows * (k / OXB_QK) * (fmt == OXB_FMT_Q1 ? OXB_Q1_AOS_BYTES : OXB_TQ2_AOS_BYTES);
    if (!aos || n_bytes < need) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: weight buffer holds %zu bytes, %zu needed", n_bytes, need);
    if (!codes || !scales || codes_cap < L.codes_bytes || scales_cap < L.scales_bytes)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: output sections too small");
    oxb_repack_aos_to_tiled(L, aos, reinterpret_cast<uint32_t*>(codes), reinterpret_cast<uint16_t*>(scales));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_unpack(int fmt, const uint8_t* codes, size_t codes_len, const uint8_t* scales, size_t scales_len,
                   uint32_t n_rows, uint32_t k, uint8_t* aos, size_t aos_cap) {
    OXB_API_BEGIN
    int rc = repack_args(fmt, n_rows, k);
    if (rc) return rc;
    OxbLayout L = oxb_make_layout((uint32_t)fmt, n_rows, k);
    const size_t need = (size_t)n_rows * (k / OXB_QK) * (fmt == OXB_FMT_Q1 ? OXB_Q1_AOS_BYTES : OXB_TQ2_AOS_BYTES);
    if (!codes || !scales || codes_len < L.codes_bytes || scales_len < L.scales_bytes || !aos || aos_cap < need)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: buffer sizes do not match the layout");
    oxb_repack_tiled_to_aos(L, reinterpret_cast<const uint32_t*>(codes), reinterpret_cast<const uint16_t*>(scales), aos);
    return OXB_HIP_OK;
    OXB_API_END
}

}  // extern "C"
