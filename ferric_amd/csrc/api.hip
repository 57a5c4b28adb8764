// The extern "C" surface of libferric_hip (declared in include/ferric_hip.h): argument checks with
// the reference's error behaviour, weight handles, and thin dispatch into the kernel launchers.
#include "common.hpp"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <vector>

namespace {

// The intermediate of fhip_ffn_noalloc: [rows_x, n_ff] f32 between the gate|up and the down mat-vec. It lives in the code
// object, so each device the library runs on holds its own copy (512 KiB) from load to process exit and no call has to
// allocate. Host code never uses the array's name as an address: fhip_init asks the runtime for the device address of the
// current device's copy and keeps it per device.
constexpr size_t WEIGHT_SLACK = 256;   // readable bytes every weight has behind its last block
constexpr size_t NOALLOC_FLOATS = 131072;
static __device__ __align__(256) float scratch[NOALLOC_FLOATS];
constexpr int MAX_DEVICES = 64;
float* g_scratch_ptr[MAX_DEVICES] = {};

thread_local char g_err[512] = "";
int g_device = -1;
// What a new weight handle starts with (fhip_matvec_precision, fhip_batch_policy); read when a handle is made, never at a launch.
int g_default_planes = 3;
int g_default_batch_policy = FHIP_BATCH_ORDERED;
int g_cus = 0;
size_t g_lds = 64 * 1024;

bool block_info(uint32_t ty, size_t& vals, size_t& bytes) {
    switch (ty) {
        case FHIP_Q8_0: vals = 32; bytes = 34; return true;
        case FHIP_Q4_K: vals = 256; bytes = 144; return true;
        case FHIP_Q6_K: vals = 256; bytes = 210; return true;
        case FHIP_Q4_0: vals = 32; bytes = 18; return true;
        case FHIP_Q4_1: vals = 32; bytes = 20; return true;
        case FHIP_Q5_0: vals = 32; bytes = 22; return true;
        case FHIP_Q5_1: vals = 32; bytes = 24; return true;
        case FHIP_Q5_K: vals = 256; bytes = 176; return true;
        case FHIP_IQ4_NL: vals = 32; bytes = 18; return true;
        case FHIP_IQ4_XS: vals = 256; bytes = 136; return true;
        case FHIP_MXFP4: vals = 32; bytes = 17; return true;
        default: return false;
    }
}

const char* type_name(uint32_t ty) {
    switch (ty) {
        case FHIP_Q8_0: return "Q8_0";
        case FHIP_Q4_K: return "Q4_K";
        case FHIP_Q6_K: return "Q6_K";
        case FHIP_Q4_0: return "Q4_0";
        case FHIP_Q4_1: return "Q4_1";
        case FHIP_Q5_0: return "Q5_0";
        case FHIP_Q5_1: return "Q5_1";
        case FHIP_Q5_K: return "Q5_K";
        case FHIP_IQ4_NL: return "IQ4_NL";
        case FHIP_IQ4_XS: return "IQ4_XS";
        case FHIP_MXFP4: return "MXFP4";
        default: return "?";
    }
}

int need_init() {
    if (g_device < 0) return fhip::set_error(FHIP_ERR_ARG, "fhip_init has not been called");
    return FHIP_OK;
}

// Shape checks of the per-format constructors: crates/ferric-tensor/src/dtype.rs:1271-1272 (Q8_0),
// :1389-1390 (Q4_K), :1148-1149 (Q6_K) -- `assert_eq!(cols % blk, 0)` and exact byte length.
int make_weight(uint32_t ty, size_t nbytes, size_t rows, size_t cols, fhip_weight& w) {
    size_t vals, bytes;
    if (!block_info(ty, vals, bytes)) return fhip::set_error(FHIP_ERR_UNSUPPORTED_TYPE, "QMatrix: no native matmul for ggml type %u", ty);
    if (cols % vals != 0) return fhip::set_error(FHIP_ERR_SHAPE, "%s cols must be a multiple of %zu", type_name(ty), vals);
    size_t row_bytes = cols / vals * bytes;
    if (nbytes != rows * row_bytes) return fhip::set_error(FHIP_ERR_SHAPE, "unexpected %s byte length", type_name(ty));
    if (rows > 0x7FFFFFFFull || cols > 0x7FFFFFFFull) return fhip::set_error(FHIP_ERR_SHAPE, "weight dimensions exceed 2^31");
    w.type = ty; w.rows = rows; w.cols = cols; w.row_bytes = row_bytes; w.nbytes = nbytes; w.d_raw = nullptr; w.owns = false;
    w.planes = g_default_planes; w.batch_policy = g_default_batch_policy;
    return FHIP_OK;
}

}  // namespace

namespace fhip {

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return FHIP_OK;
    return set_error(FHIP_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int device_cus() { return g_cus; }
size_t device_lds_bytes() { return g_lds; }

// The streaming mat-vec exists in two copies, one per activation precision; these forward to the one the weight names.
// From three rows on, Q4_K, Q5_K and Q6_K batches go four rows at a time through the kernel that multiplies on the 4 x 4 x 4 int8
// matrix instruction (gemv_quad.hip: the same arithmetic and the same bits per row, one pass over the weight for four rows);
// what is left of a batch, one or two rows, and every other format take the dot-product kernel.
bool g_quad_matvec = true, g_generic_forced = false;
int launch_gemv(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, size_t n_ff, hipStream_t s) {
    const bool p3 = w->planes == 3;
    if (rows_x >= 3 && g_quad_matvec && !g_generic_forced && d_x && d_y &&
        (p3 ? gemv_quad_supports_p3(w, 4, n_ff) : gemv_quad_supports_p2(w, 4, n_ff))) {
        const size_t out_rows = n_ff ? n_ff : w->rows;
        for (size_t m0 = 0; m0 < rows_x;) {
            const size_t t = rows_x - m0 < 4 ? rows_x - m0 : 4;
            const float* x = d_x + m0 * w->cols;
            float* y = d_y + m0 * out_rows;
            int rc;
            if (t >= 3) rc = p3 ? launch_gemv_quad_p3(w, x, t, y, n_ff, s) : launch_gemv_quad_p2(w, x, t, y, n_ff, s);
            else rc = p3 ? launch_gemv_p3(w, x, t, y, n_ff, s) : launch_gemv_p2(w, x, t, y, n_ff, s);
            if (rc) return rc;
            m0 += t;
        }
        return FHIP_OK;
    }
    return p3 ? launch_gemv_p3(w, d_x, rows_x, d_y, n_ff, s) : launch_gemv_p2(w, d_x, rows_x, d_y, n_ff, s);
}
bool gemv_quad_matvec(bool on) {
    const bool before = g_quad_matvec;
    g_quad_matvec = on;
    return before;
}
int launch_gemv_norm(const fhip_weight* w, const float* d_x, float* d_y, size_t n_ff, const NormParams& norm, hipStream_t s) {
    return w->planes == 3 ? launch_gemv_norm_p3(w, d_x, d_y, n_ff, norm, s) : launch_gemv_norm_p2(w, d_x, d_y, n_ff, norm, s);
}
int launch_gemv_sel(const fhip_weight* w, const float* d_x, float* d_y, size_t out_rows, bool swiglu, const SelParams& sel, hipStream_t s) {
    return w->planes == 3 ? launch_gemv_sel_p3(w, d_x, d_y, out_rows, swiglu, sel, s) : launch_gemv_sel_p2(w, d_x, d_y, out_rows, swiglu, sel, s);
}
void gemv_force_generic(bool on) {
    g_generic_forced = on;
    gemv_force_generic_p2(on);
    gemv_force_generic_p3(on);
}

}  // namespace fhip

using fhip::check_hip;
using fhip::set_error;

namespace {

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

// ---- the library's own workspace, one per stream -------------------------------------------------------------------------
// The one-pass small-batch kernels need a few megabytes of device memory beside their operands (prepared activation rows,
// the gate|up intermediate). The drop-in entry points (fhip_matmul_q, fhip_matmul_q_swiglu, fhip_ffn) have no argument for
// it, so the library keeps a buffer per stream: work on one stream is ordered, so calls there can share it. It only ever
// grows, to the next power of two, and a buffer that was outgrown stays allocated until fhip_workspace_release: a graph
// captured earlier may still name it. Growing means hipMalloc, which a capturing stream does not allow.
struct StreamWs { hipStream_t s; void* cur; size_t n; std::vector<void*> retired; };
std::mutex g_ws_mu;
std::vector<StreamWs> g_ws;

int lib_workspace(hipStream_t s, size_t need, void** out, const char* who) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    StreamWs* e = nullptr;
    for (auto& w : g_ws) if (w.s == s) e = &w;
    if (e && e->n >= need) { *out = e->cur; return FHIP_OK; }
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) (void)hipGetLastError();
    if (st != hipStreamCaptureStatusNone)
        return set_error(FHIP_ERR_ARG, "%s: the library workspace of this stream has to grow to %zu bytes, which a capturing stream does not "
                         "allow: call fhip_workspace_reserve(stream, %zu) before the capture begins", who, need, need);
    size_t n = 1 << 20;
    while (n < need) n <<= 1;
    void* p = nullptr;
    int rc = check_hip(hipMalloc(&p, n), "hipMalloc (library workspace)");
    if (rc) return rc;
    if (!e) { g_ws.push_back(StreamWs{s, nullptr, 0, {}}); e = &g_ws.back(); }
    if (e->cur) e->retired.push_back(e->cur);
    e->cur = p; e->n = n;
    *out = p;
    return FHIP_OK;
}

void release_workspace(hipStream_t s) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    for (size_t i = 0; i < g_ws.size(); i++) {
        if (g_ws[i].s != s) continue;
        (void)hipStreamSynchronize(s);
        if (g_ws[i].cur) (void)hipFree(g_ws[i].cur);
        for (void* p : g_ws[i].retired) (void)hipFree(p);
        g_ws.erase(g_ws.begin() + i);
        return;
    }
}

// The matrix-core GEMM with its K-split scratch (partial tiles of the tiles that several workgroups share) taken from the
// stream's library workspace.
static int gemm_bf16_lib_ws(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, hipStream_t s, const char* who) {
    const size_t need = fhip::gemm_bf16_ws_bytes(w, t);
    void* ws = nullptr;
    if (need) {
        int rc = lib_workspace(s, need, &ws, who);
        if (rc) return rc;
    }
    return fhip::launch_gemm_bf16(w, d_x, t, d_y, s, (float*)ws, need);
}

// ---- which kernel a batch takes ---------------------------------------------------------------------------------------------
// One or two activation rows go through the streaming mat-vec (one pass over the weights serves two rows). From three rows on
// (five for Q8_0) the f16 hi/lo matrix-core kernels read the weights once for up to 32 (Q8_0: 16) rows; longer batches are cut
// into such groups. FHIP_BATCH_F32_MATVEC keeps every batch on the mat-vec's arithmetic (launch_gemv: four rows a pass on the
// int8 matrix instruction for Q4_K / Q5_K / Q6_K, the dot-product kernel otherwise): a row then has the same bits whatever batch it
// is part of.

size_t f16x2_group(const fhip_weight* w) { return w->type == FHIP_Q8_0 ? 16 : 32; }
// Three and four rows of a Q4_K / Q5_K / Q6_K weight whose rows the four-row mat-vec (gemv_quad.hip) covers in one pass (up to 10240
// columns) take that kernel under every policy: one launch, no workspace, the bits of a batch of one, and faster than the f16
// kernels with their split and sum launches (cold, ordered sums: 5120 x 5120 17.7 -> 12.5 us, 7168 x 5120 19.9 -> 14.1, Q6_K
// 151936 x 5120 178 -> 164; with atomic sums 12.6 / 14.5 / 178). Longer rows take two passes and lose (5120 x 17408: 36.6 against
// 43.8), so they stay on the f16 kernels.
bool matmul_takes_quad(const fhip_weight* w, size_t t) {
    if (t < 3 || t > 4 || w->cols > 10240) return false;      // (Q8_0: 5120, gemv_quad_supports)
    return w->planes == 3 ? fhip::gemv_quad_supports_p3(w, t, 0) : fhip::gemv_quad_supports_p2(w, t, 0);
}
bool takes_f16x2(const fhip_weight* w, size_t rows_x) {
    if (w->batch_policy == FHIP_BATCH_F32_MATVEC) return false;
    if (w->type != FHIP_Q4_K && w->type != FHIP_Q5_K && w->type != FHIP_Q6_K && w->type != FHIP_Q8_0) return false;
    if (rows_x < (w->type == FHIP_Q8_0 ? 5u : 3u)) return false;
    if (matmul_takes_quad(w, rows_x)) return false;
    return fhip::gemm_f16x2_supports(w, rows_x < f16x2_group(w) ? rows_x : f16x2_group(w));
}

// Fused gate|up + SwiGLU at three or four rows: one pass of the int8 matrix-instruction mat-vec (gemv_quad.hip, 31 us on
// 34816 x 5120) is faster than the one-pass f16 kernel plus the SwiGLU launch behind it (34 + 4), and its rows carry the bits
// they have in a batch of one. The plain matmuls of such batches stay on the f16 kernels (down 5120 x 17408: 27 us against 42).
bool swiglu_takes_quad(const fhip_weight* gu, size_t t) {
    if (t < 3 || t > 4 || gu->rows % 2 != 0 || gu->cols > 10240) return false;   // (one pass of the kernel, as matmul_takes_quad)
    return gu->planes == 3 ? fhip::gemv_quad_supports_p3(gu, t, gu->rows / 2) : fhip::gemv_quad_supports_p2(gu, t, gu->rows / 2);
}

// fhip_ffn on a group of t rows needs no library workspace when the down projection does not take the f16 kernels, or when
// gate|up takes neither them nor the four-row mat-vec: both matmuls then go through the mat-vec launcher.
bool ffn_direct(const fhip_weight* gu, const fhip_weight* down, size_t t) {
    return !takes_f16x2(down, t) || (!takes_f16x2(gu, t) && !swiglu_takes_quad(gu, t));
}

// y [t, rows] = 0 on the stream, by the mat-vec launcher's fill kernel (what a weight without columns gives)
int zero_outputs(size_t t, size_t rows, float* d_y, hipStream_t s) {
    fhip_weight z{};
    z.type = FHIP_Q8_0; z.rows = rows; z.cols = 0; z.planes = 2;
    return fhip::launch_gemv(&z, d_y, t, d_y, 0, s);
}

// y [t, w->rows] = x [t, cols] W^T for t rows of one group; ws: f16x2_matmul_ws(w, t) bytes
// (FHIP_BATCH_ORDERED: behind the prepared activations, the partial sums of the groups the launch cuts along K)
size_t f16x2_matmul_ws(const fhip_weight* w, size_t t) {
    return align256(fhip::gemm_f16x2_xp_bytes(w, t)) + (w->batch_policy == FHIP_BATCH_ORDERED ? align256(fhip::gemm_f16x2_part_bytes_upto(w, t)) : 0);
}
// deferred: the ordered sum of K-split groups is left to the reader of y, which gets *deferred as its `src`
int f16x2_matmul(const fhip_weight* w, const float* d_x, size_t t, bool swiglu_in, float* d_y, void* d_ws, hipStream_t s,
                 fhip::F16Parts* deferred = nullptr, const fhip::F16Parts* src = nullptr) {
    uint16_t* xp = (uint16_t*)d_ws;
    const bool ordered = w->batch_policy == FHIP_BATCH_ORDERED;
    float* part = ordered && fhip::gemm_f16x2_part_bytes(w, t) ? (float*)((uint8_t*)d_ws + align256(fhip::gemm_f16x2_xp_bytes(w, t))) : nullptr;
    const bool clr = !part && fhip::gemm_f16x2_adds_into_y(w, t);   // then the split clears y on the side
    int rc = fhip::launch_xsplit_f16(w, d_x, t, swiglu_in, xp, s, clr ? d_y : nullptr, clr ? t * w->rows : 0, src);
    if (rc) return rc;
    return fhip::launch_gemm_f16x2(w, xp, t, d_y, s, clr, part, deferred);
}

}  // namespace

extern "C" {

int fhip_init(int device) {
    int n = 0;
    int rc = check_hip(hipGetDeviceCount(&n), "hipGetDeviceCount");
    if (rc) return rc;
    if (device < 0 || device >= n) return set_error(FHIP_ERR_ARG, "device %d out of range (%d visible)", device, n);
    if ((rc = check_hip(hipSetDevice(device), "hipSetDevice"))) return rc;
    hipDeviceProp_t prop;
    if ((rc = check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties"))) return rc;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(FHIP_ERR_HIP, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    g_cus = prop.multiProcessorCount;
    g_lds = prop.sharedMemPerBlockOptin > prop.sharedMemPerBlock ? prop.sharedMemPerBlockOptin : prop.sharedMemPerBlock;
    if (g_lds < 64 * 1024) g_lds = 64 * 1024;
    if (device < MAX_DEVICES && !g_scratch_ptr[device]) {   // this device's copy of the built-in scratch array
        float* ptr = nullptr;
        if ((rc = check_hip(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)"))) return rc;
        g_scratch_ptr[device] = ptr;
    }
    g_device = device;
    return FHIP_OK;
}

const char* fhip_last_error(void) { return g_err; }
int fhip_device_cus(void) { return g_cus; }

// bytes per element of the unquantized tensor types (crates/ferric-gguf/src/lib.rs:473-475), 0 for anything else
static size_t dense_elem_bytes(uint32_t ty) { return ty == FHIP_F32 ? 4 : (ty == FHIP_F16 || ty == FHIP_BF16 ? 2 : 0); }

size_t fhip_type_size(uint32_t ty, size_t n) {
    if (const size_t eb = dense_elem_bytes(ty)) return n * eb;
    size_t vals, bytes;
    if (!block_info(ty, vals, bytes)) { set_error(FHIP_ERR_UNSUPPORTED_TYPE, "unsupported ggml type %u", ty); return 0; }
    return n / vals * bytes;
}

int fhip_block_bytes(uint32_t ty, size_t* values, size_t* bytes) {
    size_t v, b;
    if (!values || !bytes) return set_error(FHIP_ERR_ARG, "fhip_block_bytes: NULL output");
    if (!block_info(ty, v, b)) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "unsupported ggml type %u", ty);
    *values = v; *bytes = b;
    return FHIP_OK;
}

// ---- plumbing -------------------------------------------------------------------------------

int fhip_malloc(void** d_ptr, size_t nbytes) {
    if (!d_ptr) return set_error(FHIP_ERR_ARG, "fhip_malloc: NULL output");
    int rc = need_init();
    if (rc) return rc;
    *d_ptr = nullptr;
    // 256 bytes more than asked for: a weight wrapped at the end of such a buffer (fhip_weight_wrap_device) keeps the slack
    // behind its last block that fhip_weight_create gives its own allocations
    return check_hip(hipMalloc(d_ptr, nbytes + WEIGHT_SLACK), "hipMalloc");
}
int fhip_free(void* d_ptr) { return d_ptr ? check_hip(hipFree(d_ptr), "hipFree") : FHIP_OK; }
int fhip_memcpy_h2d(void* d, const void* h, size_t n, void* s) {
    if (n == 0) return FHIP_OK;
    if (!d || !h) return set_error(FHIP_ERR_ARG, "fhip_memcpy_h2d: NULL pointer");
    return check_hip(hipMemcpyAsync(d, h, n, hipMemcpyHostToDevice, (hipStream_t)s), "hipMemcpyAsync H2D");
}
int fhip_memcpy_d2h(void* h, const void* d, size_t n, void* s) {
    if (n == 0) return FHIP_OK;
    if (!d || !h) return set_error(FHIP_ERR_ARG, "fhip_memcpy_d2h: NULL pointer");
    int rc = check_hip(hipMemcpyAsync(h, d, n, hipMemcpyDeviceToHost, (hipStream_t)s), "hipMemcpyAsync D2H");
    if (rc) return rc;
    return check_hip(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize");
}
int fhip_memcpy_d2d(void* dst, const void* src, size_t n, void* s) {
    if (n == 0) return FHIP_OK;
    if (!dst || !src) return set_error(FHIP_ERR_ARG, "fhip_memcpy_d2d: NULL pointer");
    return check_hip(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, (hipStream_t)s), "hipMemcpyAsync D2D");
}
int fhip_memcpy_2d_d2d(void* d, size_t dpitch, const void* src, size_t spitch, size_t width, size_t height, void* s) {
    if (width == 0 || height == 0) return FHIP_OK;
    if (!d || !src) return set_error(FHIP_ERR_ARG, "fhip_memcpy_2d_d2d: NULL pointer");
    if (dpitch < width || spitch < width) return set_error(FHIP_ERR_ARG, "fhip_memcpy_2d_d2d: pitch smaller than the row width");
    return check_hip(hipMemcpy2DAsync(d, dpitch, src, spitch, width, height, hipMemcpyDeviceToDevice, (hipStream_t)s), "hipMemcpy2D D2D");
}
int fhip_memset(void* d, int byte, size_t n, void* s) {
    if (n == 0) return FHIP_OK;
    if (!d) return set_error(FHIP_ERR_ARG, "fhip_memset: NULL pointer");
    return check_hip(hipMemsetAsync(d, byte, n, (hipStream_t)s), "hipMemsetAsync");
}
int fhip_stream_create(void** s) {
    if (!s) return set_error(FHIP_ERR_ARG, "fhip_stream_create: NULL output");
    int rc = need_init();
    if (rc) return rc;
    hipStream_t st;
    rc = check_hip(hipStreamCreateWithFlags(&st, hipStreamNonBlocking), "hipStreamCreate");
    *s = rc ? nullptr : (void*)st;
    return rc;
}
int fhip_stream_destroy(void* s) {
    if (!s) return FHIP_OK;
    release_workspace((hipStream_t)s);   // the library's buffer for this stream goes with it
    return check_hip(hipStreamDestroy((hipStream_t)s), "hipStreamDestroy");
}
int fhip_stream_sync(void* s) { return check_hip(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize"); }
int fhip_event_create(void** e) {
    if (!e) return set_error(FHIP_ERR_ARG, "fhip_event_create: NULL output");
    int rc = need_init();
    if (rc) return rc;
    hipEvent_t ev;
    rc = check_hip(hipEventCreate(&ev), "hipEventCreate");
    *e = rc ? nullptr : (void*)ev;
    return rc;
}
int fhip_event_destroy(void* e) { return e ? check_hip(hipEventDestroy((hipEvent_t)e), "hipEventDestroy") : FHIP_OK; }
int fhip_event_record(void* e, void* s) { return check_hip(hipEventRecord((hipEvent_t)e, (hipStream_t)s), "hipEventRecord"); }
int fhip_event_sync(void* e) { return check_hip(hipEventSynchronize((hipEvent_t)e), "hipEventSynchronize"); }
int fhip_event_elapsed_ms(void* a, void* b, float* ms) {
    if (!ms) return set_error(FHIP_ERR_ARG, "fhip_event_elapsed_ms: NULL output");
    return check_hip(hipEventElapsedTime(ms, (hipEvent_t)a, (hipEvent_t)b), "hipEventElapsedTime");
}

int fhip_graph_capture_begin(void* s) {
    int rc = need_init();
    if (rc) return rc;
    if (!s) return set_error(FHIP_ERR_ARG, "fhip_graph_capture_begin: needs a stream from fhip_stream_create");
    return check_hip(hipStreamBeginCapture((hipStream_t)s, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
}
int fhip_graph_capture_end(void* s, void** graph_exec) {
    if (!s || !graph_exec) return set_error(FHIP_ERR_ARG, "fhip_graph_capture_end: NULL argument");
    *graph_exec = nullptr;
    hipGraph_t g = nullptr;
    int rc = check_hip(hipStreamEndCapture((hipStream_t)s, &g), "hipStreamEndCapture");
    if (rc) return rc;
    hipGraphExec_t ge = nullptr;
    rc = check_hip(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0), "hipGraphInstantiate");
    (void)hipGraphDestroy(g);
    if (!rc) *graph_exec = (void*)ge;
    return rc;
}
int fhip_graph_launch(void* ge, void* s) {
    if (!ge) return set_error(FHIP_ERR_ARG, "fhip_graph_launch: NULL graph");
    return check_hip(hipGraphLaunch((hipGraphExec_t)ge, (hipStream_t)s), "hipGraphLaunch");
}
int fhip_graph_destroy(void* ge) { return ge ? check_hip(hipGraphExecDestroy((hipGraphExec_t)ge), "hipGraphExecDestroy") : FHIP_OK; }

// ---- weights --------------------------------------------------------------------------------

int fhip_weight_create(uint32_t ty, const uint8_t* h_raw, size_t nbytes, size_t rows, size_t cols, fhip_weight** out) {
    if (!out) return set_error(FHIP_ERR_ARG, "fhip_weight_create: NULL output");
    *out = nullptr;
    int rc = need_init();
    if (rc) return rc;
    fhip_weight w;
    if ((rc = make_weight(ty, nbytes, rows, cols, w))) return rc;
    if (nbytes && !h_raw) return set_error(FHIP_ERR_ARG, "fhip_weight_create: NULL bytes");
    void* d = nullptr;
    // slack past the stream: a wide load that starts inside the last block may end behind it
    if ((rc = check_hip(hipMalloc(&d, nbytes + WEIGHT_SLACK), "hipMalloc(weight)"))) return rc;
    if (nbytes && (rc = check_hip(hipMemcpy(d, h_raw, nbytes, hipMemcpyHostToDevice), "hipMemcpy(weight)"))) { (void)hipFree(d); return rc; }
    if ((rc = check_hip(hipMemset((uint8_t*)d + nbytes, 0, WEIGHT_SLACK), "hipMemset(weight tail)"))) { (void)hipFree(d); return rc; }
    w.d_raw = (const uint8_t*)d;
    w.owns = true;
    *out = new fhip_weight(w);
    return FHIP_OK;
}

int fhip_weight_create_parts(uint32_t ty, const uint8_t* const* h_parts, const size_t* part_bytes, size_t n_parts, size_t rows, size_t cols,
                             fhip_weight** out) {
    if (!out) return set_error(FHIP_ERR_ARG, "fhip_weight_create_parts: NULL output");
    *out = nullptr;
    int rc = need_init();
    if (rc) return rc;
    if (n_parts && (!h_parts || !part_bytes)) return set_error(FHIP_ERR_ARG, "fhip_weight_create_parts: NULL part list");
    size_t nbytes = 0;
    for (size_t i = 0; i < n_parts; i++) {
        if (part_bytes[i] && !h_parts[i]) return set_error(FHIP_ERR_ARG, "fhip_weight_create_parts: NULL bytes");
        nbytes += part_bytes[i];
    }
    fhip_weight w;
    if ((rc = make_weight(ty, nbytes, rows, cols, w))) return rc;
    void* d = nullptr;
    if ((rc = check_hip(hipMalloc(&d, nbytes + 256), "hipMalloc(weight)"))) return rc;
    size_t at = 0;
    for (size_t i = 0; i < n_parts && !rc; i++) {
        if (part_bytes[i]) rc = check_hip(hipMemcpy((uint8_t*)d + at, h_parts[i], part_bytes[i], hipMemcpyHostToDevice), "hipMemcpy(weight)");
        at += part_bytes[i];
    }
    if (!rc) rc = check_hip(hipMemset((uint8_t*)d + nbytes, 0, 256), "hipMemset(weight tail)");
    if (rc) { (void)hipFree(d); return rc; }
    w.d_raw = (const uint8_t*)d;
    w.owns = true;
    *out = new fhip_weight(w);
    return FHIP_OK;
}

int fhip_weight_wrap_device(uint32_t ty, const uint8_t* d_raw, size_t nbytes, size_t rows, size_t cols, fhip_weight** out) {
    if (!out) return set_error(FHIP_ERR_ARG, "fhip_weight_wrap_device: NULL output");
    *out = nullptr;
    int rc = need_init();
    if (rc) return rc;
    fhip_weight w;
    if ((rc = make_weight(ty, nbytes, rows, cols, w))) return rc;
    if (nbytes && !d_raw) return set_error(FHIP_ERR_ARG, "fhip_weight_wrap_device: NULL bytes");
    if (((uintptr_t)d_raw & 15) != 0) return set_error(FHIP_ERR_ARG, "fhip_weight_wrap_device: bytes must be 16-byte aligned");
    if (nbytes) {   // the allocation has to reach WEIGHT_SLACK bytes past the last block, as the library's own weights do
        hipDeviceptr_t base = nullptr;
        size_t size = 0;
        if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)d_raw) != hipSuccess) {
            (void)hipGetLastError();
            return set_error(FHIP_ERR_ARG, "fhip_weight_wrap_device: not a device allocation");
        }
        const uintptr_t end = (uintptr_t)base + size, need = (uintptr_t)d_raw + nbytes + WEIGHT_SLACK;
        if (need > end)
            return set_error(FHIP_ERR_ARG, "fhip_weight_wrap_device: the allocation must extend %zu bytes past the weight's last block "
                             "(it ends %zu bytes behind it); buffers from fhip_malloc always do", WEIGHT_SLACK, (size_t)(end - ((uintptr_t)d_raw + nbytes)));
    }
    w.d_raw = d_raw;
    w.owns = false;
    *out = new fhip_weight(w);
    return FHIP_OK;
}

void fhip_weight_destroy(fhip_weight* w) {
    if (!w) return;
    if (w->owns && w->d_raw) (void)hipFree((void*)w->d_raw);
    delete w;
}

size_t fhip_weight_rows(const fhip_weight* w) { return w ? w->rows : 0; }
size_t fhip_weight_cols(const fhip_weight* w) { return w ? w->cols : 0; }
size_t fhip_weight_nbytes(const fhip_weight* w) { return w ? w->nbytes : 0; }
uint32_t fhip_weight_type(const fhip_weight* w) { return w ? w->type : 0; }

// ---- unpackers ------------------------------------------------------------------------------

int fhip_f16_to_f32(const uint16_t* d_bits, size_t n, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (n && (!d_bits || !d_out)) return set_error(FHIP_ERR_ARG, "fhip_f16_to_f32: NULL pointer");
    return fhip::launch_f16_to_f32(d_bits, n, d_out, (hipStream_t)stream);
}

int fhip_dequant_rows(const fhip_weight* w, size_t row0, size_t nrows, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_dequant_rows: NULL weight");
    if (row0 > w->rows || nrows > w->rows - row0) return set_error(FHIP_ERR_SHAPE, "fhip_dequant_rows: rows [%zu, %zu) outside [0, %zu)", row0, row0 + nrows, w->rows);
    if (nrows == 0 || w->cols == 0) return FHIP_OK;
    if (!d_out) return set_error(FHIP_ERR_ARG, "fhip_dequant_rows: NULL output");
    size_t vals, bytes;
    block_info(w->type, vals, bytes);
    return fhip::launch_dequant(w->type, w->d_raw + row0 * w->row_bytes, nrows * (w->cols / vals), d_out, (hipStream_t)stream);
}

int fhip_deq_raw(const uint8_t* h_raw, size_t nbytes, size_t n, uint32_t ty, float* h_out, size_t* n_written) {
    int rc = need_init();
    if (rc) return rc;
    if (const size_t eb = dense_elem_bytes(ty)) {
        // lib.rs:499-501: raw[..n * size] first (a panic when the bytes are short), then exactly n values
        if (nbytes / eb < n) return set_error(FHIP_ERR_SHAPE, "range end index %zu out of range for slice of length %zu", n * eb, nbytes);
        if (n_written) *n_written = n;
        if (n == 0) return FHIP_OK;
        if (!h_raw || !h_out) return set_error(FHIP_ERR_ARG, "fhip_deq_raw: NULL pointer");
        if (ty == FHIP_F32) { memcpy(h_out, h_raw, n * 4); return FHIP_OK; }   // the bytes as they are
        void *d_in = nullptr, *d_out = nullptr;
        if ((rc = check_hip(hipMalloc(&d_in, n * 2), "hipMalloc"))) return rc;
        if ((rc = check_hip(hipMalloc(&d_out, n * sizeof(float)), "hipMalloc"))) { (void)hipFree(d_in); return rc; }
        rc = check_hip(hipMemcpy(d_in, h_raw, n * 2, hipMemcpyHostToDevice), "hipMemcpy H2D");
        if (!rc) rc = ty == FHIP_F16 ? fhip::launch_f16_to_f32((const uint16_t*)d_in, n, (float*)d_out, nullptr)
                                     : fhip::launch_bf16_to_f32((const uint16_t*)d_in, n, (float*)d_out, nullptr);
        if (!rc) rc = check_hip(hipMemcpy(h_out, d_out, n * sizeof(float), hipMemcpyDeviceToHost), "hipMemcpy D2H");
        (void)hipFree(d_in);
        (void)hipFree(d_out);
        return rc;
    }
    size_t vals, bytes;
    if (!block_info(ty, vals, bytes)) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "unsupported ggml type %u", ty);
    if (n && !h_out) return set_error(FHIP_ERR_ARG, "fhip_deq_raw: NULL output");
    size_t nb = n / vals;
    if (nbytes / bytes < nb) nb = nbytes / bytes;  // chunks_exact(..).take(n / blk)
    if (nb && !h_raw) return set_error(FHIP_ERR_ARG, "fhip_deq_raw: NULL bytes");
    // Every dequantizer but Q8_0's pre-sizes the output to n zeros (lib.rs:619, :634, :651, :670, :693, :722, :794); Q8_0
    // pushes whole blocks only and so returns a shorter vector (lib.rs:609-614).
    size_t produced = ty == FHIP_Q8_0 ? nb * vals : n;
    if (n_written) *n_written = produced;
    if (nb) {
        void *d_in = nullptr, *d_out = nullptr;
        if ((rc = check_hip(hipMalloc(&d_in, nb * bytes), "hipMalloc"))) return rc;
        if ((rc = check_hip(hipMalloc(&d_out, nb * vals * sizeof(float)), "hipMalloc"))) { (void)hipFree(d_in); return rc; }
        rc = check_hip(hipMemcpy(d_in, h_raw, nb * bytes, hipMemcpyHostToDevice), "hipMemcpy H2D");
        if (!rc) rc = fhip::launch_dequant(ty, (const uint8_t*)d_in, nb, (float*)d_out, nullptr);
        if (!rc) rc = check_hip(hipMemcpy(h_out, d_out, nb * vals * sizeof(float), hipMemcpyDeviceToHost), "hipMemcpy D2H");
        (void)hipFree(d_in);
        (void)hipFree(d_out);
        if (rc) return rc;
    }
    for (size_t i = nb * vals; i < produced; i++) h_out[i] = 0.0f;
    return FHIP_OK;
}

// ---- matmuls --------------------------------------------------------------------------------

int fhip_matmul_q(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_matmul_q: NULL weight");
    if (rows_x == 0 || w->rows == 0) return FHIP_OK;
    if (!d_x || !d_y) return set_error(FHIP_ERR_ARG, "fhip_matmul_q: NULL pointer");
    if (((uintptr_t)d_x & 15) != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q: x must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    if (!takes_f16x2(w, rows_x)) return fhip::launch_gemv(w, d_x, rows_x, d_y, 0, s);
    const size_t grp = f16x2_group(w);
    void* ws = nullptr;
    if ((rc = lib_workspace(s, f16x2_matmul_ws(w, rows_x < grp ? rows_x : grp), &ws, "fhip_matmul_q"))) return rc;
    for (size_t m0 = 0; m0 < rows_x; m0 += grp) {
        const size_t t = rows_x - m0 < grp ? rows_x - m0 : grp;
        if (takes_f16x2(w, t)) rc = f16x2_matmul(w, d_x + m0 * w->cols, t, false, d_y + m0 * w->rows, ws, s);
        else rc = fhip::launch_gemv(w, d_x + m0 * w->cols, t, d_y + m0 * w->rows, 0, s);   // a last group of one or two rows
        if (rc) return rc;
    }
    return FHIP_OK;
}

int fhip_matmul_q_swiglu(const fhip_weight* gu, const float* d_x, size_t rows_x, float* d_y, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!gu) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_swiglu: NULL weight");
    if (gu->type == FHIP_Q8_0) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "try_matmul_swiglu: no fused kernel for Q8_0");
    if (gu->rows % 2 != 0) return set_error(FHIP_ERR_SHAPE, "matmul_swiglu: gate_up rows must be even");
    if (rows_x == 0 || gu->rows == 0) return FHIP_OK;
    if (!d_x || !d_y) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_swiglu: NULL pointer");
    if (((uintptr_t)d_x & 15) != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_swiglu: x must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const size_t n_ff = gu->rows / 2;
    if (!takes_f16x2(gu, rows_x) || swiglu_takes_quad(gu, rows_x)) return fhip::launch_gemv(gu, d_x, rows_x, d_y, n_ff, s);
    // gate|up for the group in one pass into the workspace, then the reference's un-fused SwiGLU over it
    const size_t grp = f16x2_group(gu), t0 = rows_x < grp ? rows_x : grp;
    const size_t mm = f16x2_matmul_ws(gu, t0);
    void* ws = nullptr;
    if ((rc = lib_workspace(s, mm + align256(t0 * gu->rows * sizeof(float)), &ws, "fhip_matmul_q_swiglu"))) return rc;
    float* g = (float*)((uint8_t*)ws + mm);
    for (size_t m0 = 0; m0 < rows_x; m0 += grp) {
        const size_t t = rows_x - m0 < grp ? rows_x - m0 : grp;
        if (!takes_f16x2(gu, t) || swiglu_takes_quad(gu, t)) { rc = fhip::launch_gemv(gu, d_x + m0 * gu->cols, t, d_y + m0 * n_ff, n_ff, s); }
        else if (!(rc = f16x2_matmul(gu, d_x + m0 * gu->cols, t, false, g, ws, s))) rc = fhip::launch_swiglu(g, t, n_ff, d_y + m0 * n_ff, s);
        if (rc) return rc;
    }
    return FHIP_OK;
}

int fhip_swiglu(const float* d_gu, size_t t, size_t d, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (t * d == 0) return FHIP_OK;
    if (!d_gu || !d_out) return set_error(FHIP_ERR_ARG, "fhip_swiglu: NULL pointer");
    return fhip::launch_swiglu(d_gu, t, d, d_out, (hipStream_t)stream);
}

int fhip_ffn(const fhip_weight* gu, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y, float* d_ws, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!gu || !down) return set_error(FHIP_ERR_ARG, "fhip_ffn: NULL weight");
    if (gu->rows % 2 != 0) return set_error(FHIP_ERR_SHAPE, "ffn: gate_up rows must be even");
    size_t n_ff = gu->rows / 2;
    // crates/ferric-tensor/src/dtype.rs:979-981: down in dim must equal n_ff, down out dim is the model width.
    if (down->cols != n_ff) return set_error(FHIP_ERR_SHAPE, "down in dim must equal n_ff");
    if (rows_x == 0) return FHIP_OK;
    if (!d_x || !d_y || !d_ws) return set_error(FHIP_ERR_ARG, "fhip_ffn: NULL pointer");
    if (gu->type == FHIP_Q8_0) {
        // no fused gate/up kernel for this format: matmul_q then swiglu, as the reference's callers
        // do when try_matmul_swiglu returns None (crates/ferric-llama/src/qwen3.rs:219-227). The
        // [rows_x, 2 n_ff] intermediate then also lives in d_ws, which this path needs 3x larger.
        return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "fhip_ffn: gate_up must be Q4_K or Q6_K");
    }
    hipStream_t s = (hipStream_t)stream;
    size_t grp = f16x2_group(gu) < f16x2_group(down) ? f16x2_group(gu) : f16x2_group(down);
    const size_t t0 = rows_x < grp ? rows_x : grp;
    if (ffn_direct(gu, down, t0)) {
        if ((rc = fhip::launch_gemv(gu, d_x, rows_x, d_ws, n_ff, s))) return rc;
        return fhip::launch_gemv(down, d_ws, rows_x, d_y, 0, s);
    }
    // groups of up to 32 rows, each one pass over gate|up and one over down; SwiGLU happens while the rows are prepared
    // for the down projection. The intermediates live in the library's workspace; d_ws is left alone.
    const size_t mm1 = f16x2_matmul_ws(gu, t0), gb = align256(t0 * gu->rows * sizeof(float));
    void* ws = nullptr;
    if ((rc = lib_workspace(s, mm1 + gb + f16x2_matmul_ws(down, t0), &ws, "fhip_ffn"))) return rc;
    float* g = (float*)((uint8_t*)ws + mm1);
    void* ws2 = (uint8_t*)ws + mm1 + gb;
    for (size_t m0 = 0; m0 < rows_x; m0 += grp) {
        const size_t t = rows_x - m0 < grp ? rows_x - m0 : grp;
        if (ffn_direct(gu, down, t)) {
            if ((rc = fhip::launch_gemv(gu, d_x + m0 * gu->cols, t, d_ws + m0 * n_ff, n_ff, s))) return rc;
            rc = fhip::launch_gemv(down, d_ws + m0 * n_ff, t, d_y + m0 * down->rows, 0, s);
        } else if (swiglu_takes_quad(gu, t)) {
            // three or four rows: silu(gate) * up straight out of the mat-vec, then the down projection's one pass over it
            if (!(rc = fhip::launch_gemv(gu, d_x + m0 * gu->cols, t, g, n_ff, s)))
                rc = f16x2_matmul(down, g, t, false, d_y + m0 * down->rows, ws2, s);
        } else {
            // under the ordered policy gate|up's K-split groups stay partial sums; the split for the down projection adds them
            fhip::F16Parts parts{nullptr, 0, 0, 0, 0, 128};
            if (!(rc = f16x2_matmul(gu, d_x + m0 * gu->cols, t, false, g, ws, s, &parts)))
                rc = f16x2_matmul(down, g, t, true, d_y + m0 * down->rows, ws2, s, nullptr, &parts);
        }
        if (rc) return rc;
    }
    return FHIP_OK;
}

int fhip_ffn_noalloc(const fhip_weight* gu, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!gu || !down) return set_error(FHIP_ERR_ARG, "fhip_ffn_noalloc: NULL weight");
    if (gu->rows % 2 != 0) return set_error(FHIP_ERR_SHAPE, "ffn: gate_up rows must be even");
    const size_t n_ff = gu->rows / 2;
    if (down->cols != n_ff) return set_error(FHIP_ERR_SHAPE, "down in dim must equal n_ff");
    if (rows_x == 0) return FHIP_OK;
    if (!d_x || !d_y) return set_error(FHIP_ERR_ARG, "fhip_ffn_noalloc: NULL pointer");
    if (gu->type == FHIP_Q8_0) return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "fhip_ffn_noalloc: gate_up must be Q4_K or Q6_K");
    if (rows_x > NOALLOC_FLOATS / (n_ff ? n_ff : 1))
        return set_error(FHIP_ERR_SHAPE, "fhip_ffn_noalloc: rows_x * n_ff = %zu * %zu floats do not fit the built-in scratch of %zu floats; use fhip_ffn",
                         rows_x, n_ff, NOALLOC_FLOATS);
    float* h = g_device < MAX_DEVICES ? g_scratch_ptr[g_device] : nullptr;
    if (!h) return set_error(FHIP_ERR_HIP, "fhip_ffn_noalloc: no scratch address for device %d", g_device);
    // the mat-vec kernels for every batch width (they need nothing beside operands and this intermediate; the one-pass
    // kernels of fhip_ffn would need the library's workspace); every element of h is written before it is read
    hipStream_t s = (hipStream_t)stream;
    if ((rc = fhip::launch_gemv(gu, d_x, rows_x, h, n_ff, s))) return rc;
    return fhip::launch_gemv(down, h, rows_x, d_y, 0, s);
}

static bool known_policy(int policy) { return policy == FHIP_BATCH_AUTO || policy == FHIP_BATCH_F32_MATVEC || policy == FHIP_BATCH_ORDERED; }

int fhip_batch_policy(int policy) {
    const int before = g_default_batch_policy;
    if (known_policy(policy)) g_default_batch_policy = policy;
    return before;
}

int fhip_weight_batch_policy(fhip_weight* w, int policy) {
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_weight_batch_policy: NULL weight");
    const int before = w->batch_policy;
    if (known_policy(policy)) w->batch_policy = policy;
    return before;
}

int fhip_weight_matvec_precision(fhip_weight* w, int bits) {
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_weight_matvec_precision: NULL weight");
    const int before = w->planes == 3 ? 24 : 16;
    if (bits == 0) return before;
    if (bits != 16 && bits != 24) return set_error(FHIP_ERR_ARG, "fhip_weight_matvec_precision: 16 or 24 bits (0 to query), not %d", bits);
    w->planes = bits == 24 ? 3 : 2;
    return before;
}

int fhip_workspace_reserve(void* stream, size_t nbytes) {
    int rc = need_init();
    if (rc) return rc;
    void* p = nullptr;
    return nbytes ? lib_workspace((hipStream_t)stream, nbytes, &p, "fhip_workspace_reserve") : FHIP_OK;
}

size_t fhip_workspace_bytes(const fhip_weight* gu, const fhip_weight* down, size_t rows_x) {
    // what fhip_matmul_q (down == NULL), fhip_matmul_q_swiglu (down == NULL) or fhip_ffn asks of the workspace: the largest
    size_t need = 0;
    if (!gu || rows_x == 0) return 0;
    if (down) {      // fhip_ffn: [gate|up's workspace][the t0 x 2 n_ff intermediate][down's workspace], t0 the widest group
        const size_t grp = f16x2_group(gu) < f16x2_group(down) ? f16x2_group(gu) : f16x2_group(down);
        const size_t t0 = rows_x < grp ? rows_x : grp;
        if (ffn_direct(gu, down, t0)) return 0;
        return f16x2_matmul_ws(gu, t0) + align256(t0 * gu->rows * sizeof(float)) + f16x2_matmul_ws(down, t0);
    }
    if (takes_f16x2(gu, rows_x)) {
        const size_t t0 = rows_x < f16x2_group(gu) ? rows_x : f16x2_group(gu);
        need = f16x2_matmul_ws(gu, t0) + align256(t0 * gu->rows * sizeof(float));
    }
    return need;
}

size_t fhip_workspace_bytes_coop(const fhip_weight* w, const fhip_weight* down, size_t rows_x) {
    const size_t a = fhip::gemm_bf16_ws_bytes(w, rows_x), b = fhip::gemm_bf16_ws_bytes(down, rows_x);
    return a > b ? a : b;
}

void fhip_workspace_release(void* stream) { release_workspace((hipStream_t)stream); }

int fhip_gemm_q_bf16(const fhip_weight* w, const uint16_t* d_x, size_t t, float* d_y, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_gemm_q_bf16: NULL weight");
    if (t == 0 || w->rows == 0) return FHIP_OK;
    if (!d_y || (!d_x && w->cols)) return set_error(FHIP_ERR_ARG, "fhip_gemm_q_bf16: NULL pointer");
    if (w->cols == 0) return zero_outputs(t, w->rows, d_y, (hipStream_t)stream);   // empty inner dimension: every dot product is 0
    return gemm_bf16_lib_ws(w, d_x, t, d_y, (hipStream_t)stream, "fhip_gemm_q_bf16");
}

// ---- mixture-of-experts entry points (crates/ferric-tensor/src/dtype.rs:1582-1780) ----------------------

// ---- decode-layer steps --------------------------------------------------------------------------

int fhip_rmsnorm(const float* d_x, const float* d_weight, size_t rows, size_t d, float eps, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (rows == 0 || d == 0) return FHIP_OK;
    if (!d_x || !d_weight || !d_out) return set_error(FHIP_ERR_ARG, "fhip_rmsnorm: NULL pointer");
    return fhip::launch_rmsnorm(d_x, nullptr, d_weight, rows, d, eps, nullptr, d_out, (hipStream_t)stream);
}

int fhip_add_rmsnorm(const float* d_a, const float* d_b, const float* d_weight, size_t rows, size_t d, float eps, float* d_sum,
                     float* d_norm, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (rows == 0 || d == 0) return FHIP_OK;
    if (!d_a || !d_b || !d_weight || !d_sum || !d_norm) return set_error(FHIP_ERR_ARG, "fhip_add_rmsnorm: NULL pointer");
    return fhip::launch_rmsnorm(d_a, d_b, d_weight, rows, d, eps, d_sum, d_norm, (hipStream_t)stream);
}

int fhip_add(const float* d_a, const float* d_b, size_t n, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (n == 0) return FHIP_OK;
    if (!d_a || !d_b || !d_out) return set_error(FHIP_ERR_ARG, "fhip_add: NULL pointer");
    return fhip::launch_add(d_a, d_b, n, d_out, (hipStream_t)stream);
}

int fhip_mul_sigmoid(const float* d_a, const float* d_g, size_t n, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (n == 0) return FHIP_OK;
    if (!d_a || !d_g || !d_out) return set_error(FHIP_ERR_ARG, "fhip_mul_sigmoid: NULL pointer");
    return fhip::launch_mul_sigmoid(d_a, d_g, n, d_out, (hipStream_t)stream);
}

int fhip_geglu(const float* d_gu, size_t t, size_t d, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (t * d == 0) return FHIP_OK;
    if (!d_gu || !d_out) return set_error(FHIP_ERR_ARG, "fhip_geglu: NULL pointer");
    return fhip::launch_geglu(d_gu, t, d, d_out, (hipStream_t)stream);
}

static int kvq_checks(const char* who, int fmt, size_t width) {
    if (fmt != FHIP_KVQ_Q8_0 && fmt != FHIP_KVQ_Q4_0 && fmt != FHIP_KVQ_Q4_1) return set_error(FHIP_ERR_ARG, "%s: unknown format %d", who, fmt);
    // crates/ferric-tensor/src/kvquant.rs:470
    if (width % 32 != 0) return set_error(FHIP_ERR_SHAPE, "QKvCache row width %zu must be a multiple of 32", width);
    return FHIP_OK;
}

int fhip_kvq_sizes(int fmt, size_t rows, size_t width, size_t* code_words, size_t* scale_words) {
    int rc = kvq_checks("fhip_kvq_sizes", fmt, width);
    if (rc) return rc;
    const size_t nblk = rows * (width / 32);
    if (code_words) *code_words = nblk * (fmt == FHIP_KVQ_Q8_0 ? 8 : 4);
    if (scale_words) *scale_words = fmt == FHIP_KVQ_Q4_1 ? nblk : (nblk + 1) / 2;
    return FHIP_OK;
}

int fhip_kvq_append(int fmt, const float* d_src, size_t src_row_stride, size_t t, size_t width, const uint32_t* d_positions, uint32_t pos_off,
                    int src_at_pos, size_t cap, uint32_t* d_codes, uint32_t* d_scales, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = kvq_checks("fhip_kvq_append", fmt, width))) return rc;
    if (t == 0 || width == 0) return FHIP_OK;
    if (!d_src || !d_codes || !d_scales) return set_error(FHIP_ERR_ARG, "fhip_kvq_append: NULL pointer");
    if (src_row_stride == 0) src_row_stride = width;
    if (src_row_stride < width) return set_error(FHIP_ERR_SHAPE, "fhip_kvq_append: source row stride %zu below the width %zu", src_row_stride, width);
    if (!d_positions && (size_t)pos_off + t > cap)
        return set_error(FHIP_ERR_SHAPE, "fhip_kvq_append: rows %u + %zu exceed the capacity %zu", pos_off, t, cap);
    return fhip::launch_kvq_append(fmt, d_src, src_row_stride, t, width, d_positions, pos_off, src_at_pos != 0, cap, d_codes, (uint16_t*)d_scales,
                                   (hipStream_t)stream);
}

int fhip_kvq_dequantize_rows(int fmt, const uint32_t* d_codes, const uint32_t* d_scales, size_t row0, size_t rows, size_t width,
                             const uint32_t* d_last_pos, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = kvq_checks("fhip_kvq_dequantize_rows", fmt, width))) return rc;
    if (rows == 0 || width == 0) return FHIP_OK;
    if (!d_codes || !d_scales || !d_out) return set_error(FHIP_ERR_ARG, "fhip_kvq_dequantize_rows: NULL pointer");
    if (((uintptr_t)d_out & 15) != 0) return set_error(FHIP_ERR_ARG, "fhip_kvq_dequantize_rows: the output must be 16-byte aligned");
    return fhip::launch_kvq_dequantize(fmt, d_codes, (const uint16_t*)d_scales, row0, rows, width, d_last_pos, d_out, (hipStream_t)stream);
}

static int rope_checks(const char* who, size_t n_heads, size_t head_dim, size_t n_rot) {
    if (n_rot > head_dim || n_rot % 2 != 0) return set_error(FHIP_ERR_SHAPE, "n_rot must be even and <= head_dim");   // lib.rs:437
    if (n_heads > 0xFFFFu || head_dim > 0xFFFFu) return set_error(FHIP_ERR_SHAPE, "%s: n_heads / head_dim exceed 65535", who);
    return FHIP_OK;
}

int fhip_rope(const float* d_x, size_t src_row_stride, size_t t, size_t n_heads, size_t head_dim, size_t n_rot, float base,
              const uint32_t* d_positions, uint32_t pos_off, const float* d_freq_scale, int interleaved, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = rope_checks("fhip_rope", n_heads, head_dim, n_rot))) return rc;
    if (t == 0 || n_heads == 0 || head_dim == 0) return FHIP_OK;
    if (!d_x || !d_out) return set_error(FHIP_ERR_ARG, "fhip_rope: NULL pointer");
    if (src_row_stride == 0) src_row_stride = n_heads * head_dim;
    return fhip::launch_rope(d_x, src_row_stride, t, (int)n_heads, (int)head_dim, (int)n_rot, base, d_positions, pos_off, d_freq_scale,
                             interleaved != 0, d_out, (hipStream_t)stream);
}

int fhip_kv_append2(const float* d_k, const float* d_v, size_t t, size_t width, const uint32_t* d_positions, uint32_t pos_off,
                    float* d_k_cache, float* d_v_cache, size_t cap, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (t == 0 || width == 0) return FHIP_OK;
    if (!d_k || !d_v || !d_k_cache || !d_v_cache) return set_error(FHIP_ERR_ARG, "fhip_kv_append2: NULL pointer");
    if (cap > 0xFFFFFFFFull) return set_error(FHIP_ERR_SHAPE, "fhip_kv_append2: capacity exceeds 2^32 rows");
    return fhip::launch_kv_append(d_k, d_v, t, width, d_positions, pos_off, cap, d_k_cache, d_v_cache, (hipStream_t)stream);
}

int fhip_qkv_post(const float* d_qkv, const float* d_bias, const float* d_q_norm, const float* d_k_norm, const uint32_t* d_positions,
                  const float* d_freq_scale, size_t t, size_t n_head, size_t n_kv, size_t head_dim, size_t n_rot, int interleaved,
                  float eps, float base, float* d_q_out, float* d_k_cache, float* d_v_cache, size_t cap, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = rope_checks("fhip_qkv_post", n_head + 2 * n_kv, head_dim, n_rot))) return rc;
    if (t == 0 || head_dim == 0 || n_head + n_kv == 0) return FHIP_OK;
    if (!d_qkv || !d_positions || !d_q_out || !d_k_cache || !d_v_cache) return set_error(FHIP_ERR_ARG, "fhip_qkv_post: NULL pointer");
    if (cap > 0xFFFFFFFFull) return set_error(FHIP_ERR_SHAPE, "fhip_qkv_post: capacity exceeds 2^32 rows");
    return fhip::launch_qkv_post(d_qkv, d_bias, d_q_norm, d_k_norm, d_positions, d_freq_scale, t, (int)n_head, (int)n_kv, (int)head_dim,
                                 (int)n_rot, interleaved != 0, eps, base, d_q_out, d_k_cache, d_v_cache, cap, (hipStream_t)stream);
}

int fhip_qkv_post_packed(const float* d_qkv, const float* d_bias, const float* d_q_norm, const float* d_k_norm, const uint32_t* d_positions,
                         const float* d_freq_scale, size_t t, size_t n_head, size_t n_kv, size_t head_dim, size_t n_rot, int interleaved,
                         float eps, float base, float* d_q_out, float* d_k_out, float* d_v_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = rope_checks("fhip_qkv_post_packed", n_head + 2 * n_kv, head_dim, n_rot))) return rc;
    if (t == 0 || head_dim == 0 || n_head + n_kv == 0) return FHIP_OK;
    if (!d_qkv || !d_positions || !d_q_out || !d_k_out || !d_v_out) return set_error(FHIP_ERR_ARG, "fhip_qkv_post_packed: NULL pointer");
    return fhip::launch_qkv_post(d_qkv, d_bias, d_q_norm, d_k_norm, d_positions, d_freq_scale, t, (int)n_head, (int)n_kv, (int)head_dim,
                                 (int)n_rot, interleaved != 0, eps, base, d_q_out, d_k_out, d_v_out, 0, (hipStream_t)stream, true);
}

int fhip_kvq_append2(int fmt, const float* d_k, const float* d_v, size_t src_row_stride, size_t t, size_t width, const uint32_t* d_positions,
                     uint32_t pos_off, size_t cap, uint32_t* d_k_codes, uint32_t* d_k_scales, uint32_t* d_v_codes, uint32_t* d_v_scales,
                     void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = kvq_checks("fhip_kvq_append2", fmt, width))) return rc;
    if (t == 0 || width == 0) return FHIP_OK;
    if (!d_k || !d_v || !d_k_codes || !d_k_scales || !d_v_codes || !d_v_scales) return set_error(FHIP_ERR_ARG, "fhip_kvq_append2: NULL pointer");
    if (src_row_stride == 0) src_row_stride = width;
    if (src_row_stride < width) return set_error(FHIP_ERR_SHAPE, "fhip_kvq_append2: source row stride %zu below the width %zu", src_row_stride, width);
    if (!d_positions && (size_t)pos_off + t > cap)
        return set_error(FHIP_ERR_SHAPE, "fhip_kvq_append2: rows %u + %zu exceed the capacity %zu", pos_off, t, cap);
    return fhip::launch_kvq_append(fmt, d_k, src_row_stride, t, width, d_positions, pos_off, false, cap, d_k_codes, (uint16_t*)d_k_scales,
                                   (hipStream_t)stream, d_v, d_v_codes, (uint16_t*)d_v_scales);
}

int fhip_decode_attention_kvq(int fmt, const float* d_q, const uint32_t* d_k_codes, const uint32_t* d_k_scales, const uint32_t* d_v_codes,
                              const uint32_t* d_v_scales, size_t n_head, size_t n_kv, size_t head_dim, size_t len, const uint32_t* d_last_pos,
                              size_t window, float softcap, float* d_ws, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = kvq_checks("fhip_decode_attention_kvq", fmt, n_kv * head_dim))) return rc;
    if (n_head == 0 || head_dim == 0) return FHIP_OK;
    if (!d_q || !d_k_codes || !d_k_scales || !d_v_codes || !d_v_scales || !d_out)
        return set_error(FHIP_ERR_ARG, "fhip_decode_attention_kvq: NULL pointer");
    if (n_head > 0x7FFFFFFFull || n_kv > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "fhip_decode_attention_kvq: too many heads");
    return fhip::launch_decode_attention_kvq(fmt, d_q, d_k_codes, (const uint16_t*)d_k_scales, d_v_codes, (const uint16_t*)d_v_scales, (int)n_head,
                                             (int)n_kv, (int)head_dim, len, d_last_pos, window, softcap, d_ws, d_out, (hipStream_t)stream);
}

int fhip_causal_attention(const float* d_q, const float* d_k, const float* d_v, size_t t, size_t s, size_t n_head, size_t n_kv, size_t head_dim,
                          size_t window, float softcap, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (t == 0 || n_head == 0 || head_dim == 0) return FHIP_OK;
    if (!d_q || !d_k || !d_v || !d_out) return set_error(FHIP_ERR_ARG, "fhip_causal_attention: NULL pointer");
    if ((((uintptr_t)d_q | (uintptr_t)d_k | (uintptr_t)d_v | (uintptr_t)d_out) & 15) != 0)
        return set_error(FHIP_ERR_ARG, "fhip_causal_attention: pointers must be 16-byte aligned");
    if (n_head > 0x7FFFFFFFull || n_kv > 0x7FFFFFFFull) return set_error(FHIP_ERR_SHAPE, "fhip_causal_attention: too many heads");
    return fhip::launch_causal_attention(d_q, d_k, d_v, t, s, (int)n_head, (int)n_kv, (int)head_dim, window, softcap, d_out, (hipStream_t)stream);
}

size_t fhip_decode_attention_ws_bytes(size_t n_head, size_t n_kv, size_t head_dim, size_t len) {
    if (g_device < 0 || n_kv == 0 || len == 0) return 0;
    int splits = fhip::attn_ws_splits(len, (int)n_head, (int)n_kv);
    return splits > 1 ? n_head * (size_t)splits * (head_dim + 2) * sizeof(float) : 0;
}

int fhip_decode_attention_ex(const float* d_q, const float* d_k_cache, const float* d_v_cache, size_t n_head, size_t n_kv, size_t head_dim,
                             size_t len, const uint32_t* d_last_pos, size_t window, float softcap, float* d_ws, float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (n_head > 0xFFFFu || n_kv > 0xFFFFu || head_dim > 0xFFFFu) return set_error(FHIP_ERR_SHAPE, "fhip_decode_attention: head counts exceed 65535");
    if (n_head == 0 || head_dim == 0) return FHIP_OK;
    if (!d_q || !d_k_cache || !d_v_cache || !d_out) return set_error(FHIP_ERR_ARG, "fhip_decode_attention: NULL pointer");
    if (!(softcap >= 0.f)) return set_error(FHIP_ERR_ARG, "fhip_decode_attention: softcap must be >= 0");
    return fhip::launch_decode_attention(d_q, d_k_cache, d_v_cache, (int)n_head, (int)n_kv, (int)head_dim, len, d_last_pos, window, softcap, d_ws,
                                         d_out, (hipStream_t)stream);
}

int fhip_decode_attention(const float* d_q, const float* d_k_cache, const float* d_v_cache, size_t n_head, size_t n_kv, size_t head_dim,
                          size_t len, const uint32_t* d_last_pos, float* d_ws, float* d_out, void* stream) {
    return fhip_decode_attention_ex(d_q, d_k_cache, d_v_cache, n_head, n_kv, head_dim, len, d_last_pos, 0, 0.f, d_ws, d_out, stream);
}

int fhip_qkv_post_attention(const float* d_qkv, const float* d_bias, const float* d_q_norm, const float* d_k_norm, const uint32_t* d_pos,
                            const float* d_freq_scale, size_t n_head, size_t n_kv, size_t head_dim, size_t n_rot, int interleaved, float eps,
                            float base, float* d_k_cache, float* d_v_cache, size_t cap, size_t len, size_t window, float softcap, float* d_ws,
                            float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if ((rc = rope_checks("fhip_qkv_post_attention", n_head + 2 * n_kv, head_dim, n_rot))) return rc;
    if (n_head == 0 || head_dim == 0) return FHIP_OK;
    if (!d_qkv || !d_pos || !d_k_cache || !d_v_cache || !d_out) return set_error(FHIP_ERR_ARG, "fhip_qkv_post_attention: NULL pointer");
    if (cap > 0xFFFFFFFFull) return set_error(FHIP_ERR_SHAPE, "fhip_qkv_post_attention: capacity exceeds 2^32 rows");
    if (!(softcap >= 0.f)) return set_error(FHIP_ERR_ARG, "fhip_qkv_post_attention: softcap must be >= 0");
    return fhip::launch_qkv_post_attention(d_qkv, d_bias, d_q_norm, d_k_norm, d_pos, d_freq_scale, (int)n_head, (int)n_kv, (int)head_dim, (int)n_rot,
                                           interleaved != 0, eps, base, d_k_cache, d_v_cache, cap, len, window, softcap, d_ws, d_out,
                                           (hipStream_t)stream);
}

int fhip_norm_matmul_q(const fhip_weight* w, const float* d_x, const float* d_resid, const float* d_norm_w, float eps, float* d_x_out,
                       float* d_h_scratch, int swiglu, float* d_y, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!w || !d_x || !d_norm_w || !d_h_scratch || !d_y) return set_error(FHIP_ERR_ARG, "fhip_norm_matmul_q: NULL pointer");
    // every workgroup reads all of x and resid while one of them stores x_out, and all of them store y: none of the outputs
    // may share memory with an input or with each other
    {
        const size_t out_rows = swiglu ? w->rows / 2 : w->rows;
        auto overlap = [](const float* a, size_t na, const float* b, size_t nb) { return a && b && a < b + nb && b < a + na; };
        if (overlap(d_x_out, w->cols, d_x, w->cols) || overlap(d_x_out, w->cols, d_resid, w->cols) || overlap(d_x_out, w->cols, d_norm_w, w->cols))
            return set_error(FHIP_ERR_ARG, "fhip_norm_matmul_q: x_out must not overlap x, resid or norm_w");
        if (overlap(d_y, out_rows, d_x, w->cols) || overlap(d_y, out_rows, d_resid, w->cols) || overlap(d_y, out_rows, d_norm_w, w->cols) ||
            overlap(d_y, out_rows, d_x_out, w->cols))
            return set_error(FHIP_ERR_ARG, "fhip_norm_matmul_q: y must not overlap x, resid, norm_w or x_out");
    }
    if (swiglu && (w->type == FHIP_Q8_0 || w->rows % 2 != 0))
        return set_error(w->type == FHIP_Q8_0 ? FHIP_ERR_UNSUPPORTED_TYPE : FHIP_ERR_SHAPE, "fhip_norm_matmul_q: no fused SwiGLU for this weight");
    if (((uintptr_t)d_x | (uintptr_t)d_resid | (uintptr_t)d_norm_w | (uintptr_t)d_x_out) & 15)
        return set_error(FHIP_ERR_ARG, "fhip_norm_matmul_q: x, resid, norm_w and x_out must be 16-byte aligned");
    const size_t n_ff = swiglu ? w->rows / 2 : 0;
    fhip::NormParams np{d_norm_w, d_resid, d_resid ? d_x_out : nullptr, eps};   // without a residual there is no sum to store
    rc = fhip::launch_gemv_norm(w, d_x, d_y, n_ff, np, (hipStream_t)stream);
    if (rc != fhip::NORM_NOT_FUSED) return rc;
    if ((rc = fhip::launch_rmsnorm(d_x, d_resid, d_norm_w, 1, w->cols, eps, d_resid ? d_x_out : nullptr, d_h_scratch, (hipStream_t)stream))) return rc;
    return fhip::launch_gemv(w, d_h_scratch, 1, d_y, n_ff, (hipStream_t)stream);
}

int fhip_debug_generic_matvec(int on) {
    fhip::gemv_force_generic(on != 0);
    return FHIP_OK;
}

int fhip_debug_gemm_tile(int tile) { return fhip::gemm_bf16_force_tile(tile); }

int fhip_debug_quad_matvec(int on) { return fhip::gemv_quad_matvec(on != 0) ? 1 : 0; }

int fhip_debug_read_probe(const void* d_src, size_t nbytes, uint32_t* d_sink, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!d_src || !d_sink) return set_error(FHIP_ERR_ARG, "fhip_debug_read_probe: NULL pointer");
    if (((uintptr_t)d_src & 15) != 0) return set_error(FHIP_ERR_ARG, "fhip_debug_read_probe: src must be 16-byte aligned");
    return fhip::launch_read_probe(d_src, nbytes, d_sink, (hipStream_t)stream);
}

int fhip_debug_mfma_probe(int iters, float* d_sink, double* flops, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (iters < 1 || !d_sink) return set_error(FHIP_ERR_ARG, "fhip_debug_mfma_probe: iters >= 1 and a sink are needed");
    return fhip::launch_mfma_probe(iters, d_sink, (hipStream_t)stream, flops);
}

int fhip_debug_matmul_q_loop(const fhip_weight* const* ws, size_t n_weights, size_t launches, const float* d_x, int swiglu, float* d_y,
                             void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!ws || n_weights == 0 || !d_x || !d_y) return set_error(FHIP_ERR_ARG, "fhip_debug_matmul_q_loop: NULL pointer");
    for (size_t i = 0; i < launches; i++) {
        const fhip_weight* w = ws[i % n_weights];
        rc = swiglu ? fhip_matmul_q_swiglu(w, d_x, 1, d_y, stream) : fhip_matmul_q(w, d_x, 1, d_y, stream);
        if (rc) return rc;
    }
    return FHIP_OK;
}

int fhip_matvec_precision(int bits) {
    const int before = g_default_planes == 3 ? 24 : 16;
    if (bits == 0) return before;
    if (bits != 16 && bits != 24) return set_error(FHIP_ERR_ARG, "fhip_matvec_precision: 16 or 24 bits (0 to query), not %d", bits);
    g_default_planes = bits == 24 ? 3 : 2;
    return before;
}

int fhip_u32_add(uint32_t* d_words, size_t n, uint32_t delta, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (n == 0) return FHIP_OK;
    if (!d_words) return set_error(FHIP_ERR_ARG, "fhip_u32_add: NULL pointer");
    return fhip::launch_u32_add(d_words, n, delta, (hipStream_t)stream);
}

int fhip_moe_topk(const float* d_logits, const float* d_bias, size_t t, size_t n_expert, size_t k, int sigmoid, float scale, int norm,
                  float* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (k < 1 || k > 8) return set_error(FHIP_ERR_SHAPE, "k must be 1..=8");                                   // dtype.rs:1599
    if (n_expert > 1024) return set_error(FHIP_ERR_SHAPE, "moe_topk: n_expert <= 1024 (single-thread scan)");   // dtype.rs:1600
    if (n_expert == 0) return set_error(FHIP_ERR_SHAPE, "moe_topk: n_expert must be positive");
    if (t == 0) return FHIP_OK;
    if (!d_logits || !d_out) return set_error(FHIP_ERR_ARG, "fhip_moe_topk: NULL pointer");
    return fhip::launch_moe_topk(d_logits, d_bias, t, n_expert, (int)k, sigmoid != 0, scale, norm != 0, d_out, (hipStream_t)stream);
}

static int sel_checks(const char* who, const fhip_weight* w, size_t k, size_t expert_rows, fhip::SelParams* sel) {
    if (!w) return set_error(FHIP_ERR_ARG, "%s: NULL weight", who);
    if (k < 1 || k > 8) return set_error(FHIP_ERR_SHAPE, "k must be 1..=8");
    if (expert_rows == 0 || w->rows % expert_rows != 0)
        return set_error(FHIP_ERR_SHAPE, "%s: weight rows %zu are not a whole number of experts of %zu rows", who, w->rows, expert_rows);
    sel->k = (int)k;
    sel->n_expert = (int)(w->rows / expert_rows);
    sel->expert_rows = expert_rows;
    return FHIP_OK;
}

int fhip_matmul_q_swiglu_id(const fhip_weight* w, const float* d_x, size_t t, const float* d_selw, size_t k, size_t eff, float* d_y,
                            void* stream) {
    int rc = need_init();
    if (rc) return rc;
    fhip::SelParams sel{};
    if ((rc = sel_checks("matmul_q_swiglu_id", w, k, 2 * eff, &sel))) return rc;
    if (t == 0) return FHIP_OK;
    if (!d_x || !d_selw || !d_y) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_swiglu_id: NULL pointer");
    if (((uintptr_t)d_x & 15) != 0 || (w->cols * 4) % 16 != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_swiglu_id: x rows must be 16-byte aligned");
    sel.selw = d_selw; sel.x_per_pair = 0; sel.y_stride = eff; sel.npairs = (int)(t * k);
    return fhip::launch_gemv_sel(w, d_x, d_y, eff, true, sel, (hipStream_t)stream);
}

int fhip_matmul_q_relu2_id(const fhip_weight* w, const float* d_x, size_t t, const float* d_selw, size_t k, size_t eff, float* d_y,
                           void* stream) {
    int rc = need_init();
    if (rc) return rc;
    fhip::SelParams sel{};
    if ((rc = sel_checks("matmul_q_relu2_id", w, k, eff, &sel))) return rc;
    if (t == 0) return FHIP_OK;
    if (!d_x || !d_selw || !d_y) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_relu2_id: NULL pointer");
    if (((uintptr_t)d_x & 15) != 0 || (w->cols * 4) % 16 != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_relu2_id: x rows must be 16-byte aligned");
    sel.selw = d_selw; sel.x_per_pair = 0; sel.y_stride = eff; sel.npairs = (int)(t * k); sel.relu2 = 1;
    return fhip::launch_gemv_sel(w, d_x, d_y, eff, false, sel, (hipStream_t)stream);
}

int fhip_matmul_q_id(const fhip_weight* w, const float* d_x, const float* d_selw, size_t k, size_t out_pe, float* d_y, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    fhip::SelParams sel{};
    if ((rc = sel_checks("matmul_q_id", w, k, out_pe, &sel))) return rc;
    if (!d_x || !d_selw || !d_y) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_id: NULL pointer");
    if (((uintptr_t)d_x & 15) != 0 || (w->cols * 4) % 16 != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_id: x rows must be 16-byte aligned");
    sel.selw = d_selw; sel.x_per_pair = 1; sel.y_stride = out_pe; sel.npairs = (int)k;
    return fhip::launch_gemv_sel(w, d_x, d_y, out_pe, false, sel, (hipStream_t)stream);
}

int fhip_matmul_q_id_wsum(const fhip_weight* w, const float* d_x, size_t t, const float* d_selw, size_t k, size_t out_pe, float* d_y,
                          float* d_ws, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    fhip::SelParams sel{};
    if ((rc = sel_checks("matmul_q_id_wsum", w, k, out_pe, &sel))) return rc;
    if (t == 0) return FHIP_OK;
    if (!d_x || !d_selw || !d_y || !d_ws) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_id_wsum: NULL pointer");
    if (((uintptr_t)d_x & 15) != 0 || (w->cols * 4) % 16 != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_id_wsum: x rows must be 16-byte aligned");
    sel.selw = d_selw; sel.x_per_pair = 1; sel.y_stride = out_pe; sel.npairs = (int)(t * k);
    if ((rc = fhip::launch_gemv_sel(w, d_x, d_ws, out_pe, false, sel, (hipStream_t)stream))) return rc;
    return fhip::launch_moe_wsum(d_ws, d_selw, t, (int)k, out_pe, d_y, (hipStream_t)stream);
}

int fhip_cvt_f32_bf16(const float* d_x, size_t n, uint16_t* d_out, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (n == 0) return FHIP_OK;
    if (!d_x || !d_out) return set_error(FHIP_ERR_ARG, "fhip_cvt_f32_bf16: NULL pointer");
    return fhip::launch_cvt_bf16(d_x, n, d_out, (hipStream_t)stream);
}

int fhip_matmul_q_coop(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, uint16_t* d_ws_bf16, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_coop: NULL weight");
    if (rows_x == 0 || w->rows == 0) return FHIP_OK;
    if (w->cols == 0) return d_y ? zero_outputs(rows_x, w->rows, d_y, (hipStream_t)stream) : set_error(FHIP_ERR_ARG, "fhip_matmul_q_coop: NULL pointer");
    if (!d_x || !d_y || !d_ws_bf16) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_coop: NULL pointer");
    if ((rc = fhip::launch_cvt_bf16(d_x, rows_x * w->cols, d_ws_bf16, (hipStream_t)stream))) return rc;
    return gemm_bf16_lib_ws(w, d_ws_bf16, rows_x, d_y, (hipStream_t)stream, "fhip_matmul_q_coop");
}


size_t fhip_ffn_coop_ws_bytes(const fhip_weight* gu, const fhip_weight* down, size_t rows_x) {
    if (!gu || !down) return 0;
    return align256(rows_x * gu->cols * 2) + align256(rows_x * gu->rows * 4) + align256(rows_x * down->cols * 2);
}

int fhip_ffn_coop(const fhip_weight* gu, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y,
                  void* d_ws, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!gu || !down) return set_error(FHIP_ERR_ARG, "fhip_ffn_coop: NULL weight");
    if (gu->rows % 2 != 0) return set_error(FHIP_ERR_SHAPE, "fhip_ffn_coop: gate_up rows must be even");
    const size_t n_ff = gu->rows / 2;
    if (down->cols != n_ff) return set_error(FHIP_ERR_SHAPE, "down in dim must equal n_ff");
    if (rows_x == 0) return FHIP_OK;
    if (!d_x || !d_y || !d_ws) return set_error(FHIP_ERR_ARG, "fhip_ffn_coop: NULL pointer");
    if (((uintptr_t)d_ws & 255) != 0) return set_error(FHIP_ERR_ARG, "fhip_ffn_coop: workspace must be 256-byte aligned");
    // an empty inner dimension on either side: gate and up are 0, silu(0) * 0 = 0, and so is every output
    if (gu->cols == 0 || n_ff == 0) return zero_outputs(rows_x, down->rows, d_y, (hipStream_t)stream);
    uint8_t* ws = (uint8_t*)d_ws;
    uint16_t* xb = (uint16_t*)ws;
    float* g = (float*)(ws + align256(rows_x * gu->cols * 2));
    uint16_t* hb = (uint16_t*)((uint8_t*)g + align256(rows_x * gu->rows * 4));
    hipStream_t s = (hipStream_t)stream;
    if ((rc = fhip::launch_cvt_bf16(d_x, rows_x * gu->cols, xb, s))) return rc;
    if ((rc = gemm_bf16_lib_ws(gu, xb, rows_x, g, s, "fhip_ffn_coop"))) return rc;
    if ((rc = fhip::launch_swiglu_bf16(g, rows_x, n_ff, hb, s))) return rc;
    return gemm_bf16_lib_ws(down, hb, rows_x, d_y, s, "fhip_ffn_coop");
}

size_t fhip_matmul_q_f16x2_ws_bytes(const fhip_weight* w, size_t rows_x) {
    if (!fhip::gemm_f16x2_supports(w, rows_x)) return 0;
    return align256(fhip::gemm_f16x2_xp_bytes(w, rows_x));
}

static int f16x2_checks(const char* who, const fhip_weight* w, size_t rows_x) {
    if (rows_x > 32) return set_error(FHIP_ERR_SHAPE, "%s: at most 32 activation rows (got %zu)", who, rows_x);
    if (w->type != FHIP_Q4_K && w->type != FHIP_Q5_K && w->type != FHIP_Q6_K && w->type != FHIP_Q8_0)
        return set_error(FHIP_ERR_UNSUPPORTED_TYPE, "%s: no kernel for ggml type %u (Q4_K, Q5_K, Q6_K and Q8_0 only)", who, w->type);
    if (w->type == FHIP_Q8_0 && rows_x > 16) return set_error(FHIP_ERR_SHAPE, "%s: at most 16 activation rows for Q8_0 (got %zu)", who, rows_x);
    if (rows_x && w->rows && !fhip::gemm_f16x2_supports(w, rows_x))
        return set_error(FHIP_ERR_SHAPE, "%s: weight rows of %zu columns are outside what the kernels take", who, w->cols);
    return FHIP_OK;
}

int fhip_matmul_q_f16x2(const fhip_weight* w, const float* d_x, size_t rows_x, float* d_y, void* d_ws, void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!w) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_f16x2: NULL weight");
    if ((rc = f16x2_checks("fhip_matmul_q_f16x2", w, rows_x))) return rc;
    if (rows_x == 0 || w->rows == 0) return FHIP_OK;
    if (!d_x || !d_y || !d_ws) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_f16x2: NULL pointer");
    if (((uintptr_t)d_ws & 255) != 0) return set_error(FHIP_ERR_ARG, "fhip_matmul_q_f16x2: workspace must be 256-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    uint16_t* xp = (uint16_t*)d_ws;
    const bool clr = fhip::gemm_f16x2_adds_into_y(w, rows_x);   // then the split clears y on the side
    if ((rc = fhip::launch_xsplit_f16(w, d_x, rows_x, false, xp, s, clr ? d_y : nullptr, clr ? rows_x * w->rows : 0))) return rc;
    return fhip::launch_gemm_f16x2(w, xp, rows_x, d_y, s, clr);
}

size_t fhip_ffn_f16x2_ws_bytes(const fhip_weight* gu, const fhip_weight* down, size_t rows_x) {
    if (!fhip::gemm_f16x2_supports(gu, rows_x) || !fhip::gemm_f16x2_supports(down, rows_x)) return 0;
    return align256(fhip::gemm_f16x2_xp_bytes(gu, rows_x)) + align256(rows_x * gu->rows * 4) +
           align256(fhip::gemm_f16x2_xp_bytes(down, rows_x));
}

int fhip_ffn_f16x2(const fhip_weight* gu, const fhip_weight* down, const float* d_x, size_t rows_x, float* d_y, void* d_ws,
                   void* stream) {
    int rc = need_init();
    if (rc) return rc;
    if (!gu || !down) return set_error(FHIP_ERR_ARG, "fhip_ffn_f16x2: NULL weight");
    if (gu->rows % 2 != 0) return set_error(FHIP_ERR_SHAPE, "ffn: gate_up rows must be even");
    const size_t n_ff = gu->rows / 2;
    if (down->cols != n_ff) return set_error(FHIP_ERR_SHAPE, "down in dim must equal n_ff");
    if ((rc = f16x2_checks("fhip_ffn_f16x2", gu, rows_x)) || (rc = f16x2_checks("fhip_ffn_f16x2", down, rows_x))) return rc;
    if (rows_x == 0) return FHIP_OK;
    if (!d_x || !d_y || !d_ws) return set_error(FHIP_ERR_ARG, "fhip_ffn_f16x2: NULL pointer");
    if (((uintptr_t)d_ws & 255) != 0) return set_error(FHIP_ERR_ARG, "fhip_ffn_f16x2: workspace must be 256-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)d_ws;
    uint16_t* xp1 = (uint16_t*)ws;
    float* g = (float*)(ws + align256(fhip::gemm_f16x2_xp_bytes(gu, rows_x)));
    uint16_t* xp2 = (uint16_t*)((uint8_t*)g + align256(rows_x * gu->rows * 4));
    const bool clr1 = fhip::gemm_f16x2_adds_into_y(gu, rows_x), clr2 = fhip::gemm_f16x2_adds_into_y(down, rows_x);
    if ((rc = fhip::launch_xsplit_f16(gu, d_x, rows_x, false, xp1, s, clr1 ? g : nullptr, clr1 ? rows_x * gu->rows : 0))) return rc;
    if ((rc = fhip::launch_gemm_f16x2(gu, xp1, rows_x, g, s, clr1))) return rc;
    // SwiGLU of [gate | up] is computed while the rows are split for the down projection
    if ((rc = fhip::launch_xsplit_f16(down, g, rows_x, true, xp2, s, clr2 ? d_y : nullptr, clr2 ? rows_x * down->rows : 0))) return rc;
    return fhip::launch_gemm_f16x2(down, xp2, rows_x, d_y, s, clr2);
}

int fhip_matvec_q8_0_host(const float* h_x, const uint8_t* h_w, size_t w_len, size_t rows, size_t cols, float* h_y) {
    int rc = need_init();
    if (rc) return rc;
    // asserts of crates/ferric-tensor/src/cpu_simd.rs:80-83
    if (cols % 32 != 0) return set_error(FHIP_ERR_SHAPE, "Q8_0 cols must be a multiple of 32");
    if (w_len != rows * (cols / 32) * 34) return set_error(FHIP_ERR_SHAPE, "unexpected Q8_0 byte length");
    if (rows == 0) return FHIP_OK;
    if (!h_x || !h_w || !h_y) return set_error(FHIP_ERR_ARG, "fhip_matvec_q8_0_host: NULL pointer");
    fhip_weight* w = nullptr;
    if ((rc = fhip_weight_create(FHIP_Q8_0, h_w, w_len, rows, cols, &w))) return rc;
    void *d_x = nullptr, *d_y = nullptr;
    rc = check_hip(hipMalloc(&d_x, (cols ? cols : 1) * sizeof(float)), "hipMalloc");
    if (!rc) rc = check_hip(hipMalloc(&d_y, rows * sizeof(float)), "hipMalloc");
    if (!rc && cols) rc = check_hip(hipMemcpy(d_x, h_x, cols * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy H2D");
    if (!rc) {
        if (cols == 0) rc = check_hip(hipMemset(d_y, 0, rows * sizeof(float)), "hipMemset");
        else rc = fhip::launch_gemv(w, (const float*)d_x, 1, (float*)d_y, 0, nullptr);
    }
    if (!rc) rc = check_hip(hipMemcpy(h_y, d_y, rows * sizeof(float), hipMemcpyDeviceToHost), "hipMemcpy D2H");
    if (d_x) (void)hipFree(d_x);
    if (d_y) (void)hipFree(d_y);
    fhip_weight_destroy(w);
    return rc;
}

// ---- crates/ferric-tensor/src/cpu_simd.rs:238-331: Pool / matvec_q8_0_pooled --------------------------------
// The reference's pool exists so that a call does not pay its set-up again (thread creation there). What a call of the
// host-buffer mat-vec pays here is the upload of the weight bytes, so the pool keeps those resident: the weight the
// last call used stays in HBM, keyed by the caller's (pointer, length, cols) -- `w` is an immutable Arc<Vec<u8>> in the
// reference -- together with the staging buffers and a stream of its own.
struct fhip_pool {
    size_t threads;
    hipStream_t stream;
    const uint8_t* key;
    size_t key_len, key_cols;
    uint64_t key_print;   // fingerprint of the bytes the key pointed at when they were uploaded
    uint8_t* d_w;
    size_t w_cap;
    float *d_x, *d_y;
    size_t x_cap, y_cap;
    size_t uploads;
};

// FNV-1a over the first and the last 4 KiB and 64 evenly spaced 64-byte samples of the weight: about 12 KiB per call. It catches
// a buffer that was freed and reused, or rewritten, at the same address and length (what pointer + length alone would take for
// the resident weight); it is not a proof of equality -- a caller that edits a few bytes in place still calls fhip_pool_forget.
static uint64_t pool_fingerprint(const uint8_t* w, size_t n) {
    uint64_t h = 1469598103934665603ull;
    auto eat = [&](size_t from, size_t len) {
        for (size_t i = from; i < from + len && i < n; i++) h = (h ^ w[i]) * 1099511628211ull;
    };
    eat(0, 4096);
    if (n > 8192) {
        eat(n - 4096, 4096);
        const size_t step = (n - 8192) / 64;
        for (size_t k = 0; k < 64 && step >= 64; k++) eat(4096 + k * step, 64);
    } else if (n > 4096) {
        eat(4096, n - 4096);
    }
    return h ^ n;
}

int fhip_pool_create(size_t threads, fhip_pool** out) {
    if (!out) return set_error(FHIP_ERR_ARG, "fhip_pool_create: NULL output");
    *out = nullptr;
    int rc = need_init();
    if (rc) return rc;
    fhip_pool* p = new (std::nothrow) fhip_pool();
    if (!p) return set_error(FHIP_ERR_HIP, "fhip_pool_create: out of host memory");
    p->threads = threads ? threads : 1;   // Pool::new: n.max(1)
    if ((rc = check_hip(hipStreamCreate(&p->stream), "hipStreamCreate"))) { delete p; return rc; }
    *out = p;
    return FHIP_OK;
}

size_t fhip_pool_threads(const fhip_pool* p) { return p ? p->threads : 0; }
size_t fhip_pool_uploads(const fhip_pool* p) { return p ? p->uploads : 0; }

void fhip_pool_forget(fhip_pool* p) {
    if (p) { p->key = nullptr; p->key_len = 0; p->key_cols = 0; }
}

void fhip_pool_destroy(fhip_pool* p) {
    if (!p) return;
    (void)hipStreamSynchronize(p->stream);
    if (p->d_w) (void)hipFree(p->d_w);
    if (p->d_x) (void)hipFree(p->d_x);
    if (p->d_y) (void)hipFree(p->d_y);
    (void)hipStreamDestroy(p->stream);
    delete p;
}

static int pool_reserve(void** d, size_t* cap, size_t need, const char* what) {
    if (need <= *cap) return FHIP_OK;
    if (*d) (void)hipFree(*d);
    *d = nullptr; *cap = 0;
    int rc = check_hip(hipMalloc(d, need), what);
    if (!rc) *cap = need;
    return rc;
}

int fhip_matvec_q8_0_pooled(fhip_pool* p, const float* h_x, size_t x_len, const uint8_t* h_w, size_t w_len, size_t cols, size_t lo,
                            size_t hi, float* h_y) {
    int rc = need_init();
    if (rc) return rc;
    if (!p) return set_error(FHIP_ERR_ARG, "fhip_matvec_q8_0_pooled: NULL pool");
    if (lo > hi) return set_error(FHIP_ERR_SHAPE, "empty or inverted span");             // cpu_simd.rs:311
    const size_t rows = hi - lo;
    if (rows == 0) return FHIP_OK;                                                        // :313
    if (!h_y) return set_error(FHIP_ERR_ARG, "fhip_matvec_q8_0_pooled: NULL output");
    const size_t nblk = cols / 32, row_bytes = nblk * 34;                                 // :314; row_q8_0 walks cols / 32 blocks
    if (nblk == 0) { memset(h_y, 0, rows * sizeof(float)); return FHIP_OK; }              // no block: every sum is 0.0
    // the slices of :321 and of row_q8_0 (:62, :64) panic when the row span or the activations run past their arrays
    if (hi > w_len / row_bytes) return set_error(FHIP_ERR_SHAPE, "range end index %zu out of range for slice of length %zu", hi * row_bytes, w_len);
    if (x_len < nblk * 32) return set_error(FHIP_ERR_SHAPE, "range end index %zu out of range for slice of length %zu", nblk * 32, x_len);
    if (!h_x || !h_w) return set_error(FHIP_ERR_ARG, "fhip_matvec_q8_0_pooled: NULL pointer");
    const size_t kcols = nblk * 32, all_rows = w_len / row_bytes;
    const uint64_t print = pool_fingerprint(h_w, all_rows * row_bytes);
    if (p->key != h_w || p->key_len != w_len || p->key_cols != kcols || p->key_print != print) {
        fhip_pool_forget(p);
        if ((rc = pool_reserve((void**)&p->d_w, &p->w_cap, all_rows * row_bytes, "hipMalloc"))) return rc;
        if ((rc = check_hip(hipMemcpyAsync(p->d_w, h_w, all_rows * row_bytes, hipMemcpyHostToDevice, p->stream), "hipMemcpy H2D"))) return rc;
        p->key = h_w; p->key_len = w_len; p->key_cols = kcols; p->key_print = print;
        p->uploads++;
    }
    if ((rc = pool_reserve((void**)&p->d_x, &p->x_cap, kcols * sizeof(float), "hipMalloc"))) return rc;
    if ((rc = pool_reserve((void**)&p->d_y, &p->y_cap, rows * sizeof(float), "hipMalloc"))) return rc;
    if ((rc = check_hip(hipMemcpyAsync(p->d_x, h_x, kcols * sizeof(float), hipMemcpyHostToDevice, p->stream), "hipMemcpy H2D"))) return rc;
    fhip_weight view;
    if ((rc = make_weight(FHIP_Q8_0, rows * row_bytes, rows, kcols, view))) return rc;
    view.d_raw = p->d_w + lo * row_bytes;
    if ((rc = fhip::launch_gemv(&view, p->d_x, 1, p->d_y, 0, p->stream))) return rc;
    if ((rc = check_hip(hipMemcpyAsync(h_y, p->d_y, rows * sizeof(float), hipMemcpyDeviceToHost, p->stream), "hipMemcpy D2H"))) return rc;
    return check_hip(hipStreamSynchronize(p->stream), "hipStreamSynchronize");
}

}  // extern "C"
