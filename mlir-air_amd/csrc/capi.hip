// C ABI of libw4a16_hip.so: argument validation (before any HIP call) and dispatch.
#include <string.h>

#include <mutex>

#include "../../include/w4a16.h"
#include "common.h"
#include "kernels.h"
#include "wstream.h"

using namespace w4a16;

namespace {

thread_local char t_hip_error[256] = "";

int hip_fail(hipError_t e) {
    strncpy(t_hip_error, hipGetErrorString(e), sizeof(t_hip_error) - 1);
    t_hip_error[sizeof(t_hip_error) - 1] = 0;
    return W4A16_ERR_HIP;
}

inline bool misaligned(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

int check_quant(const void *qweight, const void *qzeros, const void *scales, int K, int N, int group, int n_mult) {
    if (!qweight || !qzeros || !scales) return W4A16_ERR_NULL;
    if (group != kGroup) return W4A16_ERR_GROUP;
    if (K <= 0 || N <= 0 || K % kGroup != 0 || N % n_mult != 0) return W4A16_ERR_SHAPE;
    if (misaligned(qweight) || misaligned(qzeros) || misaligned(scales)) return W4A16_ERR_ALIGN;
    return W4A16_OK;
}

size_t round256(size_t v) { return (v + 255) & ~size_t(255); }

// Compute units of the current device (cached per device id; 0 if the query fails).
int current_cus() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (!cached[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached[dev] = n;
    }
    return cached[dev];
}

size_t stream_partial_bytes(int M, int N, int nmat) {
    // tiles are at most 512 columns wide; a ragged last tile is stored in full
    return round256((size_t)nmat * kMaxKSplit * (size_t)(M < 16 ? M : 16) * ((size_t)N + 512) * sizeof(float));
}

// One AWQ matrix in the checkpoint layout (qweight, qzeros, scales [K / 128, N]).
struct QuantW {
    const int32_t *qw, *qz;
    const uint16_t *sc;
};

int check_w(const QuantW &w, int K, int N, int group) { return check_quant(w.qw, w.qz, w.sc, K, N, group, 32); }

hipError_t stream_w(const uint16_t *x, const QuantW &a, const QuantW *up, uint16_t *y, int M, int K, int N, void *workspace,
                    hipStream_t st, const StreamExtras &ex) {
    return launch_stream(x, a.qw, a.qz, a.sc, up ? up->qw : nullptr, up ? up->qz : nullptr, up ? up->sc : nullptr, y, M, K, N,
                         workspace, st, ex);
}

int rms_gemv_impl(const uint16_t *x, const uint16_t *norm_weight, float eps, const QuantW &w, uint16_t *y,
                  int K, int N, int group, void *workspace, size_t workspace_bytes, void *stream,
                  const float *x_sumsq = nullptr, int n_pieces = 0) {
    if (!x || !y || !norm_weight) return W4A16_ERR_NULL;
    int rc = check_w(w, K, N, group);
    if (rc) return rc;
    if (!(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(y) || misaligned(norm_weight)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_gemm_workspace_bytes(1, K, N)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    StreamExtras ex;
    ex.norm_w = norm_weight;
    ex.eps = eps;
    ex.sumsq_in = x_sumsq;
    ex.sumsq_n = x_sumsq ? n_pieces : 0;
    hipError_t e = stream_w(x, w, nullptr, y, 1, K, N, workspace, static_cast<hipStream_t>(stream), ex);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

// The decode attention's chunk partials, when stage 1 of the block merges them itself (StreamExtras::attn_*).
struct AttnPartials {
    const float *ml, *acc;
    int nsplit, hd;
};

int o_gemv_ffn_impl(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                    float eps, const QuantW &wo, const QuantW &wg, const QuantW &wu, const QuantW &wd, uint16_t *y,
                    uint16_t *res1_out, uint16_t *h_out, int E, int H, int group, void *workspace,
                    size_t workspace_bytes, void *stream, const AttnPartials *partials = nullptr, bool check_only = false,
                    float *y_sumsq = nullptr) {
    if (!attn_out || !x_residual || !ffn_norm_weight || !y) return W4A16_ERR_NULL;
    int rc = check_w(wo, E, E, group);
    if (rc) return rc;
    rc = check_w(wg, E, H, group);
    if (rc) return rc;
    rc = check_w(wu, E, H, group);
    if (rc) return rc;
    rc = check_w(wd, H, E, group);
    if (rc) return rc;
    if (!(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(attn_out) || misaligned(x_residual) || misaligned(ffn_norm_weight) || misaligned(y) ||
        (res1_out && misaligned(res1_out)) || (h_out && misaligned(h_out)))
        return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_block_workspace_bytes(E, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    if (check_only) return W4A16_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    char *tail = static_cast<char *>(workspace) + w4a16_block_workspace_bytes(E, H) - 256;
    float *res1_sumsq = reinterpret_cast<float *>(tail);
    uint16_t *res1 = res1_out ? res1_out : reinterpret_cast<uint16_t *>(tail - round256((size_t)E * sizeof(uint16_t)));
    uint16_t *h = h_out ? h_out
                        : reinterpret_cast<uint16_t *>(tail - round256((size_t)E * sizeof(uint16_t)) -
                                                       round256((size_t)H * sizeof(uint16_t)));
    // stage 1: res1 = bf16(attn_out . Wo + x_residual); its reducers also leave sum(res1^2) per column
    // tile, so that stage 2 does not have to read res1 again for the norm
    const int res1_tiles = plan_stream(1, E, E, true).ntiles;   // a launch that leaves sums of squares keeps 256-column tiles
    const bool chain_norm = res1_tiles <= 64;
    StreamExtras add;
    add.residual = x_residual;
    if (chain_norm) add.sumsq_out = res1_sumsq;
    if (partials) {
        add.attn_ml = partials->ml;
        add.attn_acc = partials->acc;
        add.attn_nsplit = partials->nsplit;
        add.attn_hd = partials->hd;
    }
    hipError_t e = stream_w(attn_out, wo, nullptr, res1, 1, E, E, workspace, st, add);
    add.attn_ml = add.attn_acc = nullptr;   // stage 3 reuses `add` for the down projection
    if (e != hipSuccess) return hip_fail(e);
    // stage 2: h = swiglu(rms_norm(res1) . Wgate, rms_norm(res1) . Wup)
    StreamExtras rms;
    rms.norm_w = ffn_norm_weight;
    rms.eps = eps;
    if (chain_norm) {
        rms.sumsq_in = res1_sumsq;
        rms.sumsq_n = res1_tiles;
    }
    e = stream_w(res1, wg, &wu, h, 1, E, H, workspace, st, rms);
    if (e != hipSuccess) return hip_fail(e);
    // stage 3: y = bf16(h . Wdown + res1)
    add.sumsq_out = y_sumsq;
    add.residual = res1;
    e = stream_w(h, wd, nullptr, y, 1, H, E, workspace, st, add);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

}  // namespace

extern "C" {

int w4a16_abi_version(void) { return W4A16_ABI_VERSION; }

const char *w4a16_strerror(int code) {
    switch (code) {
        case W4A16_OK: return "ok";
        case W4A16_ERR_NULL: return "required pointer is NULL";
        case W4A16_ERR_SHAPE: return "unsupported shape (need K % 128 == 0, N % 32 == 0 (dequant: N % 8 == 0), M >= 1)";
        case W4A16_ERR_GROUP: return "unsupported group size (only 128)";
        case W4A16_ERR_ALIGN: return "pointer is not 16-byte aligned";
        case W4A16_ERR_WORKSPACE: return "workspace is NULL or too small";
        case W4A16_ERR_HIP: return "HIP call failed";
        case W4A16_ERR_TUNE: return "unknown tuning key or value out of range";
        case W4A16_ERR_TIMEOUT: return "a split-K reducer gave up waiting for a partial result; the output is invalid";
        case W4A16_ERR_TOO_LARGE: return "shape beyond the fixed scratch of the entry point that allocates nothing (N <= 32768)";
        case W4A16_ERR_NOT_PREPARED:
            return "first use of the entry point that allocates nothing on this GPU under stream capture: call w4a16_noalloc_check outside capture first";
        default: return "unknown error code";
    }
}

const char *w4a16_last_hip_error(void) { return t_hip_error; }

int awq_dequant_bf16(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, uint16_t *out_bf16,
                     int K, int N, int group, void *stream) {
    if (!out_bf16) return W4A16_ERR_NULL;
    int rc = check_quant(qweight, qzeros, scales, K, N, group, 8);
    if (rc) return rc;
    if (misaligned(out_bf16)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_dequant(qweight, qzeros, scales, out_bf16, K, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

size_t awq_dequant_1d_tile_bytes(int n, int group, int herd_n) {
    if (n <= 0 || group <= 0 || herd_n <= 0 || group % 8 != 0 || n % herd_n != 0 || (n / herd_n) % group != 0) return 0;
    const int n_tile = n / herd_n, ng = n_tile / group;
    return (size_t)((n_tile / 2 + 3 * ng + 3) & ~3);
}

int awq_dequant_1d_bf16(const uint8_t *packed, uint16_t *out_bf16, int n, int group, int herd_n, void *stream) {
    if (!packed || !out_bf16) return W4A16_ERR_NULL;
    if (awq_dequant_1d_tile_bytes(n, group, herd_n) == 0) return W4A16_ERR_SHAPE;
    if (misaligned(packed) || misaligned(out_bf16)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_dequant_1d(packed, out_bf16, n, group, herd_n, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

size_t w4a16_gemm_workspace_bytes(int M, int K, int N) {
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    return kHeaderBytes + stream_partial_bytes(M, N, 1);
}

size_t w4a16_ffn_workspace_bytes(int K, int H) {
    if (K <= 0 || H <= 0) return 0;
    const size_t a = stream_partial_bytes(1, H, 2), b = stream_partial_bytes(1, K, 1);
    return kHeaderBytes + (a > b ? a : b) + round256((size_t)H * sizeof(uint16_t));
}

int w4a16_workspace_init(void *workspace, size_t workspace_bytes, void *stream) {
    if (!workspace) return W4A16_ERR_NULL;
    if (workspace_bytes < kHeaderBytes) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_fill_workspace(workspace, workspace_bytes & ~size_t(3), static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_workspace_check(const void *workspace, void *stream) {
    if (!workspace) return W4A16_ERR_NULL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint32_t flag = 0;
    hipError_t e = hipMemcpyAsync(&flag, workspace, sizeof(flag), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return hip_fail(e);
    return flag ? W4A16_ERR_TIMEOUT : W4A16_OK;
}

int w4a16_gemm_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                    uint16_t *y, int M, int K, int N, int group, void *workspace, size_t workspace_bytes,
                    void *stream) {
    if (!x || !y) return W4A16_ERR_NULL;
    int rc = check_quant(qweight, qzeros, scales, K, N, group, 32);
    if (rc) return rc;
    if (M <= 0) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(y)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_gemm_workspace_bytes(M, K, N)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e;
    const int stream_max_m = g_stream_tune.stream_max_m >= 16 ? g_stream_tune.stream_max_m : kStreamMaxM;
    if (M <= stream_max_m) {
        // the streaming kernel takes up to 16 rows per launch; a few more launches over the same
        // (cache-resident) weights still beat one 256-row MFMA tile that is mostly padding
        e = hipSuccess;
        for (int m0 = 0; m0 < M && e == hipSuccess; m0 += 16) {
            const int rows = M - m0 < 16 ? M - m0 : 16;
            e = launch_stream(x + (size_t)m0 * K, qweight, qzeros, scales, nullptr, nullptr, nullptr,
                              y + (size_t)m0 * N, rows, K, N, workspace, st);
        }
    } else {
        e = launch_gemm_prefill(x, qweight, qzeros, scales, y, M, K, N, st);
    }
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_gemv_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                    uint16_t *y, int K, int N, int group, void *workspace, size_t workspace_bytes, void *stream) {
    return w4a16_gemm_bf16(x, qweight, qzeros, scales, y, 1, K, N, group, workspace, workspace_bytes, stream);
}

// ---- entry point that allocates nothing -----------------------------------------------------------
// The split-K workspace of w4a16_gemv_bf16 as a file-scope device array: every GPU the library runs on holds
// its own copy until the process ends.  In host code the array's name is a stand-in, not a device address:
// the address on the current device comes from hipGetSymbolAddress, once per device, and only that pointer
// is handed to kernels.
}  // extern "C"

namespace {
constexpr int kNoAllocMaxN = 32768;
constexpr size_t kNoAllocScratchBytes = kHeaderBytes + (size_t)kMaxKSplit * (kNoAllocMaxN + 512) * sizeof(float);   // 4.06 MiB
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

void *g_scratch_ptr[64] = {nullptr};   // per device: address of `scratch` there, published once the array is prepared
std::mutex g_scratch_mutex;

// Address of this device's copy of `scratch`.  On first use the array is prepared (header zero, every slot empty) and
// the fill has FINISHED before the address is published: a zero-initialised array is not an empty one, so no launch
// on any stream may see it earlier.  That needs a synchronisation, which a capturing stream cannot give: the first
// use under capture returns W4A16_ERR_NOT_PREPARED instead (w4a16_noalloc_check prepares the array ahead of it).
int noalloc_scratch(hipStream_t st, void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= 64) return W4A16_ERR_SHAPE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(st, &cap);
        if (e != hipSuccess) return hip_fail(e);
        if (cap != hipStreamCaptureStatusNone) return W4A16_ERR_NOT_PREPARED;
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e);
        if (!ptr) return W4A16_ERR_NULL;
        e = launch_fill_workspace(ptr, kNoAllocScratchBytes, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return hip_fail(e);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return W4A16_OK;
}

// tests only (w4a16_tune("noalloc_forget", 1)): the next use on the current device prepares the array again
void noalloc_forget() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    g_scratch_ptr[dev] = nullptr;
}
}  // namespace

extern "C" {

int w4a16_gemv_noalloc_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                            uint16_t *y, int K, int N, int group, void *stream) {
    if (!x || !y) return W4A16_ERR_NULL;
    int rc = check_quant(qweight, qzeros, scales, K, N, group, 32);
    if (rc) return rc;
    if (N > kNoAllocMaxN) return W4A16_ERR_TOO_LARGE;
    if (misaligned(x) || misaligned(y)) return W4A16_ERR_ALIGN;
    static_assert(kNoAllocScratchBytes >= kHeaderBytes + (size_t)kMaxKSplit * (kNoAllocMaxN + 512) * sizeof(float), "scratch too small");
    if (w4a16_gemm_workspace_bytes(1, K, N) > kNoAllocScratchBytes) return W4A16_ERR_TOO_LARGE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    void *ws = nullptr;
    rc = noalloc_scratch(st, &ws);
    if (rc) return rc;
    hipError_t e = launch_stream(x, qweight, qzeros, scales, nullptr, nullptr, nullptr, y, 1, K, N, ws, st);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_noalloc_check(void *stream) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    void *ws = nullptr;
    int rc = noalloc_scratch(st, &ws);   // prepares the array on first use (not under capture)
    if (rc) return rc;
    rc = w4a16_workspace_check(ws, stream);
    if (rc == W4A16_ERR_TIMEOUT) {   // slots filled late are dirty: empty the array again before the next call
        hipError_t e = launch_fill_workspace(ws, kNoAllocScratchBytes, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return hip_fail(e);
    }
    return rc;
}

int w4a16_gemv_swiglu_bf16(const uint16_t *x, const int32_t *gate_qweight, const int32_t *gate_qzeros,
                           const uint16_t *gate_scales, const int32_t *up_qweight, const int32_t *up_qzeros,
                           const uint16_t *up_scales, uint16_t *h, int K, int H, int group, void *workspace,
                           size_t workspace_bytes, void *stream) {
    if (!x || !h) return W4A16_ERR_NULL;
    int rc = check_quant(gate_qweight, gate_qzeros, gate_scales, K, H, group, 32);
    if (rc) return rc;
    rc = check_quant(up_qweight, up_qzeros, up_scales, K, H, group, 32);
    if (rc) return rc;
    if (misaligned(x) || misaligned(h)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_ffn_workspace_bytes(K, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_stream(x, gate_qweight, gate_qzeros, gate_scales, up_qweight, up_qzeros, up_scales, h, 1, K, H,
                                 workspace, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_ffn_swiglu_bf16(const uint16_t *x, const int32_t *gate_qweight, const int32_t *gate_qzeros,
                          const uint16_t *gate_scales, const int32_t *up_qweight, const int32_t *up_qzeros,
                          const uint16_t *up_scales, const int32_t *down_qweight, const int32_t *down_qzeros,
                          const uint16_t *down_scales, uint16_t *y, uint16_t *h_out, int K, int H, int group,
                          void *workspace, size_t workspace_bytes, void *stream) {
    if (!x || !y) return W4A16_ERR_NULL;
    int rc = check_quant(gate_qweight, gate_qzeros, gate_scales, K, H, group, 32);
    if (rc) return rc;
    rc = check_quant(up_qweight, up_qzeros, up_scales, K, H, group, 32);
    if (rc) return rc;
    rc = check_quant(down_qweight, down_qzeros, down_scales, H, K, group, 32);
    if (rc) return rc;
    if (misaligned(x) || misaligned(y) || (h_out && misaligned(h_out))) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_ffn_workspace_bytes(K, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint16_t *h = h_out;
    if (!h) h = reinterpret_cast<uint16_t *>(static_cast<char *>(workspace) + w4a16_ffn_workspace_bytes(K, H) -
                                             round256((size_t)H * sizeof(uint16_t)));
    hipError_t e = launch_stream(x, gate_qweight, gate_qzeros, gate_scales, up_qweight, up_qzeros, up_scales, h, 1, K,
                                 H, workspace, st);
    if (e != hipSuccess) return hip_fail(e);
    e = launch_stream(h, down_qweight, down_qzeros, down_scales, nullptr, nullptr, nullptr, y, 1, H, K, workspace, st);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_gemv_add_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                        const uint16_t *residual, uint16_t *y, int K, int N, int group, void *workspace,
                        size_t workspace_bytes, void *stream) {
    if (!x || !y || !residual) return W4A16_ERR_NULL;
    int rc = check_quant(qweight, qzeros, scales, K, N, group, 32);
    if (rc) return rc;
    if (misaligned(x) || misaligned(y) || misaligned(residual)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_gemm_workspace_bytes(1, K, N)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    StreamExtras ex;
    ex.residual = residual;
    hipError_t e = launch_stream(x, qweight, qzeros, scales, nullptr, nullptr, nullptr, y, 1, K, N, workspace,
                                 static_cast<hipStream_t>(stream), ex);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_rms_gemv_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, const int32_t *qweight,
                        const int32_t *qzeros, const uint16_t *scales, uint16_t *y, int K, int N, int group,
                        void *workspace, size_t workspace_bytes, void *stream) {
    return rms_gemv_impl(x, norm_weight, eps, QuantW{qweight, qzeros, scales}, y, K, N, group, workspace,
                         workspace_bytes, stream);
}

int w4a16_rms_gemv_sumsq_bf16(const uint16_t *x, const float *x_sumsq, int n_pieces, const uint16_t *norm_weight, float eps,
                              const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, uint16_t *y, int K,
                              int N, int group, void *workspace, size_t workspace_bytes, void *stream) {
    if (!x_sumsq) return W4A16_ERR_NULL;
    if (n_pieces < 1 || n_pieces > 64) return W4A16_ERR_SHAPE;
    if (misaligned(x_sumsq)) return W4A16_ERR_ALIGN;
    return rms_gemv_impl(x, norm_weight, eps, QuantW{qweight, qzeros, scales}, y, K, N, group, workspace,
                         workspace_bytes, stream, x_sumsq, n_pieces);
}

int w4a16_rms_gemv_swiglu_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps,
                               const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                               const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                               uint16_t *h, int K, int H, int group, void *workspace, size_t workspace_bytes,
                               void *stream) {
    if (!x || !h || !norm_weight) return W4A16_ERR_NULL;
    int rc = check_quant(gate_qweight, gate_qzeros, gate_scales, K, H, group, 32);
    if (rc) return rc;
    rc = check_quant(up_qweight, up_qzeros, up_scales, K, H, group, 32);
    if (rc) return rc;
    if (!(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(h) || misaligned(norm_weight)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_ffn_workspace_bytes(K, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    StreamExtras ex;
    ex.norm_w = norm_weight;
    ex.eps = eps;
    hipError_t e = launch_stream(x, gate_qweight, gate_qzeros, gate_scales, up_qweight, up_qzeros, up_scales, h, 1, K, H,
                                 workspace, static_cast<hipStream_t>(stream), ex);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

size_t w4a16_stream_bytes(int K, int N) {
    if (K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return 0;
    return ws_matrix_bytes(K, N);
}

int w4a16_repack_stream(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, void *wstream, int K, int N,
                        int group, void *stream) {
    if (!wstream) return W4A16_ERR_NULL;
    int rc = check_quant(qweight, qzeros, scales, K, N, group, kWsTileCols);
    if (rc) return rc;
    if (misaligned(wstream)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_repack_ws(qweight, qzeros, scales, wstream, K, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_probe_stream_read(const void *wstream, uint32_t *out_words, int K, int N, void *stream) {
    if (!wstream || !out_words) return W4A16_ERR_NULL;
    if (K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return W4A16_ERR_SHAPE;
    if (misaligned(wstream) || misaligned(out_words)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_probe_ws(wstream, out_words, K, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

namespace {
// One whole-K launch on stream-order weights: argument checks shared by every stream-order entry point.
int gemv_stream_call(const uint16_t *x, const void *w, const void *w_up, uint16_t *y, int K, int N, int group, void *stream,
                     const GemvWsExtras &ex) {
    if (!x || !w || !y) return W4A16_ERR_NULL;
    if (group != kGroup) return W4A16_ERR_GROUP;
    if (K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return W4A16_ERR_SHAPE;
    if (ex.norm_w && !(ex.eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (ex.sumsq_in && (ex.sumsq_n < 1 || ex.sumsq_n > 4096)) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(w) || misaligned(y) || (w_up && misaligned(w_up)) || (ex.residual && misaligned(ex.residual)) ||
        (ex.norm_w && misaligned(ex.norm_w)) || (ex.sumsq_in && misaligned(ex.sumsq_in)) || (ex.sumsq_out && misaligned(ex.sumsq_out)))
        return W4A16_ERR_ALIGN;
    hipError_t e = launch_gemv_ws(x, w, w_up, y, K, N, static_cast<hipStream_t>(stream), ex);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

// [res1 bf16 E][h bf16 H][sum of squares of res1, one float per 16 columns]
struct BlockStreamScratch {
    uint16_t *res1, *h;
    float *res1_sumsq;
};
BlockStreamScratch block_stream_scratch(void *workspace, int E, int H) {
    char *p = static_cast<char *>(workspace);
    BlockStreamScratch s;
    s.res1 = reinterpret_cast<uint16_t *>(p);
    s.h = reinterpret_cast<uint16_t *>(p + round256((size_t)E * sizeof(uint16_t)));
    s.res1_sumsq = reinterpret_cast<float *>(p + round256((size_t)E * sizeof(uint16_t)) + round256((size_t)H * sizeof(uint16_t)));
    return s;
}

int o_gemv_ffn_stream_impl(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                           const void *wo, const void *wg, const void *wu, const void *wd, uint16_t *y, uint16_t *res1_out,
                           uint16_t *h_out, float *y_sumsq, int E, int H, int group, void *workspace, size_t workspace_bytes,
                           void *stream, bool check_only, bool q4 = false) {
    if (!attn_out || !x_residual || !ffn_norm_weight || !wo || !wg || !wu || !wd || !y) return W4A16_ERR_NULL;
    if (group != kGroup) return W4A16_ERR_GROUP;
    if (E <= 0 || H <= 0 || E % kGroup != 0 || H % kGroup != 0) return W4A16_ERR_SHAPE;
    if (!(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if ((res1_out && misaligned(res1_out)) || (h_out && misaligned(h_out)) || (y_sumsq && misaligned(y_sumsq))) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_block_stream_workspace_bytes(E, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    if (check_only) return W4A16_OK;
    const BlockStreamScratch sc = block_stream_scratch(workspace, E, H);
    uint16_t *res1 = res1_out ? res1_out : sc.res1;
    uint16_t *h = h_out ? h_out : sc.h;
    // stage 1: res1 = bf16(attn_out . Wo + x_residual), leaving sum(res1^2) per tile for the norm of stage 2
    GemvWsExtras s1;
    s1.q4 = q4;
    s1.residual = x_residual;
    s1.sumsq_out = sc.res1_sumsq;
    int rc = gemv_stream_call(attn_out, wo, nullptr, res1, E, E, group, stream, s1);
    if (rc) return rc;
    // stage 2: h = swiglu(rms_norm(res1) . Wgate, rms_norm(res1) . Wup)
    GemvWsExtras s2;
    s2.q4 = q4;
    s2.norm_w = ffn_norm_weight;
    s2.eps = eps;
    s2.sumsq_in = sc.res1_sumsq;
    s2.sumsq_n = E / kWsTileCols;
    rc = gemv_stream_call(res1, wg, wu, h, E, H, group, stream, s2);
    if (rc) return rc;
    // stage 3: y = bf16(h . Wdown + res1)
    GemvWsExtras s3;
    s3.q4 = q4;
    s3.residual = res1;
    s3.sumsq_out = y_sumsq;
    return gemv_stream_call(h, wd, nullptr, y, H, E, group, stream, s3);
}
}  // namespace

int w4a16_gemv_stream_bf16(const uint16_t *x, const void *wstream, uint16_t *y, int K, int N, int group, void *stream) {
    return gemv_stream_call(x, wstream, nullptr, y, K, N, group, stream, GemvWsExtras());
}

int w4a16_gemm_stream_bf16(const uint16_t *x, const void *wstream, uint16_t *y, int M, int K, int N, int group, void *stream) {
    if (M == 1) return gemv_stream_call(x, wstream, nullptr, y, K, N, group, stream, GemvWsExtras());
    if (!x || !wstream || !y) return W4A16_ERR_NULL;
    if (group != kGroup) return W4A16_ERR_GROUP;
    if (M <= 0 || K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(wstream) || misaligned(y)) return W4A16_ERR_ALIGN;
    // up to here the weights are streamed once per 64 rows (exact weights); from here on the tiled kernel that
    // multiplies bf16-rounded weights.  The tiled kernel takes the same time for any M <= 256 (K = 4096, N = 14336:
    // 51 us; N = 4096: 49 us; K = 2048, N = 8192: 27 us), two launches of 64 rows 46, 38 and 24 us, three 67, 56 and 36 us.
    const int prefill_min_m = g_gemv_ws_tune.prefill_min_m > 16 ? g_gemv_ws_tune.prefill_min_m : kGemmWsMaxM + 1;
    hipError_t e = M >= prefill_min_m && gemm_prefill_ws_supported(M, K, N)
                       ? launch_gemm_prefill_ws(x, wstream, y, M, K, N, static_cast<hipStream_t>(stream))
                       : launch_gemm_ws(x, wstream, y, nullptr, M, K, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

size_t w4a16_gemm_stream_scratch_bytes(int M, int K, int N) {
    if (M <= 16 || M > kGemmWsMaxM || K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return 0;
    return gemm_wsk_pays(M, K, N) ? gemm_wsk_scratch_bytes(M, K, N) : 0;
}

int w4a16_gemm_stream_scratch_bf16(const uint16_t *x, const void *wstream, uint16_t *y, int M, int K, int N, int group, void *scratch,
                                   size_t scratch_bytes, void *stream) {
    // 17 .. 128 rows of a shape where the split along K is the faster one: the split-K kernel; everything else is
    // w4a16_gemm_stream_bf16
    const int prefill_min_m = g_gemv_ws_tune.prefill_min_m > 16 ? g_gemv_ws_tune.prefill_min_m : kGemmWsMaxM + 1;
    const bool shape_ok = K > 0 && N > 0 && K % kGroup == 0 && N % kWsTileCols == 0;
    if (M <= 16 || M >= prefill_min_m || !shape_ok || !gemm_wsk_pays(M, K, N))
        return w4a16_gemm_stream_bf16(x, wstream, y, M, K, N, group, stream);
    if (!x || !wstream || !y) return W4A16_ERR_NULL;
    if (group != kGroup) return W4A16_ERR_GROUP;
    if (misaligned(x) || misaligned(wstream) || misaligned(y) || misaligned(scratch)) return W4A16_ERR_ALIGN;
    const size_t need = gemm_wsk_scratch_bytes(M, K, N);
    if (need && (!scratch || scratch_bytes < need)) return W4A16_ERR_WORKSPACE;
    hipError_t e = launch_gemm_wsk(x, wstream, y, nullptr, static_cast<float *>(scratch), M, K, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_gemv_add_stream_bf16(const uint16_t *x, const void *wstream, const uint16_t *residual, uint16_t *y, int K, int N,
                               int group, void *stream) {
    if (!residual) return W4A16_ERR_NULL;
    GemvWsExtras ex;
    ex.residual = residual;
    return gemv_stream_call(x, wstream, nullptr, y, K, N, group, stream, ex);
}

int w4a16_gemv_swiglu_stream_bf16(const uint16_t *x, const void *gate_wstream, const void *up_wstream, uint16_t *h, int K,
                                  int H, int group, void *stream) {
    if (!up_wstream) return W4A16_ERR_NULL;
    return gemv_stream_call(x, gate_wstream, up_wstream, h, K, H, group, stream, GemvWsExtras());
}

int w4a16_rms_gemv_stream_bf16(const uint16_t *x, const float *x_sumsq, int n_pieces, const uint16_t *norm_weight, float eps,
                               const void *wstream, uint16_t *y, int K, int N, int group, void *stream) {
    if (!norm_weight) return W4A16_ERR_NULL;
    GemvWsExtras ex;
    ex.norm_w = norm_weight;
    ex.eps = eps;
    ex.sumsq_in = x_sumsq;
    ex.sumsq_n = x_sumsq ? n_pieces : 0;
    return gemv_stream_call(x, wstream, nullptr, y, K, N, group, stream, ex);
}

int w4a16_rms_gemv_swiglu_stream_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, const void *gate_wstream,
                                      const void *up_wstream, uint16_t *h, int K, int H, int group, void *stream) {
    if (!norm_weight || !up_wstream) return W4A16_ERR_NULL;
    GemvWsExtras ex;
    ex.norm_w = norm_weight;
    ex.eps = eps;
    return gemv_stream_call(x, gate_wstream, up_wstream, h, K, H, group, stream, ex);
}

int w4a16_ffn_swiglu_stream_bf16(const uint16_t *x, const void *gate_wstream, const void *up_wstream, const void *down_wstream,
                                 uint16_t *y, uint16_t *h, int K, int H, int group, void *stream) {
    if (!up_wstream || !down_wstream || !h) return W4A16_ERR_NULL;
    if (H <= 0 || H % kGroup != 0) return W4A16_ERR_SHAPE;
    int rc = gemv_stream_call(x, gate_wstream, up_wstream, h, K, H, group, stream, GemvWsExtras());
    if (rc) return rc;
    return gemv_stream_call(h, down_wstream, nullptr, y, H, K, group, stream, GemvWsExtras());
}

size_t w4a16_block_stream_workspace_bytes(int E, int H) {
    if (E <= 0 || H <= 0) return 0;
    return round256((size_t)E * sizeof(uint16_t)) + round256((size_t)H * sizeof(uint16_t)) +
           round256((size_t)(E / kWsTileCols + 1) * sizeof(float));
}

int w4a16_o_gemv_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                                 float eps, const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                 const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, float *y_sumsq,
                                 int E, int H, int group, void *workspace, size_t workspace_bytes, void *stream) {
    return o_gemv_ffn_stream_impl(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream, down_wstream,
                                  y, res1_out, h_out, y_sumsq, E, H, group, workspace, workspace_bytes, stream, false);
}

int w4a16_decode_attn_o_gemv_ffn_stream_bf16(const uint16_t *qkv, const uint16_t *rope_lut_row, uint16_t *k_cache,
                                             uint16_t *v_cache, uint16_t *attn_out, int pos, int max_seq, int n_heads,
                                             int n_kv_heads, int head_dim, void *attn_workspace, size_t attn_workspace_bytes,
                                             const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                                             const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                             const void *down_wstream, uint16_t *y, float *y_sumsq, int E, int H, int group,
                                             void *workspace, size_t workspace_bytes, void *stream) {
    if (n_heads <= 0 || head_dim <= 0 || n_heads * head_dim != E) return W4A16_ERR_SHAPE;
    int rc = o_gemv_ffn_stream_impl(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream,
                                    down_wstream, y, nullptr, nullptr, y_sumsq, E, H, group, workspace, workspace_bytes, stream,
                                    true);
    if (rc) return rc;
    rc = w4a16_decode_attention_bf16(qkv, rope_lut_row, k_cache, v_cache, attn_out, pos, max_seq, n_heads, n_kv_heads, head_dim,
                                     attn_workspace, attn_workspace_bytes, stream);
    if (rc) return rc;
    return o_gemv_ffn_stream_impl(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream, down_wstream,
                                  y, nullptr, nullptr, y_sumsq, E, H, group, workspace, workspace_bytes, stream, false);
}

size_t w4a16_block_workspace_bytes(int E, int H) {
    if (E <= 0 || H <= 0) return 0;
    const size_t a = stream_partial_bytes(1, H, 2), b = stream_partial_bytes(1, E, 1);
    // [header][partial slots][h bf16 H][res1 bf16 E][sum of squares of res1, one float per column tile, <= 64]
    return kHeaderBytes + (a > b ? a : b) + round256((size_t)H * sizeof(uint16_t)) +
           round256((size_t)E * sizeof(uint16_t)) + 256;
}

int w4a16_o_gemv_ffn_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                          float eps, const int32_t *o_qweight, const int32_t *o_qzeros, const uint16_t *o_scales,
                          const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                          const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                          const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                          uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int E, int H, int group, void *workspace,
                          size_t workspace_bytes, void *stream) {
    return o_gemv_ffn_impl(attn_out, x_residual, ffn_norm_weight, eps, QuantW{o_qweight, o_qzeros, o_scales},
                           QuantW{gate_qweight, gate_qzeros, gate_scales}, QuantW{up_qweight, up_qzeros, up_scales},
                           QuantW{down_qweight, down_qzeros, down_scales}, y, res1_out, h_out, E, H, group, workspace,
                           workspace_bytes, stream);
}

size_t w4a16_prefill_block_workspace_bytes(int M, int E, int H) {
    return prefill_block_supported(M, E, H) ? prefill_block_scratch_bytes(M, E, H) : 0;
}

int rms_norm_rows_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, uint16_t *out, int M, int K,
                       void *stream) {
    if (!x || !norm_weight || !out) return W4A16_ERR_NULL;
    if (!prefill_block_supported(M, K, 8) || !(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(norm_weight) || misaligned(out)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_rmsnorm_rows(x, norm_weight, out, M, K, eps, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

size_t w4a16_prefill_qkv_workspace_bytes(int M, int E) {
    return prefill_block_supported(M, E, 8) ? round256((size_t)M * E * sizeof(uint16_t)) : 0;
}

int w4a16_prefill_rms_qkv_rope_bf16(const uint16_t *x, const uint16_t *attn_norm_weight, float eps,
                                    const int32_t *qkv_qweight, const int32_t *qkv_qzeros, const uint16_t *qkv_scales,
                                    const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out, int M, int E,
                                    int n_heads, int n_kv_heads, int head_dim, int group, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    if (!x || !attn_norm_weight || !rope_lut || !qkv_out) return W4A16_ERR_NULL;
    if (head_dim != 64 && head_dim != 128) return W4A16_ERR_SHAPE;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads > 1024 || n_kv_heads > 1024) return W4A16_ERR_SHAPE;
    const int N = (n_heads + 2 * n_kv_heads) * head_dim;
    int rc = check_quant(qkv_qweight, qkv_qzeros, qkv_scales, E, N, group, 32);
    if (rc) return rc;
    if (!prefill_block_supported(M, E, 8) || !(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (pos0 < 0 || rope_lut_rows <= 0 || pos0 > rope_lut_rows - M) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(attn_norm_weight) || misaligned(rope_lut) || misaligned(qkv_out)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_prefill_qkv_workspace_bytes(M, E)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_prefill_rms_qkv_rope(x, attn_norm_weight, eps, PrefillLinear{qkv_qweight, qkv_qzeros, qkv_scales},
                                               rope_lut, pos0, qkv_out, M, E, n_heads, n_kv_heads, head_dim,
                                               static_cast<uint16_t *>(workspace), static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_prefill_attention_bf16(const uint16_t *qkv, uint16_t *attn_out, int M, int n_heads, int n_kv_heads, int head_dim,
                                 void *stream) {
    if (!qkv || !attn_out) return W4A16_ERR_NULL;
    if (head_dim != 64 && head_dim != 128) return W4A16_ERR_SHAPE;
    if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || n_heads > 65535) return W4A16_ERR_SHAPE;
    if (misaligned(qkv) || misaligned(attn_out)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_prefill_attention(qkv, attn_out, M, n_heads, n_kv_heads, head_dim, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_prefill_o_ffn_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                             float eps, const int32_t *o_qweight, const int32_t *o_qzeros, const uint16_t *o_scales,
                             const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                             const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                             const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                             uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E, int H, int group,
                             void *workspace, size_t workspace_bytes, void *stream) {
    if (!attn_out || !x_residual || !ffn_norm_weight || !y) return W4A16_ERR_NULL;
    int rc = check_quant(o_qweight, o_qzeros, o_scales, E, E, group, 32);
    if (rc) return rc;
    rc = check_quant(gate_qweight, gate_qzeros, gate_scales, E, H, group, 32);
    if (rc) return rc;
    rc = check_quant(up_qweight, up_qzeros, up_scales, E, H, group, 32);
    if (rc) return rc;
    rc = check_quant(down_qweight, down_qzeros, down_scales, H, E, group, 32);
    if (rc) return rc;
    if (!prefill_block_supported(M, E, H) || !(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(attn_out) || misaligned(x_residual) || misaligned(ffn_norm_weight) || misaligned(y) ||
        (res1_out && misaligned(res1_out)) || (h_out && misaligned(h_out)))
        return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_prefill_block_workspace_bytes(M, E, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_prefill_o_ffn(attn_out, x_residual, ffn_norm_weight, eps,
                                        PrefillLinear{o_qweight, o_qzeros, o_scales},
                                        PrefillLinear{gate_qweight, gate_qzeros, gate_scales},
                                        PrefillLinear{up_qweight, up_qzeros, up_scales},
                                        PrefillLinear{down_qweight, down_qzeros, down_scales}, y, res1_out, h_out, M, E,
                                        H, workspace, current_cus(), static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

namespace {
int prefill_qkv_stream_call(const uint16_t *x, const uint16_t *attn_norm_weight, float eps, const void *qkv_wstream,
                            const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out, int M, int E, int n_heads,
                            int n_kv_heads, int head_dim, void *workspace, size_t workspace_bytes, void *stream, bool q4) {
    if (!x || !attn_norm_weight || !qkv_wstream || !rope_lut || !qkv_out) return W4A16_ERR_NULL;
    if (head_dim != 64 && head_dim != 128) return W4A16_ERR_SHAPE;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads > 1024 || n_kv_heads > 1024) return W4A16_ERR_SHAPE;
    const int N = (n_heads + 2 * n_kv_heads) * head_dim;
    if (!prefill_block_supported(M, E, 8) || !gemm_prefill_ws_supported(M, E, N) || !(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (pos0 < 0 || rope_lut_rows <= 0 || pos0 > rope_lut_rows - M) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(attn_norm_weight) || misaligned(qkv_wstream) || misaligned(rope_lut) || misaligned(qkv_out))
        return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_prefill_qkv_workspace_bytes(M, E)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_prefill_rms_qkv_rope_stream(x, attn_norm_weight, eps, qkv_wstream, rope_lut, pos0, qkv_out, M, E, n_heads,
                                                      n_kv_heads, head_dim, static_cast<uint16_t *>(workspace),
                                                      static_cast<hipStream_t>(stream), q4);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int prefill_o_ffn_stream_call(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                              const void *o_wstream, const void *gate_wstream, const void *up_wstream, const void *down_wstream,
                              uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E, int H, void *workspace,
                              size_t workspace_bytes, void *stream, bool q4) {
    if (!attn_out || !x_residual || !ffn_norm_weight || !y || !o_wstream || !gate_wstream || !up_wstream || !down_wstream)
        return W4A16_ERR_NULL;
    if (!prefill_block_stream_supported(M, E, H) || !(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(attn_out) || misaligned(x_residual) || misaligned(ffn_norm_weight) || misaligned(y) || misaligned(o_wstream) ||
        misaligned(gate_wstream) || misaligned(up_wstream) || misaligned(down_wstream) || (res1_out && misaligned(res1_out)) ||
        (h_out && misaligned(h_out)))
        return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_prefill_block_workspace_bytes(M, E, H)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_prefill_o_ffn_stream(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream,
                                               down_wstream, y, res1_out, h_out, M, E, H, workspace, static_cast<hipStream_t>(stream), q4);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}
}  // namespace

int w4a16_prefill_rms_qkv_rope_stream_bf16(const uint16_t *x, const uint16_t *attn_norm_weight, float eps, const void *qkv_wstream,
                                           const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out, int M, int E,
                                           int n_heads, int n_kv_heads, int head_dim, int group, void *workspace,
                                           size_t workspace_bytes, void *stream) {
    if (group != kGroup) return W4A16_ERR_GROUP;
    return prefill_qkv_stream_call(x, attn_norm_weight, eps, qkv_wstream, rope_lut, rope_lut_rows, pos0, qkv_out, M, E, n_heads,
                                   n_kv_heads, head_dim, workspace, workspace_bytes, stream, false);
}

int w4a16_prefill_o_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                                    const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                    const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E,
                                    int H, int group, void *workspace, size_t workspace_bytes, void *stream) {
    if (group != kGroup) return W4A16_ERR_GROUP;
    return prefill_o_ffn_stream_call(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream, down_wstream, y,
                                     res1_out, h_out, M, E, H, workspace, workspace_bytes, stream, false);
}

int w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16(const uint16_t *x, const uint16_t *attn_norm_weight, float eps, const void *qkv_wstream,
                                                const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out, int M,
                                                int E, int n_heads, int n_kv_heads, int head_dim, void *workspace,
                                                size_t workspace_bytes, void *stream) {
    return prefill_qkv_stream_call(x, attn_norm_weight, eps, qkv_wstream, rope_lut, rope_lut_rows, pos0, qkv_out, M, E, n_heads,
                                   n_kv_heads, head_dim, workspace, workspace_bytes, stream, true);
}

int w4a16_q4nx_prefill_o_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                                         float eps, const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                         const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E,
                                         int H, void *workspace, size_t workspace_bytes, void *stream) {
    return prefill_o_ffn_stream_call(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream, down_wstream, y,
                                     res1_out, h_out, M, E, H, workspace, workspace_bytes, stream, true);
}

size_t w4a16_attention_workspace_bytes(int n_heads, int head_dim) {
    if (n_heads <= 0 || head_dim <= 0) return 0;
    return round256(attention_workspace_bytes(n_heads, head_dim));
}

int w4a16_decode_attention_bf16(const uint16_t *qkv, const uint16_t *rope_lut_row, uint16_t *k_cache,
                                uint16_t *v_cache, uint16_t *attn_out, int pos, int max_seq, int n_heads,
                                int n_kv_heads, int head_dim, void *workspace, size_t workspace_bytes, void *stream) {
    if (!qkv || !rope_lut_row || !k_cache || !v_cache || !attn_out) return W4A16_ERR_NULL;
    if (head_dim != 64 && head_dim != 128) return W4A16_ERR_SHAPE;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads) return W4A16_ERR_SHAPE;
    const int g = n_heads / n_kv_heads;
    if (g != 1 && g != 2 && g != 4 && g != 8) return W4A16_ERR_SHAPE;
    if (max_seq <= 0 || pos < 0 || pos >= max_seq) return W4A16_ERR_SHAPE;
    if (misaligned(qkv) || misaligned(rope_lut_row) || misaligned(k_cache) || misaligned(v_cache) || misaligned(attn_out))
        return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < w4a16_attention_workspace_bytes(n_heads, head_dim)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_decode_attention(qkv, rope_lut_row, k_cache, v_cache, attn_out, pos, max_seq, n_heads,
                                           n_kv_heads, head_dim, workspace, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int rope_halfsplit_bf16(const uint16_t *x, const uint16_t *lut, uint16_t *out, int rows, int dim, void *stream) {
    if (!x || !lut || !out) return W4A16_ERR_NULL;
    if (rows <= 0 || dim <= 0 || dim % 16 != 0 || (long long)rows * dim > (1ll << 30)) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(lut) || misaligned(out)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_rope_rows(x, lut, out, rows, dim, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_decode_attn_o_gemv_ffn_bf16(const uint16_t *qkv, const uint16_t *rope_lut_row, uint16_t *k_cache,
                                      uint16_t *v_cache, uint16_t *attn_out, int pos, int max_seq, int n_heads,
                                      int n_kv_heads, int head_dim, void *attn_workspace, size_t attn_workspace_bytes,
                                      const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                                      const int32_t *o_qweight, const int32_t *o_qzeros, const uint16_t *o_scales,
                                      const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                                      const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                                      const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                                      uint16_t *y, float *y_sumsq, int E, int H, int group, void *workspace,
                                      size_t workspace_bytes, void *stream) {
    if (!qkv || !rope_lut_row || !k_cache || !v_cache || !attn_out) return W4A16_ERR_NULL;
    if (y_sumsq && (E % 256 != 0 || E / 256 > 64)) return W4A16_ERR_SHAPE;
    if (y_sumsq && misaligned(y_sumsq)) return W4A16_ERR_ALIGN;
    if (head_dim != 64 && head_dim != 128) return W4A16_ERR_SHAPE;
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || n_heads * head_dim != E) return W4A16_ERR_SHAPE;
    const int g = n_heads / n_kv_heads;
    if (g != 1 && g != 2 && g != 4 && g != 8) return W4A16_ERR_SHAPE;
    if (max_seq <= 0 || pos < 0 || pos >= max_seq) return W4A16_ERR_SHAPE;
    if (misaligned(qkv) || misaligned(rope_lut_row) || misaligned(k_cache) || misaligned(v_cache)) return W4A16_ERR_ALIGN;
    if (!attn_workspace || attn_workspace_bytes < w4a16_attention_workspace_bytes(n_heads, head_dim)) return W4A16_ERR_WORKSPACE;
    if (misaligned(attn_workspace)) return W4A16_ERR_ALIGN;
    const QuantW wo{o_qweight, o_qzeros, o_scales}, wg{gate_qweight, gate_qzeros, gate_scales},
        wu{up_qweight, up_qzeros, up_scales}, wd{down_qweight, down_qzeros, down_scales};
    int rc = o_gemv_ffn_impl(attn_out, x_residual, ffn_norm_weight, eps, wo, wg, wu, wd, y, nullptr, nullptr, E, H,
                             group, workspace, workspace_bytes, stream, nullptr, true);
    if (rc) return rc;
    // With several sequence chunks and an O projection whose units lie inside one head, the projection merges the
    // chunk partials itself and the merge launch is dropped; attn_out is then not written.
    AttnPartials ap;
    ap.nsplit = attention_nsplit(pos + 1);
    ap.hd = head_dim;
    attention_partials(attn_workspace, n_heads, &ap.ml, &ap.acc);
    const bool fuse = !g_stream_tune.no_attn_fuse && stream_attn_fusable(E, E, head_dim, ap.nsplit);
    hipError_t e = launch_decode_attention(qkv, rope_lut_row, k_cache, v_cache, attn_out, pos, max_seq, n_heads, n_kv_heads,
                                           head_dim, attn_workspace, static_cast<hipStream_t>(stream), !fuse);
    if (e != hipSuccess) return hip_fail(e);
    return o_gemv_ffn_impl(attn_out, x_residual, ffn_norm_weight, eps, wo, wg, wu, wd, y, nullptr, nullptr, E, H,
                           group, workspace, workspace_bytes, stream, fuse ? &ap : nullptr, false, y_sumsq);
}

size_t lm_head_workspace_bytes(int V) { return V > 0 ? lm_head_scratch_bytes(V) : 0; }

int lm_head_gemv_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, const uint16_t *lm_head,
                      uint16_t *logits, int32_t *argmax_out, int V, int E, void *workspace, size_t workspace_bytes,
                      void *stream) {
    if (!x || !lm_head || !logits) return W4A16_ERR_NULL;
    if (!lm_head_supported(V, E)) return W4A16_ERR_SHAPE;
    if (norm_weight && !(eps >= 0.f)) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(lm_head) || misaligned(logits) || (norm_weight && misaligned(norm_weight)))
        return W4A16_ERR_ALIGN;
    if (argmax_out && (reinterpret_cast<uintptr_t>(argmax_out) & 3)) return W4A16_ERR_ALIGN;
    if (!workspace || workspace_bytes < lm_head_workspace_bytes(V)) return W4A16_ERR_WORKSPACE;
    if (misaligned(workspace)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_lm_head(x, norm_weight, eps, lm_head, logits, argmax_out, V, E, workspace,
                                  static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int q4nx_dequant_bf16(const void *blocks, uint16_t *out_bf16, int M, int K, int mode, void *stream) {
    if (!blocks || !out_bf16) return W4A16_ERR_NULL;
    if (M <= 0 || K <= 0 || M % 32 != 0 || K % 256 != 0 || mode < 0 || mode > 2) return W4A16_ERR_SHAPE;
    if (misaligned(blocks) || misaligned(out_bf16)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_q4nx_dequant(blocks, out_bf16, M, K, mode, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int q4nx_repack(const void *blocks, int32_t *qweight, uint16_t *scales, uint16_t *mins, int M, int K, int mode,
                void *stream) {
    if (!blocks || !qweight || !scales || !mins) return W4A16_ERR_NULL;
    if (M <= 0 || K <= 0 || M % 32 != 0 || K % 256 != 0 || mode < 0 || mode > 2) return W4A16_ERR_SHAPE;
    if (misaligned(blocks) || misaligned(qweight) || misaligned(scales) || misaligned(mins)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_q4nx_repack(blocks, qweight, scales, mins, M, K, mode, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_q4nx_blocks_to_stream(const void *blocks, void *wstream, int M, int K, int mode, void *stream) {
    if (!blocks || !wstream) return W4A16_ERR_NULL;
    if (M <= 0 || K <= 0 || M % 32 != 0 || K % 256 != 0 || mode < 0 || mode > 2) return W4A16_ERR_SHAPE;
    if (misaligned(blocks) || misaligned(wstream)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_q4nx_blocks_to_stream(blocks, wstream, M, K, mode, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

size_t w4a16_q4nx_stream_bytes(int K, int N) {
    if (K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return 0;
    return ws_q4_matrix_bytes(K, N);
}

int w4a16_q4nx_repack_stream(const int32_t *qweight, const uint16_t *scales, const uint16_t *mins, void *wstream, int K, int N,
                             void *stream) {
    if (!qweight || !scales || !mins || !wstream) return W4A16_ERR_NULL;
    if (K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return W4A16_ERR_SHAPE;
    if (misaligned(qweight) || misaligned(scales) || misaligned(mins) || misaligned(wstream)) return W4A16_ERR_ALIGN;
    hipError_t e = launch_repack_ws_q4(qweight, scales, mins, wstream, K, N, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_q4nx_gemv_stream_bf16(const uint16_t *x, const void *wstream, const uint16_t *residual, uint16_t *y, int K, int N,
                                void *stream) {
    GemvWsExtras ex;
    ex.q4 = true;
    ex.residual = residual;
    return gemv_stream_call(x, wstream, nullptr, y, K, N, kGroup, stream, ex);
}

int w4a16_q4nx_gemm_stream_bf16(const uint16_t *x, const void *wstream, const uint16_t *residual, uint16_t *y, int M, int K, int N,
                                void *stream) {
    if (M == 1) return w4a16_q4nx_gemv_stream_bf16(x, wstream, residual, y, K, N, stream);
    if (!x || !wstream || !y) return W4A16_ERR_NULL;
    if (M <= 0 || K <= 0 || N <= 0 || K % kGroup != 0 || N % kWsTileCols != 0) return W4A16_ERR_SHAPE;
    if (misaligned(x) || misaligned(wstream) || misaligned(y) || (residual && misaligned(residual))) return W4A16_ERR_ALIGN;
    // launches of 16 rows take 13 us each at K = 4096, N = 14336, the tiled kernel ~55 us for up to 256 rows: from 65 rows on
    // the tiled kernel (bf16-rounded weights, as the dense dequant gives them); a residual stays with the launches of 16
    // rows, which add it in fp32 before the one rounding
    const int tiled_min_m = g_gemv_ws_tune.prefill_min_m > 16 ? g_gemv_ws_tune.prefill_min_m : 65;
    hipError_t e = M >= tiled_min_m && !residual && gemm_prefill_ws_supported(M, K, N)
                       ? launch_gemm_prefill_ws(x, wstream, y, M, K, N, static_cast<hipStream_t>(stream), kEpiNone, nullptr, nullptr, true)
                       : launch_gemm_ws(x, wstream, y, residual, M, K, N, static_cast<hipStream_t>(stream), true);
    return e == hipSuccess ? W4A16_OK : hip_fail(e);
}

int w4a16_q4nx_rms_gemv_stream_bf16(const uint16_t *x, const float *x_sumsq, int n_pieces, const uint16_t *norm_weight, float eps,
                                    const void *wstream, uint16_t *y, int K, int N, void *stream) {
    if (!norm_weight) return W4A16_ERR_NULL;
    GemvWsExtras ex;
    ex.q4 = true;
    ex.norm_w = norm_weight;
    ex.eps = eps;
    ex.sumsq_in = x_sumsq;
    ex.sumsq_n = x_sumsq ? n_pieces : 0;
    return gemv_stream_call(x, wstream, nullptr, y, K, N, kGroup, stream, ex);
}

int w4a16_q4nx_o_gemv_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                                      float eps, const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                      const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, float *y_sumsq,
                                      int E, int H, void *workspace, size_t workspace_bytes, void *stream) {
    return o_gemv_ffn_stream_impl(attn_out, x_residual, ffn_norm_weight, eps, o_wstream, gate_wstream, up_wstream, down_wstream,
                                  y, res1_out, h_out, y_sumsq, E, H, kGroup, workspace, workspace_bytes, stream, false, true);
}

int w4a16_tune(const char *key, int value) {
    if (!key || value < 0) return W4A16_ERR_TUNE;
    if (!strcmp(key, "gemv_lw")) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return W4A16_ERR_TUNE;
        g_stream_tune.lw = value;
    } else if (!strcmp(key, "gemv_ksteps")) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return W4A16_ERR_TUNE;
        g_stream_tune.ksteps = value;
    } else if (!strcmp(key, "gemv_waves")) {
        if (value != 0 && value != 4 && value != 8) return W4A16_ERR_TUNE;
        g_stream_tune.waves = value;
    } else if (!strcmp(key, "gemv_skip_publish")) {
        g_stream_tune.skip_publish = value ? 1 : 0;
    } else if (!strcmp(key, "gemv_spin_limit")) {
        g_stream_tune.spin_limit = value;
    } else if (!strcmp(key, "attn_fuse")) {
        g_stream_tune.no_attn_fuse = value ? 0 : 1;
    } else if (!strcmp(key, "gemm_stream_max_m")) {
        g_stream_tune.stream_max_m = value;
    } else if (!strcmp(key, "gemv_ws_ct")) {
        if (value != 0 && value != 4 && value != 8 && value != 16) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.ct = value;
    } else if (!strcmp(key, "prefill_tile")) {
        if (value > 5) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.prefill_tile = value;
    } else if (!strcmp(key, "prefill_swiglu_split")) {
        if (value != 0 && value != 1) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.prefill_swiglu_split = value;
    } else if (!strcmp(key, "gemm_splitk")) {
        if (value < 0 || value > 2) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.splitk = value;
    } else if (!strcmp(key, "prefill_band")) {
        if (value > 64) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.prefill_band = value;
    } else if (!strcmp(key, "prefill_min_m")) {
        g_gemv_ws_tune.prefill_min_m = value;
    } else if (!strcmp(key, "gemm_ws_rows")) {
        if (value != 0 && value != 16 && value != 32 && value != 64) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.gemm_rows = value;
    } else if (!strcmp(key, "gemm_ws_cb")) {
        if (value != 0 && value != 1 && value != 2 && value != 4) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.cb = value;
    } else if (!strcmp(key, "gemv_ws_waves")) {
        if (value > 16) return W4A16_ERR_TUNE;
        g_gemv_ws_tune.waves = value;
    } else if (!strcmp(key, "noalloc_forget")) {
        noalloc_forget();
    } else if (!strcmp(key, "gemv_ksplit")) {
        if (value > kMaxKSplit) return W4A16_ERR_TUNE;
        g_stream_tune.ksplit = value;
    } else if (!strcmp(key, "gemv_units")) {
        if (value > 64) return W4A16_ERR_TUNE;
        g_stream_tune.units = value;
    } else {
        return W4A16_ERR_TUNE;
    }
    return W4A16_OK;
}

}  // extern "C"
