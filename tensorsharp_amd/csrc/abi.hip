// C-ABI shim of libTsHipOps: argument validation, error convention, device weight cache and
// host<->device staging around the gfx950 kernels.  Entry points and their contracts mirror
// the reference bridge (TensorSharp.GGML.Native/ggml_ops_core.cpp, ggml_ops_matmul.cpp);
// see include/tship_ops.h for the export-by-export mapping.
#include "../../include/tship_ops.h"
#include "tship_internal.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace tship {

// ---- error convention: thread-local message, like ggml_ops_core.cpp:89-97 -------------------
static thread_local std::string g_last_error;

void set_last_error(const std::string& msg) { g_last_error = msg; }
void clear_last_error() { g_last_error.clear(); }

bool hip_ok(hipError_t e, const char* what)
{
    if (e == hipSuccess) return true;
    set_last_error(std::string(what) + ": " + hipGetErrorString(e));
    return false;
}

// Dynamic LDS above 64 KiB has to be allowed per kernel and device; the attribute call costs tens of
// microseconds on the host, so the largest size granted so far is remembered.
bool raise_lds_limit(const void* kern, size_t lds)
{
    if (lds <= 64 * 1024) return true;
    struct Granted { const void* kern; int dev; size_t bytes; };
    static std::mutex mu;
    static std::vector<Granted> granted;
    int dev = 0;
    if (!hip_ok(hipGetDevice(&dev), "current device")) return false;
    std::lock_guard<std::mutex> lock(mu);
    Granted* slot = nullptr;
    for (auto& g : granted)
        if (g.kern == kern && g.dev == dev) slot = &g;
    if (slot && slot->bytes >= lds) return true;
    if (!hip_ok(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "raising the dynamic LDS limit"))
        return false;
    if (slot) slot->bytes = lds;
    else granted.push_back({kern, dev, lds});
    return true;
}

// ---- backend state ----------------------------------------------------------------------------
namespace {

std::once_flag g_init_once;
bool g_backend_ready = false;
std::string g_init_error;
DeviceInfo g_device_info{256, 64 * 1024};
// The stream of the *Device entry points is a property of the calling thread (two host threads can drive two streams).
thread_local hipStream_t t_stream = nullptr;

bool probe_device(std::string& err, DeviceInfo* info)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        err = "No HIP device is available.";
        return false;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) {
        (void)hipGetLastError();
        err = "hipGetDeviceProperties failed.";
        return false;
    }
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        err = std::string("libTsHipOps is built for gfx950 only; device 0 is ") + prop.gcnArchName + ".";
        return false;
    }
    if (info) {
        info->num_cus = prop.multiProcessorCount;
        info->lds_per_block_optin = prop.sharedMemPerBlockOptin ? prop.sharedMemPerBlockOptin : prop.sharedMemPerBlock;
    }
    return true;
}

// One backend per process, initialised once (ggml_ops_core.cpp:169-195).
bool ensure_backend()
{
    std::call_once(g_init_once, [] {
        g_backend_ready = probe_device(g_init_error, &g_device_info);
        if (g_backend_ready && hipSetDevice(0) != hipSuccess) {
            g_backend_ready = false;
            g_init_error = "hipSetDevice(0) failed.";
        }
    });
    if (!g_backend_ready) set_last_error(g_init_error);
    return g_backend_ready;
}

// ---- device copies of weights ---------------------------------------------------------------
// Keyed by the pointer the caller passes as m2_data: either the key given to
// TSHip_PreloadQuantizedWeight or the host address of the raw blocks (cached on first use,
// like the bridge's host-buffer cache, ggml_ops_core.cpp:580-663).
struct CachedWeight {
    void* dev = nullptr;
    size_t bytes = 0;
    bool preloaded = false;
};
std::mutex g_cache_mutex;
std::unordered_map<const void*, CachedWeight> g_weight_cache;

// Serialises the host-pointer entry points: they share one staging workspace, and a device copy may only be freed
// (re-upload at another size, Invalidate, Clear) while no host call is between resolving its weights and the end of its
// kernels.  Every host entry point takes it before it resolves a weight and holds it until its results are back.
// Order: g_host_call_mutex, then g_cache_mutex.
std::recursive_mutex g_host_call_mutex;

struct Workspace {
    void* dev = nullptr;
    size_t dev_bytes = 0;
    void* pinned = nullptr;
    size_t pinned_bytes = 0;
};
Workspace g_ws;

// Scratch of the *Device entry points (converted activations and K-chunk sums of the prefill GEMM, intermediate rows of
// the fused wrappers, MoE tables): one grow-only buffer PER STREAM, so calls on different streams never share scratch.
// A call holds its stream's buffer (WsLease) while it enqueues its kernels; since kernels of one stream run in order,
// two threads that use the same stream are then safe too.  After the first call of a given size on a stream nothing
// is allocated any more.  Growing waits for the stream's earlier work (it may still use the old buffer).
struct StreamWs {
    std::mutex mu;
    void* ptr = nullptr;
    size_t bytes = 0;
};
std::mutex g_dev_ws_mutex;                                   // guards the map, not the buffers
std::unordered_map<hipStream_t, StreamWs*> g_dev_ws;         // entries live until the process ends

class WsLease {
public:
    WsLease(hipStream_t stream, size_t bytes)
    {
        {
            std::lock_guard<std::mutex> lock(g_dev_ws_mutex);
            StreamWs*& slot = g_dev_ws[stream];
            if (!slot) slot = new StreamWs();
            ws_ = slot;
        }
        ws_->mu.lock();
        if (bytes > ws_->bytes) {
            if (ws_->ptr) {
                if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return;
                (void)hipFree(ws_->ptr);
            }
            ws_->ptr = nullptr;
            ws_->bytes = 0;
            const size_t want = bytes + bytes / 4;
            if (!hip_ok(hipMalloc(&ws_->ptr, want), "hipMalloc(device workspace)")) return;
            ws_->bytes = want;
        }
        ptr_ = static_cast<char*>(ws_->ptr);
        ok_ = bytes == 0 || ptr_ != nullptr;
    }
    ~WsLease() { ws_->mu.unlock(); }
    WsLease(const WsLease&) = delete;
    WsLease& operator=(const WsLease&) = delete;
    bool ok() const { return ok_; }
    char* ptr() const { return ptr_; }

private:
    StreamWs* ws_ = nullptr;
    char* ptr_ = nullptr;
    bool ok_ = false;
};

bool ws_reserve(size_t dev_bytes, size_t pinned_bytes)
{
    if (dev_bytes > g_ws.dev_bytes) {
        if (g_ws.dev) (void)hipFree(g_ws.dev);
        g_ws.dev = nullptr;
        g_ws.dev_bytes = 0;
        const size_t want = dev_bytes + dev_bytes / 4;
        if (!hip_ok(hipMalloc(&g_ws.dev, want), "hipMalloc(workspace)")) return false;
        g_ws.dev_bytes = want;
    }
    if (pinned_bytes > g_ws.pinned_bytes) {
        if (g_ws.pinned) (void)hipHostFree(g_ws.pinned);
        g_ws.pinned = nullptr;
        g_ws.pinned_bytes = 0;
        const size_t want = pinned_bytes + pinned_bytes / 4;
        if (!hip_ok(hipHostMalloc(&g_ws.pinned, want, hipHostMallocDefault), "hipHostMalloc(workspace)")) return false;
        g_ws.pinned_bytes = want;
    }
    return true;
}

// ---- descriptor checks (ggml_ops_core.cpp:222-229 required_raw_bytes, :302-330 validate_desc) ----
size_t required_raw_bytes(const TSHipTensorView2D& d)
{
    const int64_t max_off = ((int64_t)d.dim0 - 1) * d.stride0 + ((int64_t)d.dim1 - 1) * d.stride1;
    return (size_t)((max_off + 1) * (int64_t)sizeof(float));
}

bool validate_desc(const TSHipTensorView2D& d, const char* name)
{
    if (d.data == nullptr) {
        set_last_error(std::string("Null pointer passed for ") + name + '.');
        return false;
    }
    if (d.dim0 <= 0 || d.dim1 <= 0) {
        set_last_error(std::string("Invalid tensor shape passed for ") + name + '.');
        return false;
    }
    if (d.stride0 < 0 || d.stride1 < 0) {
        set_last_error(std::string("Negative tensor strides are not supported for ") + name + '.');
        return false;
    }
    if (d.raw_bytes <= 0 || (d.raw_bytes % (int64_t)sizeof(float)) != 0) {
        set_last_error(std::string("Invalid raw byte size passed for ") + name + '.');
        return false;
    }
    if ((size_t)d.raw_bytes < required_raw_bytes(d)) {
        set_last_error(std::string("Raw byte span is too small for ") + name + '.');
        return false;
    }
    return true;
}

// stride1 == 1 and rows do not overlap (ggml_ops_core.cpp:441-445 can_map_standard_view)
bool is_standard_view(const TSHipTensorView2D& d)
{
    return d.stride1 == 1 && (d.dim0 == 1 || d.stride0 >= d.dim1);
}

// The *Device entry points index their operands in place: an output whose rows overlap or an input with a
// non-unit inner stride would silently give wrong numbers, so both are refused (the host forms pack such views).
bool check_device_views(const TSHipTensorView2D& out, const TSHipTensorView2D& input)
{
    if (!is_standard_view(out) || input.stride1 != 1) {
        set_last_error("Device addmm_quant needs stride1 == 1 views.");
        return false;
    }
    return true;
}

size_t row_size(int type, int64_t ne)
{
    const int64_t bs = block_elems(type);
    if (bs <= 0 || ne <= 0 || ne % bs != 0) return 0;
    return (size_t)(ne / bs * block_bytes(type));
}

const char* const kUnsupportedTypeMessage =
    "Unsupported weight type for the HIP backend (supported: Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q4_K, Q5_K, Q6_K, IQ4_NL, MXFP4, "
    "F32, F16, BF16).";

// shape agreement + weight descriptor, messages as in ggml_ops_matmul.cpp:303-329
bool validate_addmm_quant(const TSHipTensorView2D& result, const TSHipTensorView2D& m1, const void* m2_data, int type,
                          int64_t ne0, int64_t ne1, int64_t raw_bytes)
{
    if (!validate_desc(result, "result") || !validate_desc(m1, "m1")) return false;
    if (m2_data == nullptr || ne0 <= 0 || ne1 <= 0 || raw_bytes <= 0) {
        set_last_error("Invalid quantized weight descriptor.");
        return false;
    }
    if (m1.dim0 != result.dim0) {
        set_last_error("Size mismatch: m1.dim0 != result.dim0 in addmm_quant.");
        return false;
    }
    if (ne0 != m1.dim1 || ne1 != result.dim1) {
        set_last_error("Size mismatch: quantized weight dims don't match in addmm_quant.");
        return false;
    }
    if (!is_matmul_type(type)) {
        set_last_error(kUnsupportedTypeMessage);
        return false;
    }
    const size_t rs = row_size(type, ne0);
    if (rs == 0) {
        set_last_error("Quantized weight row length is not a multiple of the block size.");
        return false;
    }
    if ((size_t)raw_bytes < rs * (size_t)ne1) {
        set_last_error("Quantized weight byte span is too small for its dimensions.");
        return false;
    }
    return true;
}

// alignment the kernels assume for device operands
bool check_device_operands(const TSHipTensorView2D& m1, const void* w, int type)
{
    const uintptr_t wa = reinterpret_cast<uintptr_t>(w);
    const uintptr_t need_align = is_dense_type(type) ? (uintptr_t)block_bytes(type) : type == kTypeQ8_1 ? 1
                                 : (type == kTypeQ4_K || type == kTypeQ5_K) ? 16 : (type == kTypeMXFP4) ? 1 : 2;
    if (wa % need_align != 0) {
        set_last_error("Quantized weight pointer is not aligned for its block type.");
        return false;
    }
    if ((reinterpret_cast<uintptr_t>(m1.data) & 15) != 0 || (m1.dim0 > 1 && (m1.stride0 & 3) != 0)) {
        set_last_error("Activation rows must be 16-byte aligned on the device.");
        return false;
    }
    return true;
}

// ---- one matmul on device operands ------------------------------------------------------------
// The kernels address a weight, and the converted activations of a launch, with 32-bit offsets.  Larger operands are
// cut by rows inside the call, as the bridge does when a buffer passes INT_MAX (ggml_ops_matmul.cpp:331-367): weight
// rows (output columns) in slices below 2 GiB, activation rows in slices whose fp16 copy stays below 2 GiB.
constexpr size_t kQ81SliceBytes = (size_t)32 << 20;

// Results of fewer than this many columns, with more than three rows of activations, go through an exact fp32 copy of
// the (small) weight instead of the matrix cores: the fp16 operands of the offset formats carry rounded scale products
// (Q4_K: every result about 7.5e-4 of the results' magnitude off, one sigma), and the row norm that the 1e-3 bound is
// taken against grows with the square root of the columns - on 32 columns a sweep of random cases reached 1.03e-3.
constexpr int kNarrowColumns = 64;

struct MatmulPlan {
    bool gemv;            // decode / tiny batch: one bandwidth-bound GEMV per activation row
    bool narrow;          // few result columns: fp32 copy of the weight + the dense kernel
    int m_step;           // activation rows per launch
    int64_t n_step;       // weight rows per launch
    size_t conv_bytes;    // [row scales][fp16 activations] of one slice of rows (prefill), or the RMSNorm rows (decode)
    size_t chunk_bytes;   // sums of K chunks of one launch
    size_t total() const { return conv_bytes + chunk_bytes; }
};

MatmulPlan plan_matmul(int type, int M, int64_t K, int64_t N, bool norm, bool accumulate)
{
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    MatmulPlan p{};
    const size_t rs = row_size(type, K);
    p.n_step = N;
    if (is_dense_type(type) || type == kTypeQ8_1) {
        // dense weights: one kernel with 64-bit addressing, no conversion of the activations
        p.m_step = M;
        p.conv_bytes = norm ? al((size_t)M * (size_t)K * sizeof(float)) : 0;
        if (type == kTypeQ8_1) {
            // fp32 copies of at most kQ81SliceBytes of weight rows at a time
            p.n_step = std::min<int64_t>(N, std::max<int64_t>(1, (int64_t)(kQ81SliceBytes / ((size_t)K * sizeof(float)))));
            p.chunk_bytes = al((size_t)p.n_step * (size_t)K * sizeof(float));
        }
        return p;
    }
    if (rs * (size_t)N >= (size_t)kMaxOperandBytes) {
        // slices of whole rows; a multiple of 256 rows keeps every slice's first row as aligned as the tensor itself
        p.n_step = std::max<int64_t>(256, (int64_t)((size_t)(kMaxOperandBytes - 1) / rs) / 256 * 256);
    }
    p.gemv = M <= 3 && K <= gemv_max_k(type);
    if (!p.gemv && N < kNarrowColumns) {
        p.narrow = true;
        p.m_step = M;
        p.conv_bytes = norm ? al((size_t)M * (size_t)K * sizeof(float)) : 0;
        p.chunk_bytes = al((size_t)N * (size_t)K * sizeof(float));
        return p;
    }
    if (p.gemv) {
        p.m_step = M;
        // RMSNorm is formed by the GEMV while it stages x (rows up to gemv_rms_max_k()), else by a kernel of its own
        p.conv_bytes = norm && K > gemv_rms_max_k() ? al((size_t)M * (size_t)K * sizeof(float)) : 0;
        return p;
    }
    const size_t kp = (size_t)((K + 63) / 64) * 64;
    p.m_step = (int)std::min<int64_t>(M, std::max<int64_t>(256, ((kMaxOperandBytes - 1) / (int64_t)(kp * 2)) / 256 * 256));
    p.conv_bytes = al(gemm_workspace_bytes(p.m_step, (int)K));
    // the launches of a call differ only in their last, smaller slices: the first one needs the most
    p.chunk_bytes = al(gemm_chunk_ws_bytes(type, p.m_step, (int)std::min<int64_t>(N, p.n_step), (int)K, nullptr, accumulate));
    return p;
}

// bytes of device workspace one matmul needs (norm: RMSNorm prologue on the activations)
size_t matmul_ws_bytes(int type, int M, int64_t K, int64_t N, bool norm, bool accumulate)
{
    return plan_matmul(type, M, K, N, norm, accumulate).total();
}

// result (+)= f(m1) * W^T with f = identity or RMSNorm(eps) * norm_w.  All pointers are device pointers; `ws` has
// ws_bytes >= matmul_ws_bytes() bytes (with fewer, the K-chunk sums are given up first: see launch_gemm).
bool run_matmul_device_ws(const TSHipTensorView2D& result, const TSHipTensorView2D& m1, const void* w, int type, int64_t K,
                          int64_t N, hipStream_t stream, void* ws, size_t ws_bytes, const float* norm_w, float eps, bool accumulate)
{
    const size_t rs = row_size(type, K);
    if (!check_device_operands(m1, w, type)) return false;
    if (norm_w && (reinterpret_cast<uintptr_t>(norm_w) & 15) != 0) {
        set_last_error("The norm weight must be 16-byte aligned on the device.");
        return false;
    }
    const int M = m1.dim0;
    const MatmulPlan plan = plan_matmul(type, M, K, N, norm_w != nullptr, accumulate);
    if (plan.conv_bytes > ws_bytes) {
        set_last_error("matmul: the device workspace is too small for the converted activations.");
        return false;
    }
    const uint8_t* wb = static_cast<const uint8_t*>(w);
    float* out = static_cast<float*>(result.data);
    if (is_dense_type(type) || type == kTypeQ8_1 || plan.narrow) {
        const float* xs = static_cast<const float*>(m1.data);
        int64_t ldx = m1.stride0;
        if (norm_w) {
            if (!launch_rms_norm_rows(xs, ldx, norm_w, eps, M, (int)K, static_cast<float*>(ws), stream)) return false;
            xs = static_cast<const float*>(ws);
            ldx = K;
        }
        if (is_dense_type(type)) return launch_dense_matmul(type, w, xs, ldx, out, result.stride0, M, (int)N, (int)K, accumulate, stream);
        if (plan.total() > ws_bytes) {
            set_last_error("matmul: the device workspace is too small for the fp32 copy of a weight slice.");
            return false;
        }
        float* rows = reinterpret_cast<float*>(static_cast<char*>(ws) + plan.conv_bytes);
        for (int64_t n0 = 0; n0 < N; n0 += plan.n_step) {
            const int64_t n = std::min<int64_t>(plan.n_step, N - n0);
            if (!launch_dequant(type, wb + (size_t)n0 * rs, n * K, rows, stream)) return false;
            if (!launch_dense_matmul(kTypeF32, rows, xs, ldx, out + n0, result.stride0, M, (int)n, (int)K, accumulate, stream)) return false;
        }
        return true;
    }
    if (plan.gemv) {
        const float* xs = static_cast<const float*>(m1.data);
        int64_t ldx = m1.stride0;
        const bool norm_in_gemv = norm_w && K <= gemv_rms_max_k();
        if (norm_w && !norm_in_gemv) {
            if (!launch_rms_norm_rows(xs, ldx, norm_w, eps, M, (int)K, static_cast<float*>(ws), stream)) return false;
            xs = static_cast<const float*>(ws);
            ldx = K;
        }
        for (int64_t n0 = 0; n0 < N; n0 += plan.n_step) {
            const int64_t n = std::min<int64_t>(plan.n_step, N - n0);
            for (int m = 0; m < M; ++m) {
                float* y = out + (int64_t)m * result.stride0 + n0;
                if (!launch_gemv(type, wb + (size_t)n0 * rs, (int64_t)(rs * (size_t)n), xs + (int64_t)m * ldx, y, (int)n, (int)K, stream,
                                 accumulate ? y : nullptr, norm_in_gemv ? 1 : 0, norm_w, eps))
                    return false;
            }
        }
        return true;
    }
    // prefill: activations -> fp16 workspace, then the MFMA GEMM
    char* chunk_ws = static_cast<char*>(ws) + plan.conv_bytes;
    const size_t chunk_bytes = ws_bytes - plan.conv_bytes;
    for (int m0 = 0; m0 < M; m0 += plan.m_step) {
        const int m = std::min(plan.m_step, M - m0);
        const float* x = static_cast<const float*>(m1.data) + (int64_t)m0 * m1.stride0;
        int converted = -1;         // activation layout in the workspace (row slices of an over-large weight may differ)
        for (int64_t n0 = 0; n0 < N; n0 += plan.n_step) {
            const int64_t n = std::min<int64_t>(plan.n_step, N - n0);
            const int layout = gemm_x_layout(type, m, (int)n, (int)K);
            if (layout != converted) {
                if (!launch_convert_x(type, x, m1.stride0, nullptr, m, (int)K, ws, stream, norm_w, eps, layout)) return false;
                converted = layout;
            }
            if (!launch_gemm(type, wb + (size_t)n0 * rs, (int64_t)(rs * (size_t)n), ws, out + (int64_t)m0 * result.stride0 + n0,
                             result.stride0, nullptr, m, (int)n, (int)K, nullptr, stream, accumulate, chunk_ws, chunk_bytes, layout))
                return false;
        }
    }
    return true;
}

bool run_matmul_device(const TSHipTensorView2D& result, const TSHipTensorView2D& m1, const void* w, int type, int64_t K,
                       int64_t N, hipStream_t stream)
{
    const size_t need = matmul_ws_bytes(type, m1.dim0, K, N, false, false);
    WsLease ws(stream, need);
    if (!ws.ok()) return false;
    return run_matmul_device_ws(result, m1, w, type, K, N, stream, ws.ptr(), need, nullptr, 0.f, false);
}

// ---- static device scratch of the entry point that allocates nothing ---------------------------
// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.  In
// host code the array's name is only a handle for hipGetSymbolAddress: the address a kernel may use is looked up
// once per device and kept in g_scratch_ptr.
constexpr size_t kScratchBytes = (size_t)TSHIP_NO_ALLOC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device (looked up on the first call per device)
unsigned char* scratch_ptr()
{
    int dev = 0;
    if (!hip_ok(hipGetDevice(&dev), "current device")) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        set_last_error("Device index out of range for the static scratch buffer.");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (!hip_ok(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
        g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
    }
    return g_scratch_ptr[dev];
}

// FFN of the fused entry points on device operands (ggml_ops_fused.cpp:390-640):
//   residual += W_down * ( silu(g) * u ),  [g | u] = W_gate_up * (RMSNorm(input) * norm_w)
// `ws` has ffn_ws_bytes() bytes.
size_t ffn_ws_bytes(int M, int gu_type, int dn_type, int hidden, int half)
{
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    return al((size_t)M * 2 * half * sizeof(float)) + al((size_t)M * half * sizeof(float)) +
           std::max(matmul_ws_bytes(gu_type, M, hidden, 2 * (int64_t)half, true, false), matmul_ws_bytes(dn_type, M, half, hidden, false, true));
}

bool run_ffn_swiglu_device(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const float* norm_w, float eps,
                           const void* gate_up, int gu_type, const void* down, int dn_type, int hidden, int half,
                           hipStream_t stream, char* ws)
{
    const int M = input.dim0;
    const size_t gu_bytes = ((size_t)M * 2 * half * sizeof(float) + 255) & ~(size_t)255;
    const size_t act_bytes = ((size_t)M * half * sizeof(float) + 255) & ~(size_t)255;
    const size_t mm_bytes = ffn_ws_bytes(M, gu_type, dn_type, hidden, half) - gu_bytes - act_bytes;
    float* gu = reinterpret_cast<float*>(ws);
    float* act = reinterpret_cast<float*>(ws + gu_bytes);
    void* mm_ws = ws + gu_bytes + act_bytes;
    auto streams = [](int type, int64_t rows, int64_t k) {
        return has_gemv(type) && k <= gemv_max_k(type) && row_size(type, k) * (size_t)rows < (size_t)kMaxOperandBytes;
    };
    if (M <= 3 && streams(gu_type, 2 * (int64_t)half, hidden) && streams(dn_type, hidden, half)) {
        // decode, two launches per row: the gate_up GEMV stages RMSNorm(x) * w, computes gate row j and up row j in one
        // wavefront and stores silu(gate_j) * up_j; the down GEMV adds the residual in its store
        if (!check_device_operands(input, gate_up, gu_type) || !check_device_operands(input, down, dn_type)) return false;
        if ((reinterpret_cast<uintptr_t>(norm_w) & 15) != 0) {
            set_last_error("The norm weight must be 16-byte aligned on the device.");
            return false;
        }
        const size_t gu_w_bytes = row_size(gu_type, hidden) * (size_t)(2 * half), dn_w_bytes = row_size(dn_type, half) * (size_t)hidden;
        for (int m = 0; m < M; ++m) {
            GemvArgs a{};
            a.w = gate_up, a.w_bytes = (int64_t)gu_w_bytes, a.x = static_cast<const float*>(input.data) + (int64_t)m * input.stride0;
            a.y = gu + (size_t)m * half, a.N = 2 * half, a.K = hidden, a.act = 1, a.norm_w = norm_w, a.eps = eps, a.pair_rows = half;
            if (!launch_gemv_group(gu_type, 1, &a, stream)) return false;
        }
        for (int m = 0; m < M; ++m) {
            float* y = static_cast<float*>(residual.data) + (int64_t)m * residual.stride0;
            if (!launch_gemv(dn_type, down, (int64_t)dn_w_bytes, gu + (size_t)m * half, y, hidden, half, stream, y, 0, nullptr, 0.f)) return false;
        }
        return true;
    }
    const TSHipTensorView2D gu_view{gu, M, 2 * half, 2 * half, 1, (int64_t)((size_t)M * 2 * half * sizeof(float))};
    if (!run_matmul_device_ws(gu_view, input, gate_up, gu_type, hidden, 2 * half, stream, mm_ws, mm_bytes, norm_w, eps, false)) return false;
    if (!launch_silu_mul(gu, 2 * half, M, half, act, stream)) return false;
    const TSHipTensorView2D act_view{act, M, half, half, 1, (int64_t)((size_t)M * half * sizeof(float))};
    return run_matmul_device_ws(residual, act_view, down, dn_type, half, hidden, stream, mm_ws, mm_bytes, nullptr, 0.f, true);
}

// ---- a weighted set of expert FFNs on device operands ------------------------------------------
// out = (base ? base : 0) + sum_e weight_e * W_down[e] * act_e(x), experts added in index order, with
//   act_e(x) = silu(W_gate[e] x) * (W_up[e] x)      when the expert has a gate weight   (ggml_ops_fused.cpp:1876-1890)
//            = max(W_up[e] x, 0)^2                  when it has none                    (ggml_ops_fused.cpp:1700-1722)
// Every expert maps H -> I -> N.  The routed experts of the bridge calls share their types; a shared expert may differ.
constexpr int kMaxExpertSet = 33;   // 32 routed experts and one shared expert
struct ExpertFfn {
    const void* gate;   // device pointers to raw blocks; gate == nullptr selects the squared-ReLU expert
    const void* up;
    const void* down;
    int gate_type, up_type, down_type;
    float weight;
};

struct ExpertSetLayout {
    size_t act_stride;   // floats between the activation rows of consecutive experts
    size_t dn_stride;    // floats between their down outputs
    size_t act_off, dn_off, tmp_off, mm_off, mm_bytes, total;
    // more than one row, block formats only: every linear of the set is one tile-table GEMM per block type over the experts'
    // pointers (rows e * M .. of the packed [n * M] activation / result matrices belong to expert e)
    bool tiled;
    int bm;              // rows per m-tile
    size_t x1_off, x2_off;        // converted activations of the [n M x H] gathered input and of the [n M x I] gated rows
    size_t tbl_off, tbl_bytes;    // tile tables, offset table, row map
    size_t chunk_off, chunk_bytes;
};

// block formats with a tile-table GEMM
bool has_tile_gemm(int type)
{
    switch (type) {
    case kTypeQ8_0: case kTypeQ4_K: case kTypeMXFP4: case kTypeQ6_K: case kTypeQ5_K:
    case kTypeQ4_0: case kTypeQ4_1: case kTypeQ5_0: case kTypeQ5_1: case kTypeIQ4_NL: return true;
    default: return false;
    }
}

// activation layout of a tile-table launch over expert pointers: MXFP4 on 32-row units reads MX fp6 pairs (rows of at least
// 256 outputs: the error of fp6 pairs against a short row's norm is too close to the 1e-3 bound)
int expert_tiles_x_layout(int type, int bm, int K, int out_features)
{
    return type == kTypeMXFP4 && bm == 32 && K <= 32768 && out_features >= 256 ? 1 : 0;
}

ExpertSetLayout expert_set_layout(int M, int n, const ExpertFfn* ex, int H, int I, int N)
{
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    ExpertSetLayout L{};
    L.act_stride = al((size_t)M * 2 * I * sizeof(float)) / sizeof(float);
    L.dn_stride = al((size_t)M * N * sizeof(float)) / sizeof(float);
    L.act_off = 0;
    L.dn_off = L.act_off + (size_t)n * L.act_stride * sizeof(float);
    L.tmp_off = L.dn_off + (size_t)n * L.dn_stride * sizeof(float);
    L.mm_off = L.tmp_off + al((size_t)M * I * sizeof(float));
    for (int e = 0; e < n; ++e) {
        if (ex[e].gate) L.mm_bytes = std::max(L.mm_bytes, matmul_ws_bytes(ex[e].gate_type, M, H, I, false, false));
        L.mm_bytes = std::max(L.mm_bytes, matmul_ws_bytes(ex[e].up_type, M, H, I, false, false));
        L.mm_bytes = std::max(L.mm_bytes, matmul_ws_bytes(ex[e].down_type, M, I, N, false, false));
    }
    L.total = L.mm_off + L.mm_bytes;
    // the tiled form
    const int64_t rows = (int64_t)n * M;
    bool tiled = M > 1 && rows <= 65535;
    for (int e = 0; e < n && tiled; ++e) {
        auto fits = [](int type, int64_t wrows, int64_t k) {
            return has_tile_gemm(type) && row_size(type, k) * (size_t)wrows < (size_t)kMaxOperandBytes;
        };
        tiled = (ex[e].gate != nullptr) == (ex[0].gate != nullptr) && fits(ex[e].up_type, I, H) && fits(ex[e].down_type, N, I) &&
                (!ex[e].gate || fits(ex[e].gate_type, I, H));
    }
    tiled = tiled && gemm_workspace_bytes((int)rows, std::max(H, I)) < (size_t)kMaxOperandBytes;
    if (!tiled) return L;
    L.tiled = true;
    L.bm = M > 160 ? 128 : 32;
    const int ld = ex[0].gate ? 2 * I : I;
    L.act_stride = (size_t)M * ld;
    L.dn_stride = (size_t)M * N;
    const int max_tiles = n * ((M + L.bm - 1) / L.bm);
    size_t off = 0;
    auto take = [&](size_t b) { const size_t o = off; off += al(b); return o; };
    L.act_off = take((size_t)rows * ld * sizeof(float));
    L.dn_off = take((size_t)rows * N * sizeof(float));
    L.tmp_off = take((size_t)rows * I * sizeof(float));
    L.x1_off = take(gemm_workspace_bytes((int)rows, H));
    L.x2_off = take(gemm_workspace_bytes((int)rows, I));
    L.tbl_bytes = al((size_t)max_tiles * 4) * 3 + al((size_t)n * 8) + al((size_t)rows * 4);
    L.tbl_off = take(L.tbl_bytes);
    const GemmTiles plan_tiles{nullptr, nullptr, nullptr, max_tiles, L.bm, 0};
    for (int e = 0; e < n; ++e) {
        auto need = [&](int type, int nn, int kk) {
            return gemm_chunk_ws_bytes(type, (int)rows, nn, kk, &plan_tiles, false, expert_tiles_x_layout(type, L.bm, kk, nn));
        };
        if (ex[e].gate) L.chunk_bytes = std::max(L.chunk_bytes, need(ex[e].gate_type, I, H));
        L.chunk_bytes = std::max(L.chunk_bytes, need(ex[e].up_type, I, H));
        L.chunk_bytes = std::max(L.chunk_bytes, need(ex[e].down_type, N, I));
    }
    L.chunk_off = take(L.chunk_bytes);
    L.mm_off = off, L.mm_bytes = 0;
    L.total = off;
    return L;
}

// One linear of a tiled expert set: per block type one tile-table GEMM over the members whose weight has that type.
// x: fp32 source rows (ldx), gathered through row_map when given; the members' results go to rows slot * M .. of c.
struct ExpertLinear {
    const void* w[kMaxExpertSet];
    int type[kMaxExpertSet];
};

bool run_expert_linear_tiled(const ExpertSetLayout& L, char* ws, int n, int M, const ExpertLinear& lin, const float* x, int64_t ldx,
                             bool gather, size_t x_off, float* c, int64_t ldc, int out_features, int K, hipStream_t stream)
{
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const int per = (M + L.bm - 1) / L.bm;
    const size_t tile_bytes = al((size_t)n * per * 4);
    int* t_expert = reinterpret_cast<int*>(ws + L.tbl_off);
    int* t_row0 = reinterpret_cast<int*>(ws + L.tbl_off + tile_bytes);
    int* t_rows = reinterpret_cast<int*>(ws + L.tbl_off + 2 * tile_bytes);
    int64_t* offs = reinterpret_cast<int64_t*>(ws + L.tbl_off + 3 * tile_bytes);
    int* row_map = reinterpret_cast<int*>(ws + L.tbl_off + 3 * tile_bytes + al((size_t)n * 8));
    const int rows = n * M;
    bool handled[kMaxExpertSet] = {};
    for (int first = 0; first < n; ++first) {
        if (handled[first]) continue;
        const int t = lin.type[first];
        // base pointer: the lowest address among the type's members, so that every offset is >= 0
        uintptr_t base = reinterpret_cast<uintptr_t>(lin.w[first]);
        for (int e = first; e < n; ++e)
            if (lin.type[e] == t) base = std::min(base, reinterpret_cast<uintptr_t>(lin.w[e]));
        ExpertTileSpec spec{};
        for (int e = first; e < n; ++e) {
            if (lin.type[e] != t) continue;
            handled[e] = true;
            spec.off[spec.count] = (int64_t)(reinterpret_cast<uintptr_t>(lin.w[e]) - base);
            spec.slot[spec.count] = e;
            ++spec.count;
        }
        const int layout = expert_tiles_x_layout(t, L.bm, K, out_features);
        if (!launch_expert_tiles(spec, M, L.bm, t_expert, t_row0, t_rows, offs, gather ? row_map : nullptr, rows, stream)) return false;
        if (!launch_convert_x(t, x, ldx, gather ? row_map : nullptr, rows, K, ws + x_off, stream, nullptr, 0.f, layout)) return false;
        GemmTiles tiles{t_expert, t_row0, t_rows, spec.count * per, L.bm, (int64_t)(row_size(t, K) * (size_t)out_features)};
        tiles.expert_off = offs;
        if (!launch_gemm(t, reinterpret_cast<const void*>(base), tiles.expert_stride, ws + x_off, c, ldc, nullptr, rows, out_features, K, &tiles,
                         stream, false, L.chunk_bytes ? ws + L.chunk_off : nullptr, L.chunk_bytes, layout))
            return false;
    }
    return true;
}

// problems of one block type, at most gemv_max_group() per launch
bool launch_gemv_batches(int type, std::vector<GemvArgs>& list, hipStream_t stream)
{
    const int group = gemv_max_group();
    for (size_t i = 0; i < list.size(); i += (size_t)group)
        if (!launch_gemv_group(type, (int)std::min<size_t>((size_t)group, list.size() - i), list.data() + i, stream)) return false;
    return true;
}

bool run_expert_set_device(const TSHipTensorView2D& out, const float* base, int64_t ldb, const TSHipTensorView2D& x, int n,
                           const ExpertFfn* ex, int H, int I, int N, hipStream_t stream, char* ws)
{
    const int M = x.dim0;
    const ExpertSetLayout L = expert_set_layout(M, n, ex, H, I, N);
    float* act = reinterpret_cast<float*>(ws + L.act_off);
    float* dn = reinterpret_cast<float*>(ws + L.dn_off);
    float* tmp = reinterpret_cast<float*>(ws + L.tmp_off);
    void* mm_ws = ws + L.mm_off;
    WeightedSumCoeffs coeffs{};
    for (int e = 0; e < n; ++e) coeffs.v[e] = ex[e].weight;

    // single token, every format with a GEMV: the experts' linears run as grouped GEMV launches
    bool grouped = M == 1;
    for (int e = 0; e < n && grouped; ++e) {
        auto fits = [](int type, int64_t rows, int64_t k) {
            return has_gemv(type) && k <= gemv_max_k(type) && row_size(type, k) * (size_t)rows < (size_t)kMaxOperandBytes;
        };
        grouped = fits(ex[e].up_type, I, H) && fits(ex[e].down_type, N, I) && (!ex[e].gate || fits(ex[e].gate_type, I, H));
    }
    if (grouped) {
        const float* xv = static_cast<const float*>(x.data);
        const int types[] = {kTypeQ8_0, kTypeQ4_K, kTypeMXFP4, kTypeQ6_K, kTypeQ5_K, kTypeQ4_0, kTypeQ4_1, kTypeQ5_0, kTypeQ5_1, kTypeIQ4_NL};
        for (int e = 0; e < n; ++e)
            if (!check_device_operands(x, ex[e].up, ex[e].up_type) || !check_device_operands(x, ex[e].down, ex[e].down_type) ||
                (ex[e].gate && !check_device_operands(x, ex[e].gate, ex[e].gate_type)))
                return false;
        std::vector<GemvArgs> list;
        for (int t : types) {      // gate and up projections: x -> act[e] = [gate | up] (or [up] alone)
            list.clear();
            for (int e = 0; e < n; ++e) {
                float* row = act + (size_t)e * L.act_stride;
                if (ex[e].gate && ex[e].gate_type == t) {
                    GemvArgs a{};
                    a.w = ex[e].gate, a.w_bytes = (int64_t)(row_size(t, H) * (size_t)I), a.x = xv, a.y = row, a.N = I, a.K = H;
                    list.push_back(a);
                }
                if (ex[e].up_type == t) {
                    GemvArgs a{};
                    a.w = ex[e].up, a.w_bytes = (int64_t)(row_size(t, H) * (size_t)I), a.x = xv, a.y = ex[e].gate ? row + I : row, a.N = I, a.K = H;
                    list.push_back(a);
                }
            }
            if (!launch_gemv_batches(t, list, stream)) return false;
        }
        for (int e = 0; e < n; ++e)
            if (!ex[e].gate && !launch_relu_sqr(act + (size_t)e * L.act_stride, I, stream)) return false;
        for (int t : types)        // down projections; the gated product is formed while the activation row is staged
            for (int gated = 0; gated < 2; ++gated) {
                list.clear();
                for (int e = 0; e < n; ++e) {
                    if (ex[e].down_type != t || (ex[e].gate != nullptr) != (gated != 0)) continue;
                    GemvArgs a{};
                    a.w = ex[e].down, a.w_bytes = (int64_t)(row_size(t, I) * (size_t)N), a.x = act + (size_t)e * L.act_stride;
                    a.y = dn + (size_t)e * L.dn_stride, a.N = N, a.K = I, a.act = gated ? 2 : 0;
                    list.push_back(a);
                }
                if (!launch_gemv_batches(t, list, stream)) return false;
            }
    } else if (L.tiled) {
        // several rows, block formats: gate, up and down are one tile-table GEMM each (per block type) over the experts'
        // pointers; the M input rows are gathered once per expert into the [n M x H] activations
        for (int e = 0; e < n; ++e)
            if (!check_device_operands(x, ex[e].up, ex[e].up_type) || !check_device_operands(x, ex[e].down, ex[e].down_type) ||
                (ex[e].gate && !check_device_operands(x, ex[e].gate, ex[e].gate_type)))
                return false;
        const bool gated = ex[0].gate != nullptr;
        const int ld = gated ? 2 * I : I;
        const float* xv = static_cast<const float*>(x.data);
        ExpertLinear lin{};
        if (gated) {
            for (int e = 0; e < n; ++e) lin.w[e] = ex[e].gate, lin.type[e] = ex[e].gate_type;
            if (!run_expert_linear_tiled(L, ws, n, M, lin, xv, x.stride0, true, L.x1_off, act, ld, I, H, stream)) return false;
        }
        for (int e = 0; e < n; ++e) lin.w[e] = ex[e].up, lin.type[e] = ex[e].up_type;
        if (!run_expert_linear_tiled(L, ws, n, M, lin, xv, x.stride0, true, L.x1_off, gated ? act + I : act, ld, I, H, stream)) return false;
        const float* rows_in = act;
        if (gated) {
            if (!launch_silu_mul(act, ld, n * M, I, tmp, stream)) return false;
            rows_in = tmp;
        } else if (!launch_relu_sqr(act, (int64_t)n * M * I, stream)) {
            return false;
        }
        for (int e = 0; e < n; ++e) lin.w[e] = ex[e].down, lin.type[e] = ex[e].down_type;
        if (!run_expert_linear_tiled(L, ws, n, M, lin, rows_in, I, false, L.x2_off, dn, N, N, I, stream)) return false;
    } else {
        for (int e = 0; e < n; ++e) {
            float* a_e = act + (size_t)e * L.act_stride;
            float* d_e = dn + (size_t)e * L.dn_stride;
            const TSHipTensorView2D d_view{d_e, M, N, N, 1, (int64_t)((size_t)M * N * sizeof(float))};
            if (ex[e].gate) {
                const int64_t span = (int64_t)(((size_t)(M - 1) * 2 * I + I) * sizeof(float));
                const TSHipTensorView2D g_view{a_e, M, I, 2 * I, 1, span};
                const TSHipTensorView2D u_view{a_e + I, M, I, 2 * I, 1, span};
                if (!run_matmul_device_ws(g_view, x, ex[e].gate, ex[e].gate_type, H, I, stream, mm_ws, L.mm_bytes, nullptr, 0.f, false)) return false;
                if (!run_matmul_device_ws(u_view, x, ex[e].up, ex[e].up_type, H, I, stream, mm_ws, L.mm_bytes, nullptr, 0.f, false)) return false;
                if (!launch_silu_mul(a_e, 2 * I, M, I, tmp, stream)) return false;
                const TSHipTensorView2D t_view{tmp, M, I, I, 1, (int64_t)((size_t)M * I * sizeof(float))};
                if (!run_matmul_device_ws(d_view, t_view, ex[e].down, ex[e].down_type, I, N, stream, mm_ws, L.mm_bytes, nullptr, 0.f, false)) return false;
            } else {
                const TSHipTensorView2D u_view{a_e, M, I, I, 1, (int64_t)((size_t)M * I * sizeof(float))};
                if (!run_matmul_device_ws(u_view, x, ex[e].up, ex[e].up_type, H, I, stream, mm_ws, L.mm_bytes, nullptr, 0.f, false)) return false;
                if (!launch_relu_sqr(a_e, (int64_t)M * I, stream)) return false;
                if (!run_matmul_device_ws(d_view, u_view, ex[e].down, ex[e].down_type, I, N, stream, mm_ws, L.mm_bytes, nullptr, 0.f, false)) return false;
            }
        }
    }
    return launch_weighted_sum(dn, (int64_t)L.dn_stride, coeffs, n, M, N, base, ldb, static_cast<float*>(out.data), out.stride0, stream);
}

// Device pointer for m2_data: preloaded key, cached host pointer, or upload now.  The caller holds g_host_call_mutex.
// Hit rules: a copy made from caller memory on first use is reused only for exactly the same byte count (the bridge's
// rule, ggml_ops_core.cpp:604-640: a host address reused for a tensor of another size is uploaded again); a preloaded
// entry serves any view that fits into the bytes it was given (preload takes the caller's raw byte span, which may
// exceed rows x row size) and is never re-read from the key, which need not be readable memory.
const void* resolve_weight(void* m2_data, size_t bytes)
{
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_weight_cache.find(m2_data);
    if (it != g_weight_cache.end()) {
        if (it->second.preloaded) {
            if (bytes <= it->second.bytes) return it->second.dev;
            set_last_error("Preloaded quantized weight is smaller than the requested view.");
            return nullptr;
        }
        if (it->second.bytes == bytes) return it->second.dev;
        (void)hipFree(it->second.dev);
        g_weight_cache.erase(it);
    }
    CachedWeight cw;
    if (!hip_ok(hipMalloc(&cw.dev, bytes + 16), "hipMalloc(weight)")) return nullptr;
    if (!hip_ok(hipMemcpy(cw.dev, m2_data, bytes, hipMemcpyHostToDevice), "hipMemcpy(weight)")) {
        (void)hipFree(cw.dev);
        return nullptr;
    }
    cw.bytes = bytes;
    g_weight_cache[m2_data] = cw;
    return cw.dev;
}

// Sub-weight [offset, offset + bytes) of a stacked weight (AddmmQuantBatch): served from the device copy of the whole
// stack when `base` is a preloaded key or an already cached host pointer that covers the range - a deliberate range
// hit, the key need not be readable; otherwise the sub-weight is cached under its own host address like any weight.
const void* resolve_weight_range(void* base, size_t offset, size_t bytes)
{
    {
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        auto it = g_weight_cache.find(base);
        if (it != g_weight_cache.end() && offset + bytes <= it->second.bytes) return static_cast<const char*>(it->second.dev) + offset;
    }
    return resolve_weight(static_cast<char*>(base) + offset, bytes);
}

// w_dev_given: the device copy when the caller has resolved the weight already (sub-weights of a stack)
int addmm_quant_host(const TSHipTensorView2D& result, const TSHipTensorView2D& m1, void* m2_data, int type, int64_t ne0,
                     int64_t ne1, int64_t raw_bytes, const void* w_dev_given = nullptr)
{
    if (!ensure_backend()) return 0;
    if (!validate_addmm_quant(result, m1, m2_data, type, ne0, ne1, raw_bytes)) return 0;
    if (!is_standard_view(result)) {
        set_last_error("result must be a standard (stride1 == 1, non-overlapping) view in addmm_quant.");
        return 0;
    }
    const int M = m1.dim0;
    const int64_t K = ne0, N = ne1;
    const size_t w_bytes = row_size(type, K) * (size_t)N;
    std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
    const void* w_dev = w_dev_given ? w_dev_given : resolve_weight(m2_data, w_bytes);
    if (!w_dev) return 0;
    const size_t x_bytes = (size_t)M * K * sizeof(float);
    const size_t y_bytes = (size_t)M * N * sizeof(float);
    const size_t x_off = 0, y_off = (x_bytes + 255) & ~(size_t)255;
    if (!ws_reserve(y_off + y_bytes, std::max(x_bytes, y_bytes))) return 0;
    float* x_dev = reinterpret_cast<float*>(static_cast<char*>(g_ws.dev) + x_off);
    float* y_dev = reinterpret_cast<float*>(static_cast<char*>(g_ws.dev) + y_off);

    // pack the (possibly strided) activation view into pinned memory, then one H2D copy
    float* stage = static_cast<float*>(g_ws.pinned);
    const float* src = static_cast<const float*>(m1.data);
    if (m1.stride1 == 1) {
        for (int m = 0; m < M; ++m) std::memcpy(stage + (size_t)m * K, src + (size_t)m * m1.stride0, (size_t)K * sizeof(float));
    } else {
        for (int m = 0; m < M; ++m)
            for (int64_t k = 0; k < K; ++k) stage[(size_t)m * K + k] = src[(size_t)m * m1.stride0 + (size_t)k * m1.stride1];
    }
    hipStream_t stream = nullptr;
    if (!hip_ok(hipMemcpyAsync(x_dev, stage, x_bytes, hipMemcpyHostToDevice, stream), "hipMemcpy(activations)")) return 0;

    TSHipTensorView2D r_dev{y_dev, M, (int)N, (int)N, 1, (int64_t)y_bytes};
    TSHipTensorView2D x_desc{x_dev, M, (int)K, (int)K, 1, (int64_t)x_bytes};
    if (!run_matmul_device(r_dev, x_desc, w_dev, type, K, N, stream)) return 0;

    if (!hip_ok(hipMemcpyAsync(stage, y_dev, y_bytes, hipMemcpyDeviceToHost, stream), "hipMemcpy(result)")) return 0;
    if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
    float* dst = static_cast<float*>(result.data);
    for (int m = 0; m < M; ++m) std::memcpy(dst + (size_t)m * result.stride0, stage + (size_t)m * N, (size_t)N * sizeof(float));
    clear_last_error();
    return 1;
}

}  // namespace

const DeviceInfo& device_info() { return g_device_info; }

}  // namespace tship

using namespace tship;

// Nothing unwinds across the ABI (ggml_ops_matmul.cpp:1317-1336 pattern).
template <typename F>
static int guarded(int fallback, const char* what, F&& body)
{
    try {
        return body();
    } catch (const std::exception& ex) {
        set_last_error(ex.what());
        return fallback;
    } catch (...) {
        set_last_error(std::string("Unknown HIP ") + what + " failure.");
        return fallback;
    }
}

// ---- helpers of the fused entry points ---------------------------------------------------------
namespace {

bool validate_weight(const void* data, int type, int64_t ne0, int64_t ne1, int64_t raw_bytes, const char* what)
{
    if (data == nullptr || ne0 <= 0 || ne1 <= 0 || raw_bytes <= 0) {
        set_last_error(std::string("Invalid quantized weight descriptor for ") + what + ".");
        return false;
    }
    if (!is_matmul_type(type)) {
        set_last_error(kUnsupportedTypeMessage);
        return false;
    }
    const size_t rs = row_size(type, ne0);
    if (rs == 0) {
        set_last_error("Quantized weight row length is not a multiple of the block size.");
        return false;
    }
    if ((size_t)raw_bytes < rs * (size_t)ne1) {
        set_last_error("Quantized weight byte span is too small for its dimensions.");
        return false;
    }
    return true;
}

bool validate_fused_matmul(const TSHipTensorView2D& out, const TSHipTensorView2D& input, const void* norm_w, int norm_count,
                           bool with_norm, const void* w, int type, int64_t ne0, int64_t ne1, int64_t raw_bytes, const char* what,
                           const char* out_name)
{
    if (!validate_desc(out, out_name) || !validate_desc(input, "input")) return false;
    if (with_norm && (norm_w == nullptr || norm_count <= 0)) {
        set_last_error("Invalid norm weight data.");
        return false;
    }
    if (!validate_weight(w, type, ne0, ne1, raw_bytes, what)) return false;
    if (out.dim0 != input.dim0) {
        set_last_error(std::string("Size mismatch: ") + out_name + ".dim0 != input.dim0 in " + what + ".");
        return false;
    }
    if (ne0 != input.dim1 || ne1 != out.dim1 || (with_norm && norm_count != input.dim1)) {
        set_last_error(std::string("Size mismatch: weight dims don't match in ") + what + ".");
        return false;
    }
    if (out.stride1 != 1) {
        set_last_error(std::string(out_name) + " must be a standard (stride1 == 1) view in " + what + ".");
        return false;
    }
    return true;
}

bool validate_ffn(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const void* norm_w, int norm_count,
                  const void* gu, int gu_type, int64_t gu_ne0, int64_t gu_ne1, int64_t gu_bytes, const void* dn, int dn_type,
                  int64_t dn_ne0, int64_t dn_ne1, int64_t dn_bytes, int half_dim)
{
    if (!validate_desc(residual, "residual") || !validate_desc(input, "input")) return false;
    if (norm_w == nullptr || norm_count <= 0) {
        set_last_error("fused_ffn_swiglu: invalid norm weight.");
        return false;
    }
    if (!validate_weight(gu, gu_type, gu_ne0, gu_ne1, gu_bytes, "fused_ffn_swiglu gate_up")) return false;
    if (!validate_weight(dn, dn_type, dn_ne0, dn_ne1, dn_bytes, "fused_ffn_swiglu down")) return false;
    const int hidden = input.dim1;
    if (residual.dim0 != input.dim0 || residual.dim1 != hidden) {
        set_last_error("fused_ffn_swiglu: residual shape mismatch.");
        return false;
    }
    if (norm_count != hidden) {
        set_last_error("fused_ffn_swiglu: norm_weight_count != hidden.");
        return false;
    }
    if (gu_ne0 != hidden) {
        set_last_error("fused_ffn_swiglu: gate_up.ne0 != hidden.");
        return false;
    }
    if (half_dim <= 0 || gu_ne1 != 2 * (int64_t)half_dim) {
        set_last_error("fused_ffn_swiglu: gate_up.ne1 != 2*half_dim.");
        return false;
    }
    if (dn_ne0 != half_dim || dn_ne1 != hidden) {
        set_last_error("fused_ffn_swiglu: down weight shape mismatch.");
        return false;
    }
    if (residual.stride1 != 1) {
        set_last_error("fused_ffn_swiglu: residual must be a standard (stride1 == 1) view.");
        return false;
    }
    return true;
}

// Host tensors around a device computation: `input` (any non-negative-stride view) and optionally the current
// contents of `inout` go up, `inout` comes back.  body(input_dev_view, inout_dev_view, norm_dev, stream).
template <typename Body>
int with_host_tensors(const TSHipTensorView2D& inout, bool upload_inout, const TSHipTensorView2D& input, const void* norm_w,
                      int norm_count, Body&& body)
{
    if (!is_standard_view(inout)) {
        set_last_error("The result / residual tensor must be a standard (stride1 == 1, non-overlapping) view.");
        return 0;
    }
    std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
    const int M = input.dim0;
    const size_t K = (size_t)input.dim1, N = (size_t)inout.dim1;
    const size_t x_bytes = ((size_t)M * K * sizeof(float) + 255) & ~(size_t)255;
    const size_t y_bytes = ((size_t)M * N * sizeof(float) + 255) & ~(size_t)255;
    const size_t n_bytes = ((size_t)std::max(norm_count, 0) * sizeof(float) + 255) & ~(size_t)255;
    if (!ws_reserve(x_bytes + y_bytes + n_bytes, x_bytes + y_bytes + n_bytes)) return 0;
    char* dev = static_cast<char*>(g_ws.dev);
    char* pin = static_cast<char*>(g_ws.pinned);
    float* stage_x = reinterpret_cast<float*>(pin);
    float* stage_y = reinterpret_cast<float*>(pin + x_bytes);
    float* stage_n = reinterpret_cast<float*>(pin + x_bytes + y_bytes);
    const float* src = static_cast<const float*>(input.data);
    for (int m = 0; m < M; ++m)
        for (size_t k = 0; k < K; ++k) stage_x[(size_t)m * K + k] = src[(size_t)m * input.stride0 + k * (size_t)input.stride1];
    float* io = static_cast<float*>(inout.data);
    if (upload_inout)
        for (int m = 0; m < M; ++m) std::memcpy(stage_y + (size_t)m * N, io + (size_t)m * inout.stride0, N * sizeof(float));
    if (norm_w) std::memcpy(stage_n, norm_w, (size_t)norm_count * sizeof(float));
    hipStream_t stream = nullptr;
    const size_t up = upload_inout ? x_bytes + y_bytes + (norm_w ? n_bytes : 0) : x_bytes;
    if (!hip_ok(hipMemcpyAsync(dev, pin, up, hipMemcpyHostToDevice, stream), "hipMemcpy(inputs)")) return 0;
    if (!upload_inout && norm_w &&
        !hip_ok(hipMemcpyAsync(dev + x_bytes + y_bytes, stage_n, n_bytes, hipMemcpyHostToDevice, stream), "hipMemcpy(norm weight)"))
        return 0;
    const TSHipTensorView2D x_dev{dev, M, (int)K, (int)K, 1, (int64_t)((size_t)M * K * sizeof(float))};
    const TSHipTensorView2D y_dev{dev + x_bytes, M, (int)N, (int)N, 1, (int64_t)((size_t)M * N * sizeof(float))};
    if (!body(x_dev, y_dev, norm_w ? reinterpret_cast<const float*>(dev + x_bytes + y_bytes) : nullptr, stream)) return 0;
    if (!hip_ok(hipMemcpyAsync(stage_y, dev + x_bytes, (size_t)M * N * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpy(result)"))
        return 0;
    if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
    for (int m = 0; m < M; ++m) std::memcpy(io + (size_t)m * inout.stride0, stage_y + (size_t)m * N, N * sizeof(float));
    clear_last_error();
    return 1;
}

// Several host tensors around a device computation.  Each tensor is packed to [dim0 x dim1] in one pinned region,
// the region goes up in one copy, body(dev_views, norm_dev, stream) runs, the region comes back in one copy and the
// tensors marked `down` are written to the caller's views.
struct HostTensor {
    const TSHipTensorView2D* view;
    bool up;
    bool down;
};

template <typename Body>
int with_host_io(const HostTensor* t, int count, const void* norm_w, int norm_count, Body&& body)
{
    constexpr int kMaxIo = 6;
    if (count > kMaxIo) {
        set_last_error("Too many host tensors in one call.");
        return 0;
    }
    std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    size_t off[kMaxIo + 1], total = 0;
    for (int i = 0; i < count; ++i) {
        off[i] = total;
        total += al((size_t)t[i].view->dim0 * (size_t)t[i].view->dim1 * sizeof(float));
    }
    off[count] = total;
    total += al((size_t)std::max(norm_count, 0) * sizeof(float));
    if (!ws_reserve(total, total)) return 0;
    char* dev = static_cast<char*>(g_ws.dev);
    char* pin = static_cast<char*>(g_ws.pinned);
    TSHipTensorView2D dv[kMaxIo];
    for (int i = 0; i < count; ++i) {
        const TSHipTensorView2D& v = *t[i].view;
        dv[i] = TSHipTensorView2D{dev + off[i], v.dim0, v.dim1, v.dim1, 1, (int64_t)((size_t)v.dim0 * (size_t)v.dim1 * sizeof(float))};
        if (!t[i].up) continue;
        float* stage = reinterpret_cast<float*>(pin + off[i]);
        const float* src = static_cast<const float*>(v.data);
        for (int m = 0; m < v.dim0; ++m) {
            if (v.stride1 == 1) {
                std::memcpy(stage + (size_t)m * v.dim1, src + (size_t)m * v.stride0, (size_t)v.dim1 * sizeof(float));
            } else {
                for (int k = 0; k < v.dim1; ++k) stage[(size_t)m * v.dim1 + k] = src[(size_t)m * v.stride0 + (size_t)k * v.stride1];
            }
        }
    }
    if (norm_w) std::memcpy(pin + off[count], norm_w, (size_t)norm_count * sizeof(float));
    hipStream_t stream = nullptr;
    for (int i = 0; i <= count; ++i) {
        const bool wanted = i < count ? t[i].up : norm_w != nullptr;
        const size_t bytes = i < count ? (size_t)dv[i].raw_bytes : (size_t)std::max(norm_count, 0) * sizeof(float);
        if (wanted && !hip_ok(hipMemcpyAsync(dev + off[i], pin + off[i], bytes, hipMemcpyHostToDevice, stream), "hipMemcpy(inputs)")) return 0;
    }
    if (!body(dv, norm_w ? reinterpret_cast<const float*>(dev + off[count]) : nullptr, stream)) return 0;
    for (int i = 0; i < count; ++i)
        if (t[i].down && !hip_ok(hipMemcpyAsync(pin + off[i], dev + off[i], (size_t)dv[i].raw_bytes, hipMemcpyDeviceToHost, stream), "hipMemcpy(result)"))
            return 0;
    if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
    for (int i = 0; i < count; ++i) {
        if (!t[i].down) continue;
        const TSHipTensorView2D& v = *t[i].view;
        const float* stage = reinterpret_cast<const float*>(pin + off[i]);
        float* dst = static_cast<float*>(v.data);
        for (int m = 0; m < v.dim0; ++m) {
            if (v.stride1 == 1) {
                std::memcpy(dst + (size_t)m * v.stride0, stage + (size_t)m * v.dim1, (size_t)v.dim1 * sizeof(float));
            } else {
                for (int k = 0; k < v.dim1; ++k) dst[(size_t)m * v.stride0 + (size_t)k * v.stride1] = stage[(size_t)m * v.dim1 + k];
            }
        }
    }
    clear_last_error();
    return 1;
}

struct WeightDesc {
    const void* data;
    int type;
    int64_t ne0, ne1, raw_bytes;
    size_t bytes() const { return row_size(type, ne0) * (size_t)ne1; }
};

// residual [M x hidden] += input [M x ne0] * W_out^T, then (ffn) the SwiGLU FFN on the new residual
bool validate_outproj(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const WeightDesc& out_w, const void* norm_w,
                      int norm_count, const char* what)
{
    if (!validate_desc(residual, "residual") || !validate_desc(input, "input")) return false;
    if (!validate_weight(out_w.data, out_w.type, out_w.ne0, out_w.ne1, out_w.raw_bytes, what)) return false;
    if (norm_w == nullptr || norm_count <= 0) {
        set_last_error(std::string(what) + ": invalid norm weight.");
        return false;
    }
    if (residual.dim0 != input.dim0 || out_w.ne0 != input.dim1 || out_w.ne1 != residual.dim1 || norm_count != residual.dim1) {
        set_last_error(std::string(what) + ": shape mismatch between residual, input, the output projection and the norm weight.");
        return false;
    }
    if (residual.stride1 != 1) {
        set_last_error(std::string(what) + ": residual must be a standard (stride1 == 1) view.");
        return false;
    }
    return true;
}

bool validate_outproj_ffn(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const WeightDesc& out_w, const void* norm_w,
                          int norm_count, const WeightDesc& gu, const WeightDesc& dn, int half_dim)
{
    if (!validate_outproj(residual, input, out_w, norm_w, norm_count, "fused_outproj_ffn")) return false;
    if (!validate_weight(gu.data, gu.type, gu.ne0, gu.ne1, gu.raw_bytes, "fused_outproj_ffn gate_up")) return false;
    if (!validate_weight(dn.data, dn.type, dn.ne0, dn.ne1, dn.raw_bytes, "fused_outproj_ffn down")) return false;
    const int hidden = residual.dim1;
    if (half_dim <= 0 || gu.ne0 != hidden || gu.ne1 != 2 * (int64_t)half_dim || dn.ne0 != half_dim || dn.ne1 != hidden) {
        set_last_error("fused_outproj_ffn: gate_up / down weight shape mismatch.");
        return false;
    }
    return true;
}

size_t outproj_ffn_ws_bytes(int M, const WeightDesc& out_w, const WeightDesc& gu, const WeightDesc& dn, int hidden, int half)
{
    return std::max(matmul_ws_bytes(out_w.type, M, out_w.ne0, out_w.ne1, false, true), ffn_ws_bytes(M, gu.type, dn.type, hidden, half));
}

bool run_outproj_ffn_device(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const void* out_w, const WeightDesc& od,
                            const float* norm_w, float eps, const void* gu, int gu_type, const void* dn, int dn_type, int half,
                            hipStream_t stream, char* ws, size_t ws_bytes)
{
    if (!run_matmul_device_ws(residual, input, out_w, od.type, od.ne0, od.ne1, stream, ws, ws_bytes, nullptr, 0.f, true)) return false;
    return run_ffn_swiglu_device(residual, residual, norm_w, eps, gu, gu_type, dn, dn_type, residual.dim1, half, stream, ws);
}

bool validate_outproj_router(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const WeightDesc& out_w, const void* norm_w,
                             int norm_count, const TSHipTensorView2D& normed_out, const WeightDesc& router, const TSHipTensorView2D& router_out)
{
    if (!validate_outproj(residual, input, out_w, norm_w, norm_count, "fused_outproj_norm_router")) return false;
    if (!validate_desc(normed_out, "normedOut") || !validate_desc(router_out, "routerOut")) return false;
    if (!validate_weight(router.data, router.type, router.ne0, router.ne1, router.raw_bytes, "fused_outproj_norm_router router")) return false;
    const int hidden = residual.dim1;
    if (normed_out.dim0 != residual.dim0 || normed_out.dim1 != hidden || router_out.dim0 != residual.dim0 || router.ne0 != hidden ||
        router.ne1 != router_out.dim1) {
        set_last_error("fused_outproj_norm_router: normedOut / router shape mismatch.");
        return false;
    }
    return true;
}

size_t outproj_router_ws_bytes(int M, const WeightDesc& out_w, const WeightDesc& router)
{
    return std::max(matmul_ws_bytes(out_w.type, M, out_w.ne0, out_w.ne1, false, true), matmul_ws_bytes(router.type, M, router.ne0, router.ne1, false, false));
}

// residual += input * W_out^T; normed_out = RMSNorm(residual) * norm_w; router_out = normed_out * W_router^T
// (ggml_ops_fused.cpp:1310-1330).  normed_out must be a contiguous [M x hidden] device view.
bool run_outproj_router_device(const TSHipTensorView2D& residual, const TSHipTensorView2D& input, const void* out_w, const WeightDesc& od,
                               const float* norm_w, float eps, const TSHipTensorView2D& normed_out, const void* router_w,
                               const WeightDesc& rd, const TSHipTensorView2D& router_out, hipStream_t stream, char* ws, size_t ws_bytes)
{
    if (normed_out.stride1 != 1 || (normed_out.dim0 > 1 && normed_out.stride0 != normed_out.dim1) || router_out.stride1 != 1) {
        set_last_error("fused_outproj_norm_router: normedOut must be contiguous and routerOut a standard view on the device.");
        return false;
    }
    if (!run_matmul_device_ws(residual, input, out_w, od.type, od.ne0, od.ne1, stream, ws, ws_bytes, nullptr, 0.f, true)) return false;
    if (!launch_rms_norm_rows(static_cast<const float*>(residual.data), residual.stride0, norm_w, eps, residual.dim0, residual.dim1,
                              static_cast<float*>(normed_out.data), stream))
        return false;
    return run_matmul_device_ws(router_out, normed_out, router_w, rd.type, rd.ne0, rd.ne1, stream, ws, ws_bytes, nullptr, 0.f, false);
}

// ---- weighted expert sets (the bridge's per-token MoE calls) ------------------------------------
struct ExpertSetArgs {
    const char* what;
    int max_experts;
    int num_experts;
    bool gated;            // SwiGLU experts (gate, up, down); otherwise squared-ReLU experts (up, down)
    void* const* gate;
    void* const* up;
    void* const* down;
    WeightDesc gate_d, up_d, down_d;     // data unused; shapes shared by the routed experts
    const float* route_weights;
    bool has_shared;
    WeightDesc sh_gate, sh_up, sh_down;
    float shared_scalar;
};

bool validate_expert_set(const TSHipTensorView2D& out, const TSHipTensorView2D& input, const ExpertSetArgs& a, const char* out_name)
{
    if (!validate_desc(out, out_name) || !validate_desc(input, "input")) return false;
    if (a.num_experts <= 0 || a.num_experts > a.max_experts) {
        set_last_error(std::string(a.what) + ": num_experts must be 1.." + std::to_string(a.max_experts));
        return false;
    }
    if ((a.gated && a.gate == nullptr) || a.up == nullptr || a.down == nullptr || a.route_weights == nullptr) {
        set_last_error(std::string(a.what) + ": null expert pointer array or route weights.");
        return false;
    }
    const std::string w = a.what;
    for (int e = 0; e < a.num_experts; ++e) {
        if (a.gate && !validate_weight(a.gate[e], a.gate_d.type, a.gate_d.ne0, a.gate_d.ne1, a.gate_d.raw_bytes, (w + " gate").c_str())) return false;
        if (!validate_weight(a.up[e], a.up_d.type, a.up_d.ne0, a.up_d.ne1, a.up_d.raw_bytes, (w + " up").c_str())) return false;
        if (!validate_weight(a.down[e], a.down_d.type, a.down_d.ne0, a.down_d.ne1, a.down_d.raw_bytes, (w + " down").c_str())) return false;
    }
    const int64_t H = input.dim1, I = a.up_d.ne1, N = out.dim1;
    bool ok = out.dim0 == input.dim0 && a.up_d.ne0 == H && a.down_d.ne0 == I && a.down_d.ne1 == N &&
              (!a.gate || (a.gate_d.ne0 == H && a.gate_d.ne1 == I));
    if (a.has_shared) {
        if (!validate_weight(a.sh_gate.data, a.sh_gate.type, a.sh_gate.ne0, a.sh_gate.ne1, a.sh_gate.raw_bytes, (w + " shared gate").c_str()) ||
            !validate_weight(a.sh_up.data, a.sh_up.type, a.sh_up.ne0, a.sh_up.ne1, a.sh_up.raw_bytes, (w + " shared up").c_str()) ||
            !validate_weight(a.sh_down.data, a.sh_down.type, a.sh_down.ne0, a.sh_down.ne1, a.sh_down.raw_bytes, (w + " shared down").c_str()))
            return false;
        // the shared expert may have its own intermediate width
        ok = ok && a.sh_gate.ne0 == H && a.sh_up.ne0 == H && a.sh_gate.ne1 == a.sh_up.ne1 && a.sh_down.ne0 == a.sh_up.ne1 && a.sh_down.ne1 == N;
    }
    if (!ok) {
        set_last_error(w + ": weight shapes do not match the input / output tensors.");
        return false;
    }
    if (out.stride1 != 1) {
        set_last_error(w + ": the output must be a standard (stride1 == 1) view.");
        return false;
    }
    return true;
}

// Runs a validated expert set on device views; `resolve` maps a caller pointer to the device address of its blocks.
// The shared expert runs as a set of its own (its width may differ) and is added after the routed experts.
template <typename Resolve>
bool run_expert_set(const TSHipTensorView2D& out, bool add_to_out, const TSHipTensorView2D& x, const ExpertSetArgs& a, hipStream_t stream,
                    Resolve&& resolve)
{
    ExpertFfn ex[kMaxExpertSet];
    const int n = a.num_experts;
    for (int e = 0; e < n; ++e) {
        ex[e].gate = a.gate ? resolve(a.gate[e], a.gate_d.bytes()) : nullptr;
        ex[e].up = resolve(a.up[e], a.up_d.bytes());
        ex[e].down = resolve(a.down[e], a.down_d.bytes());
        if ((a.gate && !ex[e].gate) || !ex[e].up || !ex[e].down) return false;
        ex[e].gate_type = a.gate_d.type, ex[e].up_type = a.up_d.type, ex[e].down_type = a.down_d.type;
        ex[e].weight = a.route_weights[e];
    }
    const int M = x.dim0, H = x.dim1, I = (int)a.up_d.ne1, N = out.dim1;
    const bool same_width = a.has_shared && a.sh_up.ne1 == a.up_d.ne1;
    ExpertFfn sh{};
    if (a.has_shared) {
        sh.gate = resolve(const_cast<void*>(a.sh_gate.data), a.sh_gate.bytes());
        sh.up = resolve(const_cast<void*>(a.sh_up.data), a.sh_up.bytes());
        sh.down = resolve(const_cast<void*>(a.sh_down.data), a.sh_down.bytes());
        if (!sh.gate || !sh.up || !sh.down) return false;
        sh.gate_type = a.sh_gate.type, sh.up_type = a.sh_up.type, sh.down_type = a.sh_down.type;
        sh.weight = a.shared_scalar;
    }
    int count = n;
    if (same_width) ex[count++] = sh;     // one weighted sum over routed + shared, in the bridge's order
    const size_t need = std::max(expert_set_layout(M, count, ex, H, I, N).total,
                                 a.has_shared && !same_width ? expert_set_layout(M, 1, &sh, H, (int)a.sh_up.ne1, N).total : (size_t)0);
    WsLease ws(stream, need);
    if (!ws.ok()) return false;
    const float* base = add_to_out ? static_cast<const float*>(out.data) : nullptr;
    if (a.has_shared && !same_width) {
        // (routed sum) + shared, then + residual: the shared term is added into a copy-free second pass on `out`
        if (!run_expert_set_device(out, base, out.stride0, x, n, ex, H, I, N, stream, ws.ptr())) return false;
        return run_expert_set_device(out, static_cast<const float*>(out.data), out.stride0, x, 1, &sh, H, (int)a.sh_up.ne1, N, stream, ws.ptr());
    }
    return run_expert_set_device(out, base, out.stride0, x, count, ex, H, I, N, stream, ws.ptr());
}

}  // namespace

extern "C" {

const char* TSHip_GetLastError(void) { return g_last_error.c_str(); }

int TSHip_CanInitializeBackend(int backendType)
{
    clear_last_error();
    if (backendType != TSHIP_BACKEND_HIP) return 0;
    std::string err;
    if (probe_device(err, nullptr)) return 1;
    set_last_error(err);
    return 0;
}

int TSHip_IsBackendAvailable(int backendType)
{
    clear_last_error();
    if (backendType != TSHIP_BACKEND_HIP) {
        set_last_error("libTsHipOps provides the HIP backend only.");
        return 0;
    }
    return ensure_backend() ? 1 : 0;
}

size_t TSHip_RowSize(int ggml_type, int64_t ne) { return row_size(ggml_type, ne); }

void* TSHip_AlignedAlloc(size_t size)
{
    if (size == 0) return nullptr;
    void* p = nullptr;
    if (posix_memalign(&p, 16384, size) != 0) return nullptr;
    return p;
}

void TSHip_AlignedFree(void* ptr)
{
    if (ptr) free(ptr);
}

int TSHip_SetStream(void* hip_stream)
{
    t_stream = static_cast<hipStream_t>(hip_stream);
    clear_last_error();
    return 1;
}

int TSHip_SetGemvTimeline(void* device_buffer, int64_t capacity_bytes)
{
    const int64_t per_wave = (int64_t)gemv_timeline_slots() * (int64_t)sizeof(uint64_t);
    if (device_buffer != nullptr && (capacity_bytes < per_wave || (reinterpret_cast<uintptr_t>(device_buffer) & 7) != 0)) {
        set_last_error("gemv timeline: the buffer must be 8-byte aligned device memory of at least 64 bytes per wavefront.");
        return 0;
    }
    set_gemv_timeline(static_cast<uint64_t*>(device_buffer), device_buffer ? capacity_bytes / per_wave : 0);
    clear_last_error();
    return 1;
}

int TSHip_DequantizeToF32Device(int ggml_type, const void* src, int64_t num_elements, float* dst)
{
    return guarded(-1, "dequantize", [&]() -> int {
        if (src == nullptr || dst == nullptr || num_elements < 0) return -1;
        if (num_elements == 0) return 0;
        if (ggml_type != kTypeF32 && !is_dequant_type(ggml_type)) return -2;
        if (!ensure_backend()) return -1;
        if (ggml_type == kTypeF32)
            return hip_ok(hipMemcpyAsync(dst, src, (size_t)num_elements * 4, hipMemcpyDeviceToDevice, t_stream),
                          "hipMemcpy")
                       ? 0
                       : -1;
        if (num_elements % block_elems(ggml_type) != 0) return -1;
        return launch_dequant(ggml_type, src, num_elements, dst, t_stream) ? 0 : -1;
    });
}

int TSHip_DequantizeToF32(int ggml_type, const void* src, int64_t num_elements, float* dst)
{
    return guarded(-1, "dequantize", [&]() -> int {
        if (src == nullptr || dst == nullptr || num_elements < 0) return -1;
        if (num_elements == 0) return 0;
        if (ggml_type == kTypeF32) {
            std::memcpy(dst, src, (size_t)num_elements * sizeof(float));
            return 0;
        }
        if (!is_dequant_type(ggml_type)) return -2;
        if (num_elements % block_elems(ggml_type) != 0) return -1;
        if (!ensure_backend()) return -1;
        const size_t in_bytes = row_size(ggml_type, num_elements);
        const size_t out_bytes = (size_t)num_elements * sizeof(float);
        std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
        const size_t out_off = (in_bytes + 255) & ~(size_t)255;
        if (!ws_reserve(out_off + out_bytes, 0)) return -1;
        char* base = static_cast<char*>(g_ws.dev);
        if (!hip_ok(hipMemcpy(base, src, in_bytes, hipMemcpyHostToDevice), "hipMemcpy(src)")) return -1;
        if (!launch_dequant(ggml_type, base, num_elements, reinterpret_cast<float*>(base + out_off), nullptr)) return -1;
        if (!hip_ok(hipMemcpy(dst, base + out_off, out_bytes, hipMemcpyDeviceToHost), "hipMemcpy(dst)")) return -1;
        return 0;
    });
}

int TSHip_AddmmQuantF32Device(TSHipTensorView2D result, TSHipTensorView2D m1, const void* m2_data, int m2_ggml_type,
                              int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "addmm_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_addmm_quant(result, m1, m2_data, m2_ggml_type, m2_ne0, m2_ne1, m2_raw_bytes)) return 0;
        if (!check_device_views(result, m1)) return 0;
        if (!run_matmul_device(result, m1, m2_data, m2_ggml_type, m2_ne0, m2_ne1, t_stream)) return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_AddmmQuantF32DeviceNoAlloc(TSHipTensorView2D result, TSHipTensorView2D m1, const void* m2_data, int m2_ggml_type,
                                     int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "addmm_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_addmm_quant(result, m1, m2_data, m2_ggml_type, m2_ne0, m2_ne1, m2_raw_bytes)) return 0;
        if (!check_device_views(result, m1)) return 0;
        // [converted activations + row scales][sums of K chunks]: both live in the static array
        const size_t need = plan_matmul(m2_ggml_type, m1.dim0, m2_ne0, m2_ne1, false, false).conv_bytes;
        if (need > kScratchBytes) {
            set_last_error("addmm_quant (no-alloc): the converted activations of this call (" + std::to_string(need) +
                           " bytes) exceed the static scratch buffer of " + std::to_string(kScratchBytes) +
                           " bytes; use fewer rows per call or TSHip_AddmmQuantF32Device.");
            return 0;
        }
        unsigned char* ws = scratch_ptr();
        if (!ws) return 0;
        // what the converted activations leave of the array takes the sums of K chunks
        if (!run_matmul_device_ws(result, m1, m2_data, m2_ggml_type, m2_ne0, m2_ne1, t_stream, ws, kScratchBytes, nullptr, 0.f, false))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_AddmmQuantGroupF32Device(int count, const TSHipTensorView2D* results, const TSHipTensorView2D* m1s,
                                   const void* const* m2_datas, int m2_ggml_type, const int64_t* m2_ne0s,
                                   const int64_t* m2_ne1s, const int64_t* m2_raw_bytes)
{
    return guarded(0, "addmm_quant_group", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (count <= 0 || !results || !m1s || !m2_datas || !m2_ne0s || !m2_ne1s || !m2_raw_bytes) {
            set_last_error("Invalid arguments for addmm_quant_group.");
            return 0;
        }
        bool decode = count <= gemv_max_group();
        for (int i = 0; i < count; ++i) {
            if (!validate_addmm_quant(results[i], m1s[i], m2_datas[i], m2_ggml_type, m2_ne0s[i], m2_ne1s[i],
                                      m2_raw_bytes[i]))
                return 0;
            if (!check_device_views(results[i], m1s[i])) return 0;
            if (!check_device_operands(m1s[i], m2_datas[i], m2_ggml_type)) return 0;
            decode = decode && m1s[i].dim0 == 1 && m2_ne0s[i] <= gemv_max_k(m2_ggml_type);
        }
        hipStream_t stream = t_stream;
        if (decode) {
            GemvArgs args[16];
            for (int i = 0; i < count; ++i) {
                args[i].w = m2_datas[i];
                args[i].w_bytes = (int64_t)(row_size(m2_ggml_type, m2_ne0s[i]) * (size_t)m2_ne1s[i]);
                args[i].x = static_cast<const float*>(m1s[i].data);
                args[i].y = static_cast<float*>(results[i].data);
                args[i].N = (int)m2_ne1s[i];
                args[i].K = (int)m2_ne0s[i];
            }
            if (!launch_gemv_group(m2_ggml_type, count, args, stream)) return 0;
        } else {
            for (int i = 0; i < count; ++i)
                if (!run_matmul_device(results[i], m1s[i], m2_datas[i], m2_ggml_type, m2_ne0s[i], m2_ne1s[i], stream))
                    return 0;
        }
        clear_last_error();
        return 1;
    });
}

int TSHip_MoERouteF32Device(TSHipTensorView2D logits, int k, int32_t* ids, float* weights)
{
    return guarded(0, "moe_route", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_desc(logits, "logits")) return 0;
        if (ids == nullptr || weights == nullptr || logits.stride1 != 1) {
            set_last_error("Invalid arguments for moe_route.");
            return 0;
        }
        if (!launch_moe_route(static_cast<const float*>(logits.data), logits.stride0, logits.dim0, logits.dim1, k, ids, weights,
                              t_stream))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_MoEExpertsGptOssForwardF32Device(TSHipTensorView2D result, TSHipTensorView2D hidden, const int32_t* ids,
                                     const float* weights, int k, const void* gate_up_w, const float* gate_up_bias,
                                     const void* down_w, const float* down_bias, int ggml_type, int n_experts, int64_t H,
                                     int64_t F, float alpha, float limit)
{
    return guarded(0, "moe_experts_forward", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_desc(result, "result") || !validate_desc(hidden, "hidden")) return 0;
        if (!ids || !weights || !gate_up_w || !down_w || k < 1 || k > 16 || n_experts < 1 || H <= 0 || F <= 0) {
            set_last_error("Invalid arguments for moe_experts_forward.");
            return 0;
        }
        if (hidden.dim1 != H || result.dim1 != H || hidden.dim0 != result.dim0 || hidden.stride1 != 1 || !is_standard_view(result)) {
            set_last_error("Size mismatch: hidden / result must be [T x H] row-contiguous views in moe_experts_forward.");
            return 0;
        }
        const size_t rs_h = row_size(ggml_type, H), rs_f = row_size(ggml_type, F);
        if (!is_quant_type(ggml_type) || rs_h == 0 || rs_f == 0) {
            set_last_error("Unsupported quantized weight type or row length for moe_experts_forward.");
            return 0;
        }
        if (!check_device_operands(hidden, gate_up_w, ggml_type) || !check_device_operands(hidden, down_w, ggml_type)) return 0;
        const int T = hidden.dim0;
        const int64_t A64 = (int64_t)T * k;
        if (A64 > (1 << 24)) {
            set_last_error("moe_experts_forward: too many (token, expert) assignments for one call.");
            return 0;
        }
        const int A = (int)A64, E = n_experts;
        const int64_t gu_bytes = (int64_t)rs_h * 2 * F, dn_bytes = (int64_t)rs_f * H;   // per expert
        hipStream_t stream = t_stream;
        auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
        const bool small = A <= gemv_max_group() && H <= gemv_max_k(ggml_type) && F <= gemv_max_k(ggml_type);
        // rows per tile of the grouped GEMMs: up to about 160 tokens per expert the 32-row register-resident kernel
        // is fastest (measured at 32 experts of 2880 x 2880: T = 256 ... 1024), beyond that 128-row tiles
        const int per_expert = A / E;
        // MXFP4 experts run on the block-scaled matrix instruction (activations converted to MX fp6 pairs): with K <= 3072
        // on both matmuls in 48-row units of the register-resident kernel once an expert's tokens often pass 32 (nearly
        // every expert of a 256-token batch then streams its weights once; measured faster than the 128-row tiles up to
        // 2048 tokens per expert: 16384 tokens 4.17 vs 4.96 ms), else in its 32-row units up to 160 tokens per expert
        // MX fp6 pairs leave each activation with an error of up to 2^-10 of its BLOCK's largest magnitude (fp16: 2^-11 of
        // the value itself).  Against the norm of a result row that is a few 1e-5 for rows of thousands of outputs but
        // approaches 1e-3 for rows of 32: narrow stages stay on fp16 operands.
        const bool mx_type = ggml_type == kTypeMXFP4 && H <= 32768 && F <= 32768 && H >= 256 && F >= 128;
        const bool rows48 = mx_type && per_expert > 20 && H <= 3072 && F <= 3072;
        const bool mx = mx_type && (rows48 || per_expert <= 160);
        const int x_layout = mx ? 1 : 0;
        const int bm = rows48 ? 48 : per_expert > 160 ? 128 : 32;
        const int max_tiles = A / bm + E;
        // carve the workspace
        size_t off = 0;
        auto take = [&](size_t b) { const size_t o = off; off += al(b); return o; };
        const size_t o_offsets = take((size_t)(E + 1) * 4), o_token = take((size_t)A * 4), o_expert = take((size_t)A * 4);
        const size_t o_pos = take((size_t)A * 4), o_te = take((size_t)max_tiles * 4), o_tr0 = take((size_t)max_tiles * 4);
        const size_t o_trn = take((size_t)max_tiles * 4);
        const size_t o_ws1 = take(gemm_workspace_bytes(A, (int)H)), o_ws2 = take(gemm_workspace_bytes(A, (int)F));
        const size_t o_gu = take((size_t)A * 2 * F * 4), o_dn = take((size_t)A * H * 4);
        const GemmTiles plan_tiles{nullptr, nullptr, nullptr, max_tiles, bm, 0};
        const size_t chunk_bytes = small ? 0
                                         : std::max(gemm_chunk_ws_bytes(ggml_type, A, (int)(2 * F), (int)H, &plan_tiles, false, x_layout),
                                                    gemm_chunk_ws_bytes(ggml_type, A, (int)H, (int)F, &plan_tiles, false, x_layout));
        const size_t o_chunk = take(chunk_bytes);
        WsLease lease(stream, off);
        if (!lease.ok()) return 0;
        char* ws = lease.ptr();
        float* gu = reinterpret_cast<float*>(ws + o_gu);
        float* dn = reinterpret_cast<float*>(ws + o_dn);
        const float* hid = static_cast<const float*>(hidden.data);
        if (small) {
            // decode: one GEMV per (token, slot), expert chosen on the device through ids.  The gate_up launch computes
            // gate row j and up row j side by side and stores bias + SwiGLU-OAI of the pair: gu holds [A][F] activations.
            GemvArgs args[16];
            for (int a = 0; a < A; ++a) {
                args[a] = GemvArgs{gate_up_w, gu_bytes, hid + (int64_t)(a / k) * hidden.stride0, gu + (int64_t)a * F,
                                   (int)(2 * F), (int)H, ids + a, gu_bytes, E};
                args[a].pair_rows = (int)F;
                args[a].pair_kind = 1;
                args[a].norm_w = gate_up_bias;
                args[a].eps = alpha;
                args[a].limit = limit;
            }
            if (!launch_gemv_group(ggml_type, A, args, stream)) return 0;
            // The down projections and the weighted sum over a token's experts.  Where the format's row groups hold as
            // many rows as a token has experts (k = 4 for the 16-lane formats) one launch does both: a wavefront takes
            // row h of the token's k experts side by side and stores sum_s w_s (row . act_s + bias), in slot order: the
            // order of the reference's single-token path (GptOssModel.cs:718-735; a batch adds in expert order, :737-812).
            const bool routed = T == 1 && k == gemv_routed_slots(ggml_type) && (dn_bytes & 3) == 0 &&
                                (int64_t)E * dn_bytes < kMaxOperandBytes && (int64_t)k * F <= gemv_max_k(ggml_type);
            if (routed) {
                for (int t = 0; t < T; ++t) {
                    args[t] = GemvArgs{down_w, (int64_t)E * dn_bytes, gu + (int64_t)t * k * F,
                                       static_cast<float*>(result.data) + (int64_t)t * result.stride0, (int)H, (int)F};
                    args[t].expert_stride = dn_bytes;
                    args[t].n_experts = E;
                    args[t].slot_ids = ids + (int64_t)t * k;
                    args[t].slot_w = weights + (int64_t)t * k;
                    args[t].slot_bias = down_bias;
                }
                if (!launch_gemv_group(ggml_type, T, args, stream)) return 0;
            } else {
                for (int a = 0; a < A; ++a)
                    args[a] = GemvArgs{down_w, dn_bytes, gu + (int64_t)a * F, dn + (int64_t)a * H, (int)H, (int)F, ids + a, dn_bytes, E};
                if (!launch_gemv_group(ggml_type, A, args, stream)) return 0;
                if (!launch_moe_combine(dn, down_bias, ids, weights, nullptr, T, k, E, (int)H, T == 1, static_cast<float*>(result.data),
                                        result.stride0, stream))
                    return 0;
            }
        } else {
            MoeMaps maps{reinterpret_cast<int*>(ws + o_offsets), reinterpret_cast<int*>(ws + o_token),
                         reinterpret_cast<int*>(ws + o_expert), reinterpret_cast<int*>(ws + o_pos),
                         reinterpret_cast<int*>(ws + o_te),      reinterpret_cast<int*>(ws + o_tr0),
                         reinterpret_cast<int*>(ws + o_trn)};
            if (!launch_moe_group(ids, A, k, E, bm, max_tiles, maps, stream)) return 0;
            GemmTiles tiles{maps.tile_expert, maps.tile_row0, maps.tile_rows, max_tiles, bm, gu_bytes};
            if (!launch_convert_x(ggml_type, hid, hidden.stride0, maps.token_of, A, (int)H, ws + o_ws1, stream, nullptr, 0.f, x_layout))
                return 0;
            if (mx && bm <= 48 && gemm_swiglu_mx_fits((int)F, (int)H)) {
                // bias + SwiGLU-OAI and the conversion of the down projection's activations happen in the GEMM's epilogue
                if (!launch_gemm_swiglu_mx(gate_up_w, ws + o_ws1, ws + o_ws2, gu, gate_up_bias, alpha, limit, A, (int)F, (int)H, &tiles, stream))
                    return 0;
            } else {
                if (!launch_gemm(ggml_type, gate_up_w, gu_bytes, ws + o_ws1, gu, 2 * F, nullptr, A, (int)(2 * F), (int)H, &tiles, stream,
                                 false, ws + o_chunk, chunk_bytes, x_layout))
                    return 0;
                // bias + SwiGLU-OAI are formed while the down projection's activations are converted
                if (!launch_convert_x_swiglu(ggml_type, gu, gate_up_bias, maps.expert_of, alpha, limit, A, (int)F, ws + o_ws2, stream,
                                             x_layout))
                    return 0;
            }
            tiles.expert_stride = dn_bytes;
            if (!launch_gemm(ggml_type, down_w, dn_bytes, ws + o_ws2, dn, H, nullptr, A, (int)H, (int)F, &tiles, stream, false,
                             ws + o_chunk, chunk_bytes, x_layout))
                return 0;
            if (!launch_moe_combine(dn, down_bias, ids, weights, maps.pos_of, T, k, E, (int)H, false,
                                    static_cast<float*>(result.data), result.stride0, stream))
                return 0;
        }
        clear_last_error();
        return 1;
    });
}

int TSHip_AddmmQuantF32(TSHipTensorView2D result, TSHipTensorView2D m1, void* m2_data, int m2_ggml_type, int64_t m2_ne0,
                        int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "addmm_quant", [&]() -> int {
        return addmm_quant_host(result, m1, m2_data, m2_ggml_type, m2_ne0, m2_ne1, m2_raw_bytes);
    });
}

int TSHip_AddmmQuantBatchF32(TSHipTensorView2D result, TSHipTensorView2D m1, void* m2_data, int m2_ggml_type,
                             int64_t m2_ne0, int64_t m2_raw_bytes, int batch_count, int64_t* weight_offsets,
                             int64_t* weight_ne1_arr)
{
    return guarded(0, "addmm_quant_batch", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_desc(result, "result") || !validate_desc(m1, "m1")) return 0;
        if (m2_data == nullptr || batch_count <= 0 || weight_offsets == nullptr || weight_ne1_arr == nullptr) {
            set_last_error("Invalid arguments for addmm_quant_batch.");
            return 0;
        }
        const size_t rs = row_size(m2_ggml_type, m2_ne0);
        if (!is_matmul_type(m2_ggml_type) || rs == 0) {
            set_last_error("Unsupported quantized weight type or row length for addmm_quant_batch.");
            return 0;
        }
        if (batch_count > result.dim0 || batch_count > m1.dim0) {
            set_last_error("addmm_quant_batch: batch_count exceeds the number of rows.");
            return 0;
        }
        // row b of m1 times the sub-weight at weight_offsets[b] -> row b of result (ggml_ops_matmul.cpp:672-729)
        for (int b = 0; b < batch_count; ++b) {
            const int64_t ne1 = weight_ne1_arr[b], off = weight_offsets[b];
            if (off < 0 || ne1 <= 0 || (size_t)off + (size_t)ne1 * rs > (size_t)m2_raw_bytes) {
                set_last_error("addmm_quant_batch: sub-weight lies outside the weight bytes.");
                return 0;
            }
            if (ne1 > result.dim1) {
                set_last_error("addmm_quant_batch: a sub-weight has more rows than the result has columns.");
                return 0;
            }
            TSHipTensorView2D r = result;
            r.dim0 = 1;
            r.dim1 = (int)ne1;        // a sub-weight with fewer rows than result.dim1 fills the first ne1 columns of its row
            r.data = static_cast<char*>(result.data) + (size_t)b * result.stride0 * sizeof(float);
            r.raw_bytes = (int64_t)r.dim1 * (int64_t)sizeof(float);
            TSHipTensorView2D x = m1;
            x.dim0 = 1;
            x.data = static_cast<char*>(m1.data) + (size_t)b * m1.stride0 * sizeof(float);
            x.raw_bytes = (int64_t)required_raw_bytes(x);
            void* sub = static_cast<char*>(m2_data) + off;
            std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
            const void* sub_dev = resolve_weight_range(m2_data, (size_t)off, (size_t)ne1 * rs);
            if (!sub_dev) return 0;
            if (!addmm_quant_host(r, x, sub, m2_ggml_type, m2_ne0, ne1, (int64_t)((size_t)ne1 * rs), sub_dev)) return 0;
        }
        clear_last_error();
        return 1;
    });
}

int TSHip_PreloadQuantizedWeight(void* cache_key, void* host_data, int ggml_type, int64_t ne0, int64_t ne1,
                                 int64_t raw_bytes)
{
    return guarded(0, "preload", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (cache_key == nullptr || host_data == nullptr || ne0 <= 0 || ne1 <= 0 || raw_bytes <= 0) {
            set_last_error("Invalid arguments for quantized weight preload.");
            return 0;
        }
        const size_t rs = row_size(ggml_type, ne0);
        if (!is_matmul_type(ggml_type) || rs == 0 || (size_t)raw_bytes < rs * (size_t)ne1) {
            set_last_error("Unsupported type or inconsistent size for quantized weight preload.");
            return 0;
        }
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        auto it = g_weight_cache.find(cache_key);
        if (it != g_weight_cache.end()) {
            if (it->second.preloaded && it->second.bytes == (size_t)raw_bytes) {
                clear_last_error();
                return 1;  // idempotent
            }
            (void)hipFree(it->second.dev);
            g_weight_cache.erase(it);
        }
        CachedWeight cw;
        if (!hip_ok(hipMalloc(&cw.dev, (size_t)raw_bytes + 16), "hipMalloc(preload)")) return 0;
        if (!hip_ok(hipMemcpy(cw.dev, host_data, (size_t)raw_bytes, hipMemcpyHostToDevice), "hipMemcpy(preload)")) {
            (void)hipFree(cw.dev);
            return 0;
        }
        cw.bytes = (size_t)raw_bytes;
        cw.preloaded = true;
        g_weight_cache[cache_key] = cw;
        clear_last_error();
        return 1;
    });
}

void TSHip_InvalidateHostBuffer(void* ptr)
{
    std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_weight_cache.find(ptr);
    if (it == g_weight_cache.end()) return;
    (void)hipFree(it->second.dev);
    g_weight_cache.erase(it);
}

void TSHip_ClearHostBufferCache(void)
{
    std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (auto& kv : g_weight_cache) (void)hipFree(kv.second.dev);
    g_weight_cache.clear();
}

// ggml_ops_core.cpp:664-684: nothing to do (success) for a null pointer, a zero size, a pointer that is not cached or
// an entry that is not a device copy of caller memory (here: a preloaded key); an error only when more bytes are
// asked for than the copy holds, or when the copy fails.
int TSHip_SyncHostBuffer(void* ptr, size_t size)
{
    return guarded(0, "sync_host_buffer", [&]() -> int {
        clear_last_error();
        if (ptr == nullptr || size == 0) return 1;
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        auto it = g_weight_cache.find(ptr);
        if (it == g_weight_cache.end() || it->second.preloaded) return 1;
        if (size > it->second.bytes) {
            set_last_error("Failed to synchronize cached HIP device buffer back to host memory.");
            return 0;
        }
        if (!hip_ok(hipMemcpy(ptr, it->second.dev, size, hipMemcpyDeviceToHost), "hipMemcpy(sync)")) return 0;
        return 1;
    });
}

/* ---- embedding gather ----------------------------------------------------------------- */

int TSHip_GetRowsQuantF32Device(TSHipTensorView2D result, const void* src_data, int src_ggml_type, int64_t src_ne0,
                                int64_t src_ne1, int64_t src_raw_bytes, const int32_t* indices, int64_t num_indices)
{
    return guarded(0, "get_rows_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_desc(result, "result")) return 0;
        if (src_data == nullptr || src_ne0 <= 0 || src_ne1 <= 0 || src_raw_bytes <= 0) {
            set_last_error("Invalid quantized weight descriptor for get_rows_quant.");
            return 0;
        }
        if (indices == nullptr || num_indices <= 0) {
            set_last_error("Invalid element count passed for indices.");
            return 0;
        }
        if (result.dim0 != num_indices || result.dim1 != src_ne0) {
            set_last_error("Shape mismatch in get_rows_quant: result must be [num_indices, ne0].");
            return 0;
        }
        const size_t rs = row_size(src_ggml_type, src_ne0);
        if ((src_ggml_type != kTypeF32 && !is_dequant_type(src_ggml_type)) || rs == 0 || src_ne0 % 4 != 0) {
            set_last_error("Unsupported source type or row length for get_rows_quant.");
            return 0;
        }
        if ((size_t)src_raw_bytes < rs * (size_t)src_ne1) {
            set_last_error("Quantized weight bytes are smaller than ne0 x ne1 for get_rows_quant.");
            return 0;
        }
        if (result.stride1 != 1) {
            set_last_error("result must be a standard (stride1 == 1) view in get_rows_quant.");
            return 0;
        }
        // one launch serves at most 65535 indices (grid dimension): more are served in slices, like the host form
        for (int64_t i0 = 0; i0 < num_indices; i0 += 65535) {
            const int64_t cnt = std::min<int64_t>(65535, num_indices - i0);
            if (!launch_get_rows(src_ggml_type, src_data, (int64_t)rs, src_ne1, indices + i0, cnt, src_ne0,
                                 static_cast<float*>(result.data) + i0 * result.stride0, result.stride0, t_stream))
                return 0;
        }
        clear_last_error();
        return 1;
    });
}

int TSHip_GetRowsQuantF32(TSHipTensorView2D result, void* src_data, int src_ggml_type, int64_t src_ne0, int64_t src_ne1,
                          int64_t src_raw_bytes, TSHipContiguousTensor indices)
{
    return guarded(0, "get_rows_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_desc(result, "result")) return 0;
        if (indices.data == nullptr) {
            set_last_error("Null pointer passed for indices.");
            return 0;
        }
        if (indices.element_count <= 0) {
            set_last_error("Invalid element count passed for indices.");
            return 0;
        }
        if (indices.element_type != 0 && indices.element_type != 3) {
            set_last_error("Unsupported contiguous tensor element type passed for indices.");
            return 0;
        }
        if (src_data == nullptr || src_ne0 <= 0 || src_ne1 <= 0 || src_raw_bytes <= 0) {
            set_last_error("Invalid quantized weight descriptor for get_rows_quant.");
            return 0;
        }
        const int64_t n = indices.element_count;
        if (result.dim0 != n || result.dim1 != src_ne0) {
            set_last_error("Shape mismatch in get_rows_quant: result must be [num_indices, ne0].");
            return 0;
        }
        const size_t rs = row_size(src_ggml_type, src_ne0);
        if ((src_ggml_type != kTypeF32 && !is_dequant_type(src_ggml_type)) || rs == 0 || src_ne0 % 4 != 0) {
            set_last_error("Unsupported source type or row length for get_rows_quant.");
            return 0;
        }
        if ((size_t)src_raw_bytes < rs * (size_t)src_ne1) {
            set_last_error("Quantized weight bytes are smaller than ne0 x ne1 for get_rows_quant.");
            return 0;
        }
        if (!is_standard_view(result)) {
            set_last_error("result must be a standard (stride1 == 1, non-overlapping) view in get_rows_quant.");
            return 0;
        }
        // indices as int32 (F32 indices are truncated like the bridge's read_i32_values, ggml_ops_core.cpp:419-437)
        std::vector<int32_t> ids((size_t)n);
        if (indices.element_type == 3) {
            std::memcpy(ids.data(), indices.data, (size_t)n * sizeof(int32_t));
        } else {
            const float* f = static_cast<const float*>(indices.data);
            for (int64_t i = 0; i < n; ++i) ids[(size_t)i] = (int32_t)f[i];
        }
        for (int64_t i = 0; i < n; ++i)
            if (ids[(size_t)i] < 0 || ids[(size_t)i] >= src_ne1) {
                set_last_error("Index out of range in get_rows_quant.");
                return 0;
            }
        std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
        const void* w_dev = resolve_weight(src_data, rs * (size_t)src_ne1);
        if (!w_dev) return 0;

        const size_t K = (size_t)src_ne0;
        const size_t y_bytes = (size_t)n * K * sizeof(float);
        const size_t id_bytes = ((size_t)n * sizeof(int32_t) + 255) & ~(size_t)255;
        if (!ws_reserve(id_bytes + y_bytes, std::max(id_bytes, y_bytes))) return 0;
        int32_t* ids_dev = static_cast<int32_t*>(g_ws.dev);
        float* y_dev = reinterpret_cast<float*>(static_cast<char*>(g_ws.dev) + id_bytes);
        hipStream_t stream = nullptr;
        std::memcpy(g_ws.pinned, ids.data(), (size_t)n * sizeof(int32_t));
        if (!hip_ok(hipMemcpyAsync(ids_dev, g_ws.pinned, (size_t)n * sizeof(int32_t), hipMemcpyHostToDevice, stream), "hipMemcpy(indices)")) return 0;
        if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;       // the pinned block is reused below
        for (int64_t i0 = 0; i0 < n; i0 += 65535) {
            const int64_t cnt = std::min<int64_t>(65535, n - i0);
            if (!launch_get_rows(src_ggml_type, w_dev, (int64_t)rs, src_ne1, ids_dev + i0, cnt, src_ne0, y_dev + (size_t)i0 * K, (int64_t)K, stream))
                return 0;
        }
        if (!hip_ok(hipMemcpyAsync(g_ws.pinned, y_dev, y_bytes, hipMemcpyDeviceToHost, stream), "hipMemcpy(result)")) return 0;
        if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
        float* dst = static_cast<float*>(result.data);
        const float* stage = static_cast<const float*>(g_ws.pinned);
        for (int64_t i = 0; i < n; ++i) std::memcpy(dst + (size_t)i * result.stride0, stage + (size_t)i * K, K * sizeof(float));
        clear_last_error();
        return 1;
    });
}

/* ---- fused wrappers (ggml_ops_fused.cpp) ---------------------------------------------------- */

int TSHip_FusedRmsNormMatMulQuantF32Device(TSHipTensorView2D result, TSHipTensorView2D input, const float* norm_weight,
                                           int norm_weight_count, float eps, const void* m2_data, int m2_ggml_type,
                                           int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "fused_rms_norm_matmul_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_fused_matmul(result, input, norm_weight, norm_weight_count, true, m2_data, m2_ggml_type, m2_ne0, m2_ne1,
                                   m2_raw_bytes, "fused rms_norm_matmul", "result"))
            return 0;
        if (!check_device_views(result, input)) return 0;
        const size_t need = matmul_ws_bytes(m2_ggml_type, input.dim0, m2_ne0, m2_ne1, true, false);
        WsLease ws(t_stream, need);
        if (!ws.ok()) return 0;
        if (!run_matmul_device_ws(result, input, m2_data, m2_ggml_type, m2_ne0, m2_ne1, t_stream, ws.ptr(), need, norm_weight, eps, false))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_FusedMatMulQuantAddF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, const void* m2_data,
                                       int m2_ggml_type, int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "fused_matmul_quant_add", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_fused_matmul(residual, input, nullptr, 0, false, m2_data, m2_ggml_type, m2_ne0, m2_ne1, m2_raw_bytes,
                                   "fused matmul_add", "residual"))
            return 0;
        if (!check_device_views(residual, input)) return 0;
        const size_t need = matmul_ws_bytes(m2_ggml_type, input.dim0, m2_ne0, m2_ne1, false, true);
        WsLease ws(t_stream, need);
        if (!ws.ok()) return 0;
        if (!run_matmul_device_ws(residual, input, m2_data, m2_ggml_type, m2_ne0, m2_ne1, t_stream, ws.ptr(), need, nullptr, 0.f, true))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_FusedFFNSwiGLUQuantF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, const float* norm_weight,
                                       int norm_weight_count, float eps, const void* gate_up_data, int gate_up_ggml_type,
                                       int64_t gate_up_ne0, int64_t gate_up_ne1, int64_t gate_up_raw_bytes,
                                       const void* down_data, int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                       int64_t down_raw_bytes, int half_dim)
{
    return guarded(0, "fused_ffn_swiglu_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_ffn(residual, input, norm_weight, norm_weight_count, gate_up_data, gate_up_ggml_type, gate_up_ne0,
                          gate_up_ne1, gate_up_raw_bytes, down_data, down_ggml_type, down_ne0, down_ne1, down_raw_bytes, half_dim))
            return 0;
        if (!check_device_views(residual, input)) return 0;
        WsLease ws(t_stream, ffn_ws_bytes(input.dim0, gate_up_ggml_type, down_ggml_type, input.dim1, half_dim));
        if (!ws.ok()) return 0;
        if (!run_ffn_swiglu_device(residual, input, norm_weight, eps, gate_up_data, gate_up_ggml_type, down_data, down_ggml_type,
                                   input.dim1, half_dim, t_stream, ws.ptr()))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_FusedRmsNormMatMulQuantF32(TSHipTensorView2D result, TSHipTensorView2D input, void* norm_weight_data,
                                     int norm_weight_count, float eps, void* m2_data, int m2_ggml_type, int64_t m2_ne0,
                                     int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "fused_rms_norm_matmul_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_fused_matmul(result, input, norm_weight_data, norm_weight_count, true, m2_data, m2_ggml_type, m2_ne0,
                                   m2_ne1, m2_raw_bytes, "fused rms_norm_matmul", "result"))
            return 0;
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        const void* w = resolve_weight(m2_data, row_size(m2_ggml_type, m2_ne0) * (size_t)m2_ne1);
        if (!w) return 0;
        return with_host_tensors(result, false, input, norm_weight_data, norm_weight_count,
                                 [&](const TSHipTensorView2D& x, const TSHipTensorView2D& y, const float* nw, hipStream_t st) {
                                     const size_t need = matmul_ws_bytes(m2_ggml_type, x.dim0, m2_ne0, m2_ne1, true, false);
                                     WsLease ws(st, need);
                                     return ws.ok() && run_matmul_device_ws(y, x, w, m2_ggml_type, m2_ne0, m2_ne1, st, ws.ptr(), need, nw, eps, false);
                                 });
    });
}

int TSHip_FusedMatMulQuantAddF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* m2_data, int m2_ggml_type,
                                 int64_t m2_ne0, int64_t m2_ne1, int64_t m2_raw_bytes)
{
    return guarded(0, "fused_matmul_quant_add", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_fused_matmul(residual, input, nullptr, 0, false, m2_data, m2_ggml_type, m2_ne0, m2_ne1, m2_raw_bytes,
                                   "fused matmul_add", "residual"))
            return 0;
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        const void* w = resolve_weight(m2_data, row_size(m2_ggml_type, m2_ne0) * (size_t)m2_ne1);
        if (!w) return 0;
        return with_host_tensors(residual, true, input, nullptr, 0,
                                 [&](const TSHipTensorView2D& x, const TSHipTensorView2D& y, const float*, hipStream_t st) {
                                     const size_t need = matmul_ws_bytes(m2_ggml_type, x.dim0, m2_ne0, m2_ne1, false, true);
                                     WsLease ws(st, need);
                                     return ws.ok() && run_matmul_device_ws(y, x, w, m2_ggml_type, m2_ne0, m2_ne1, st, ws.ptr(), need, nullptr, 0.f, true);
                                 });
    });
}

int TSHip_FusedFFNSwiGLUQuantF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* norm_weight_data,
                                 int norm_weight_count, float eps, void* gate_up_data, int gate_up_ggml_type,
                                 int64_t gate_up_ne0, int64_t gate_up_ne1, int64_t gate_up_raw_bytes, void* down_data,
                                 int down_ggml_type, int64_t down_ne0, int64_t down_ne1, int64_t down_raw_bytes, int half_dim)
{
    return guarded(0, "fused_ffn_swiglu_quant", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_ffn(residual, input, norm_weight_data, norm_weight_count, gate_up_data, gate_up_ggml_type, gate_up_ne0,
                          gate_up_ne1, gate_up_raw_bytes, down_data, down_ggml_type, down_ne0, down_ne1, down_raw_bytes, half_dim))
            return 0;
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        const void* gu = resolve_weight(gate_up_data, row_size(gate_up_ggml_type, gate_up_ne0) * (size_t)gate_up_ne1);
        if (!gu) return 0;
        const void* dn = resolve_weight(down_data, row_size(down_ggml_type, down_ne0) * (size_t)down_ne1);
        if (!dn) return 0;
        return with_host_tensors(residual, true, input, norm_weight_data, norm_weight_count,
                                 [&](const TSHipTensorView2D& x, const TSHipTensorView2D& y, const float* nw, hipStream_t st) {
                                     WsLease ws(st, ffn_ws_bytes(x.dim0, gate_up_ggml_type, down_ggml_type, x.dim1, half_dim));
                                     return ws.ok() && run_ffn_swiglu_device(y, x, nw, eps, gu, gate_up_ggml_type, dn, down_ggml_type, x.dim1,
                                                                             half_dim, st, ws.ptr());
                                 });
    });
}

int TSHip_FusedOutProjFFNQuantF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, const void* out_proj_data,
                                        int out_proj_type, int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes,
                                        const float* ffn_norm_weight, int ffn_norm_count, float eps, const void* gu_data, int gu_type,
                                        int64_t gu_ne0, int64_t gu_ne1, int64_t gu_raw_bytes, const void* dn_data, int dn_type,
                                        int64_t dn_ne0, int64_t dn_ne1, int64_t dn_raw_bytes, int half_dim)
{
    return guarded(0, "fused_outproj_ffn", [&]() -> int {
        if (!ensure_backend()) return 0;
        const WeightDesc od{out_proj_data, out_proj_type, out_ne0, out_ne1, out_raw_bytes};
        const WeightDesc gd{gu_data, gu_type, gu_ne0, gu_ne1, gu_raw_bytes}, dd{dn_data, dn_type, dn_ne0, dn_ne1, dn_raw_bytes};
        if (!validate_outproj_ffn(residual, input, od, ffn_norm_weight, ffn_norm_count, gd, dd, half_dim)) return 0;
        if (!check_device_views(residual, input)) return 0;
        const size_t need = outproj_ffn_ws_bytes(input.dim0, od, gd, dd, residual.dim1, half_dim);
        WsLease ws(t_stream, need);
        if (!ws.ok()) return 0;
        if (!run_outproj_ffn_device(residual, input, out_proj_data, od, ffn_norm_weight, eps, gu_data, gu_type, dn_data, dn_type, half_dim,
                                    t_stream, ws.ptr(), need))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_FusedOutProjFFNQuantF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* out_proj_data, int out_proj_type,
                                  int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes, void* ffn_norm_data, int ffn_norm_count,
                                  float eps, void* gu_data, int gu_type, int64_t gu_ne0, int64_t gu_ne1, int64_t gu_raw_bytes,
                                  void* dn_data, int dn_type, int64_t dn_ne0, int64_t dn_ne1, int64_t dn_raw_bytes, int half_dim)
{
    return guarded(0, "fused_outproj_ffn", [&]() -> int {
        if (!ensure_backend()) return 0;
        const WeightDesc od{out_proj_data, out_proj_type, out_ne0, out_ne1, out_raw_bytes};
        const WeightDesc gd{gu_data, gu_type, gu_ne0, gu_ne1, gu_raw_bytes}, dd{dn_data, dn_type, dn_ne0, dn_ne1, dn_raw_bytes};
        if (!validate_outproj_ffn(residual, input, od, ffn_norm_data, ffn_norm_count, gd, dd, half_dim)) return 0;
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        const void* ow = resolve_weight(out_proj_data, od.bytes());
        const void* gu = ow ? resolve_weight(gu_data, gd.bytes()) : nullptr;
        const void* dn = gu ? resolve_weight(dn_data, dd.bytes()) : nullptr;
        if (!dn) return 0;
        const HostTensor io[2] = {{&residual, true, true}, {&input, true, false}};
        return with_host_io(io, 2, ffn_norm_data, ffn_norm_count, [&](const TSHipTensorView2D* dv, const float* nw, hipStream_t st) {
            const size_t need = outproj_ffn_ws_bytes(dv[1].dim0, od, gd, dd, dv[0].dim1, half_dim);
            WsLease ws(st, need);
            return ws.ok() && run_outproj_ffn_device(dv[0], dv[1], ow, od, nw, eps, gu, gu_type, dn, dn_type, half_dim, st, ws.ptr(), need);
        });
    });
}

int TSHip_FusedOutProjNormRouterQuantF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, const void* out_proj_data,
                                               int out_proj_type, int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes,
                                               const float* norm_weight, int norm_count, float eps, TSHipTensorView2D normed_out,
                                               const void* router_data, int router_type, int64_t router_ne0, int64_t router_ne1,
                                               int64_t router_raw_bytes, TSHipTensorView2D router_out)
{
    return guarded(0, "fused_outproj_norm_router", [&]() -> int {
        if (!ensure_backend()) return 0;
        const WeightDesc od{out_proj_data, out_proj_type, out_ne0, out_ne1, out_raw_bytes};
        const WeightDesc rd{router_data, router_type, router_ne0, router_ne1, router_raw_bytes};
        if (!validate_outproj_router(residual, input, od, norm_weight, norm_count, normed_out, rd, router_out)) return 0;
        if (!check_device_views(residual, input) || !is_standard_view(router_out)) {
            set_last_error("Device addmm_quant needs stride1 == 1 views.");
            return 0;
        }
        const size_t need = outproj_router_ws_bytes(input.dim0, od, rd);
        WsLease ws(t_stream, need);
        if (!ws.ok()) return 0;
        if (!run_outproj_router_device(residual, input, out_proj_data, od, norm_weight, eps, normed_out, router_data, rd, router_out,
                                       t_stream, ws.ptr(), need))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_FusedOutProjNormRouterQuantF32(TSHipTensorView2D residual, TSHipTensorView2D input, void* out_proj_data, int out_proj_type,
                                         int64_t out_ne0, int64_t out_ne1, int64_t out_raw_bytes, void* norm_data, int norm_count,
                                         float eps, TSHipTensorView2D normed_out, void* router_data, int router_type,
                                         int64_t router_ne0, int64_t router_ne1, int64_t router_raw_bytes, TSHipTensorView2D router_out)
{
    return guarded(0, "fused_outproj_norm_router", [&]() -> int {
        if (!ensure_backend()) return 0;
        const WeightDesc od{out_proj_data, out_proj_type, out_ne0, out_ne1, out_raw_bytes};
        const WeightDesc rd{router_data, router_type, router_ne0, router_ne1, router_raw_bytes};
        if (!validate_outproj_router(residual, input, od, norm_data, norm_count, normed_out, rd, router_out)) return 0;
        std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
        const void* ow = resolve_weight(out_proj_data, od.bytes());
        const void* rw = ow ? resolve_weight(router_data, rd.bytes()) : nullptr;
        if (!rw) return 0;
        const HostTensor io[4] = {{&residual, true, true}, {&input, true, false}, {&normed_out, false, true}, {&router_out, false, true}};
        return with_host_io(io, 4, norm_data, norm_count, [&](const TSHipTensorView2D* dv, const float* nw, hipStream_t st) {
            const size_t need = outproj_router_ws_bytes(dv[1].dim0, od, rd);
            WsLease ws(st, need);
            return ws.ok() && run_outproj_router_device(dv[0], dv[1], ow, od, nw, eps, dv[2], rw, rd, dv[3], st, ws.ptr(), need);
        });
    });
}

/* ---- weighted expert sets (ggml_ops_fused.cpp:1576-2160) -------------------------------------- */
namespace {

// the caller's arrays hold device pointers
int expert_set_device(TSHipTensorView2D out, bool add_to_out, TSHipTensorView2D input, const ExpertSetArgs& a, const char* out_name)
{
    if (!ensure_backend()) return 0;
    if (!validate_expert_set(out, input, a, out_name)) return 0;
    if (!check_device_views(out, input)) return 0;
    if (!run_expert_set(out, add_to_out, input, a, t_stream, [](void* p, size_t) -> const void* { return p; })) return 0;
    clear_last_error();
    return 1;
}

// the caller's arrays hold host pointers: each expert's blocks are cached on the device under its host address
int expert_set_host(TSHipTensorView2D out, bool add_to_out, TSHipTensorView2D input, const ExpertSetArgs& a, const char* out_name)
{
    if (!ensure_backend()) return 0;
    if (!validate_expert_set(out, input, a, out_name)) return 0;
    std::lock_guard<std::recursive_mutex> call_lock(g_host_call_mutex);
    const HostTensor io[2] = {{&out, add_to_out, true}, {&input, true, false}};
    return with_host_io(io, 2, nullptr, 0, [&](const TSHipTensorView2D* dv, const float*, hipStream_t st) {
        return run_expert_set(dv[0], add_to_out, dv[1], a, st, [](void* p, size_t bytes) { return resolve_weight(p, bytes); });
    });
}

ExpertSetArgs relu2_args(int num_experts, void* const* up, void* const* down, int up_type, int64_t up_ne0, int64_t up_ne1,
                         int64_t up_bytes, int down_type, int64_t down_ne0, int64_t down_ne1, int64_t down_bytes, const float* route_weights)
{
    ExpertSetArgs a{};
    a.what = "MoE", a.max_experts = 16, a.num_experts = num_experts, a.gated = false, a.gate = nullptr, a.up = up, a.down = down;
    a.up_d = WeightDesc{nullptr, up_type, up_ne0, up_ne1, up_bytes};
    a.down_d = WeightDesc{nullptr, down_type, down_ne0, down_ne1, down_bytes};
    a.route_weights = route_weights;
    return a;
}

ExpertSetArgs swiglu_args(const char* what, int max_experts, int num_experts, void* const* gate, void* const* up, void* const* down,
                          int gate_type, int64_t gate_ne0, int64_t gate_ne1, int64_t gate_bytes, int up_type, int64_t up_ne0,
                          int64_t up_ne1, int64_t up_bytes, int down_type, int64_t down_ne0, int64_t down_ne1, int64_t down_bytes,
                          const float* route_weights)
{
    ExpertSetArgs a{};
    a.what = what, a.max_experts = max_experts, a.num_experts = num_experts, a.gated = true, a.gate = gate, a.up = up, a.down = down;
    a.gate_d = WeightDesc{nullptr, gate_type, gate_ne0, gate_ne1, gate_bytes};
    a.up_d = WeightDesc{nullptr, up_type, up_ne0, up_ne1, up_bytes};
    a.down_d = WeightDesc{nullptr, down_type, down_ne0, down_ne1, down_bytes};
    a.route_weights = route_weights;
    return a;
}

void set_shared(ExpertSetArgs& a, int use_shared, void* gate, void* up, void* down, int gate_type, int64_t gate_ne0, int64_t gate_ne1,
                int64_t gate_bytes, int up_type, int64_t up_ne0, int64_t up_ne1, int64_t up_bytes, int down_type, int64_t down_ne0,
                int64_t down_ne1, int64_t down_bytes, float scalar)
{
    // as the bridge: the shared expert takes part only when the flag is set and all three weights are given
    a.has_shared = use_shared != 0 && gate != nullptr && up != nullptr && down != nullptr;
    a.sh_gate = WeightDesc{gate, gate_type, gate_ne0, gate_ne1, gate_bytes};
    a.sh_up = WeightDesc{up, up_type, up_ne0, up_ne1, up_bytes};
    a.sh_down = WeightDesc{down, down_type, down_ne0, down_ne1, down_bytes};
    a.shared_scalar = scalar;
}

}  // namespace

int TSHip_MoEExpertsForwardF32(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts, void** up_data_ptrs,
                               void** down_data_ptrs, int up_ggml_type, int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each,
                               int down_ggml_type, int64_t down_ne0, int64_t down_ne1, int64_t down_raw_bytes_each,
                               float* route_weights)
{
    return guarded(0, "MoE experts", [&]() -> int {
        return expert_set_host(result, false, input,
                               relu2_args(num_experts, up_data_ptrs, down_data_ptrs, up_ggml_type, up_ne0, up_ne1, up_raw_bytes_each,
                                          down_ggml_type, down_ne0, down_ne1, down_raw_bytes_each, route_weights),
                               "result");
    });
}

int TSHip_MoEExpertsForwardF32Device(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts, void* const* up_data_ptrs,
                                     void* const* down_data_ptrs, int up_ggml_type, int64_t up_ne0, int64_t up_ne1,
                                     int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                     int64_t down_raw_bytes_each, const float* route_weights)
{
    return guarded(0, "MoE experts", [&]() -> int {
        return expert_set_device(result, false, input,
                                 relu2_args(num_experts, up_data_ptrs, down_data_ptrs, up_ggml_type, up_ne0, up_ne1, up_raw_bytes_each,
                                            down_ggml_type, down_ne0, down_ne1, down_raw_bytes_each, route_weights),
                                 "result");
    });
}

int TSHip_MoEExpertsSwiGLUForwardF32(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts, void** gate_data_ptrs,
                                     void** up_data_ptrs, void** down_data_ptrs, int gate_ggml_type, int64_t gate_ne0, int64_t gate_ne1,
                                     int64_t gate_raw_bytes_each, int up_ggml_type, int64_t up_ne0, int64_t up_ne1,
                                     int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                     int64_t down_raw_bytes_each, float* route_weights)
{
    return guarded(0, "MoE SwiGLU experts", [&]() -> int {
        return expert_set_host(result, false, input,
                               swiglu_args("MoE SwiGLU", 32, num_experts, gate_data_ptrs, up_data_ptrs, down_data_ptrs, gate_ggml_type,
                                           gate_ne0, gate_ne1, gate_raw_bytes_each, up_ggml_type, up_ne0, up_ne1, up_raw_bytes_each,
                                           down_ggml_type, down_ne0, down_ne1, down_raw_bytes_each, route_weights),
                               "result");
    });
}

int TSHip_MoEExpertsSwiGLUForwardF32Device(TSHipTensorView2D result, TSHipTensorView2D input, int num_experts,
                                           void* const* gate_data_ptrs, void* const* up_data_ptrs, void* const* down_data_ptrs,
                                           int gate_ggml_type, int64_t gate_ne0, int64_t gate_ne1, int64_t gate_raw_bytes_each,
                                           int up_ggml_type, int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each,
                                           int down_ggml_type, int64_t down_ne0, int64_t down_ne1, int64_t down_raw_bytes_each,
                                           const float* route_weights)
{
    return guarded(0, "MoE SwiGLU experts", [&]() -> int {
        return expert_set_device(result, false, input,
                                 swiglu_args("MoE SwiGLU", 32, num_experts, gate_data_ptrs, up_data_ptrs, down_data_ptrs, gate_ggml_type,
                                             gate_ne0, gate_ne1, gate_raw_bytes_each, up_ggml_type, up_ne0, up_ne1, up_raw_bytes_each,
                                             down_ggml_type, down_ne0, down_ne1, down_raw_bytes_each, route_weights),
                                 "result");
    });
}

int TSHip_MoEExpertsSwiGLUResidualF32(TSHipTensorView2D residual, TSHipTensorView2D input, int num_experts, void** gate_data_ptrs,
                                      void** up_data_ptrs, void** down_data_ptrs, int gate_ggml_type, int64_t gate_ne0,
                                      int64_t gate_ne1, int64_t gate_raw_bytes_each, int up_ggml_type, int64_t up_ne0, int64_t up_ne1,
                                      int64_t up_raw_bytes_each, int down_ggml_type, int64_t down_ne0, int64_t down_ne1,
                                      int64_t down_raw_bytes_each, float* route_weights, int use_shared, void* shared_gate_data,
                                      void* shared_up_data, void* shared_down_data, int shared_gate_ggml_type, int64_t shared_gate_ne0,
                                      int64_t shared_gate_ne1, int64_t shared_gate_raw_bytes, int shared_up_ggml_type,
                                      int64_t shared_up_ne0, int64_t shared_up_ne1, int64_t shared_up_raw_bytes,
                                      int shared_down_ggml_type, int64_t shared_down_ne0, int64_t shared_down_ne1,
                                      int64_t shared_down_raw_bytes, float shared_scalar)
{
    return guarded(0, "MoE SwiGLU residual", [&]() -> int {
        ExpertSetArgs a = swiglu_args("MoE SwiGLU residual", 32, num_experts, gate_data_ptrs, up_data_ptrs, down_data_ptrs, gate_ggml_type,
                                      gate_ne0, gate_ne1, gate_raw_bytes_each, up_ggml_type, up_ne0, up_ne1, up_raw_bytes_each,
                                      down_ggml_type, down_ne0, down_ne1, down_raw_bytes_each, route_weights);
        set_shared(a, use_shared, shared_gate_data, shared_up_data, shared_down_data, shared_gate_ggml_type, shared_gate_ne0, shared_gate_ne1,
                   shared_gate_raw_bytes, shared_up_ggml_type, shared_up_ne0, shared_up_ne1, shared_up_raw_bytes, shared_down_ggml_type,
                   shared_down_ne0, shared_down_ne1, shared_down_raw_bytes, shared_scalar);
        return expert_set_host(residual, true, input, a, "residual");
    });
}

int TSHip_MoEExpertsSwiGLUResidualF32Device(TSHipTensorView2D residual, TSHipTensorView2D input, int num_experts,
                                            void* const* gate_data_ptrs, void* const* up_data_ptrs, void* const* down_data_ptrs,
                                            int gate_ggml_type, int64_t gate_ne0, int64_t gate_ne1, int64_t gate_raw_bytes_each,
                                            int up_ggml_type, int64_t up_ne0, int64_t up_ne1, int64_t up_raw_bytes_each,
                                            int down_ggml_type, int64_t down_ne0, int64_t down_ne1, int64_t down_raw_bytes_each,
                                            const float* route_weights, int use_shared, void* shared_gate_data, void* shared_up_data,
                                            void* shared_down_data, int shared_gate_ggml_type, int64_t shared_gate_ne0,
                                            int64_t shared_gate_ne1, int64_t shared_gate_raw_bytes, int shared_up_ggml_type,
                                            int64_t shared_up_ne0, int64_t shared_up_ne1, int64_t shared_up_raw_bytes,
                                            int shared_down_ggml_type, int64_t shared_down_ne0, int64_t shared_down_ne1,
                                            int64_t shared_down_raw_bytes, float shared_scalar)
{
    return guarded(0, "MoE SwiGLU residual", [&]() -> int {
        ExpertSetArgs a = swiglu_args("MoE SwiGLU residual", 32, num_experts, gate_data_ptrs, up_data_ptrs, down_data_ptrs, gate_ggml_type,
                                      gate_ne0, gate_ne1, gate_raw_bytes_each, up_ggml_type, up_ne0, up_ne1, up_raw_bytes_each,
                                      down_ggml_type, down_ne0, down_ne1, down_raw_bytes_each, route_weights);
        set_shared(a, use_shared, shared_gate_data, shared_up_data, shared_down_data, shared_gate_ggml_type, shared_gate_ne0, shared_gate_ne1,
                   shared_gate_raw_bytes, shared_up_ggml_type, shared_up_ne0, shared_up_ne1, shared_up_raw_bytes, shared_down_ggml_type,
                   shared_down_ne0, shared_down_ne1, shared_down_raw_bytes, shared_scalar);
        return expert_set_device(residual, true, input, a, "residual");
    });
}

/* ---- ggml_mul_mat_id with F32 experts (ggml_ops_matmul.cpp:958-1121) --------------------------- */
namespace {

bool validate_desc3(const TSHipTensorView3D& d, const char* name)
{
    if (d.data == nullptr) {
        set_last_error(std::string("Null pointer passed for ") + name + '.');
        return false;
    }
    if (d.dim0 <= 0 || d.dim1 <= 0 || d.dim2 <= 0) {
        set_last_error(std::string("Invalid tensor shape passed for ") + name + '.');
        return false;
    }
    if (d.stride0 < 0 || d.stride1 < 0 || d.stride2 < 0) {
        set_last_error(std::string("Negative tensor strides are not supported for ") + name + '.');
        return false;
    }
    const int64_t max_off = ((int64_t)d.dim0 - 1) * d.stride0 + ((int64_t)d.dim1 - 1) * d.stride1 + ((int64_t)d.dim2 - 1) * d.stride2;
    if (d.raw_bytes <= 0 || (d.raw_bytes % (int64_t)sizeof(float)) != 0 || d.raw_bytes < (max_off + 1) * (int64_t)sizeof(float)) {
        set_last_error(std::string("Invalid raw byte size passed for ") + name + '.');
        return false;
    }
    return true;
}

// innermost stride 1, rows and planes do not overlap (ggml_ops_core.cpp can_map_standard_view, 3-D form)
bool is_standard_view3(const TSHipTensorView3D& d)
{
    return d.stride2 == 1 && (d.dim1 == 1 || d.stride1 >= d.dim2) && (d.dim0 == 1 || (int64_t)d.stride0 >= (int64_t)d.stride1 * (d.dim1 - 1) + d.dim2);
}

bool validate_mul_mat_id(const TSHipTensorView3D& result, const TSHipTensorView3D& experts, const TSHipTensorView3D& input, const void* ids,
                         int ids_rows, int ids_cols)
{
    if (!validate_desc3(result, "result") || !validate_desc3(experts, "expertWeights") || !validate_desc3(input, "input")) return false;
    if (ids == nullptr) {
        set_last_error("Null pointer passed for ids.");
        return false;
    }
    if (ids_rows <= 0 || ids_cols <= 0) {
        set_last_error("mulmatid requires positive id matrix dimensions.");
        return false;
    }
    if (experts.dim2 != input.dim2) {
        set_last_error("mulmatid expects expert weights and input to share the inner dimension.");
        return false;
    }
    if (input.dim0 != ids_rows || (ids_cols % input.dim1) != 0) {
        set_last_error("mulmatid expects ids rows to match input tokens and ids cols to broadcast over input expert slots.");
        return false;
    }
    if (result.dim0 != input.dim0 || result.dim1 != ids_cols || result.dim2 != experts.dim1) {
        set_last_error("mulmatid expects result shape [tokens, expert_used, rows].");
        return false;
    }
    if (!is_standard_view3(result) || !is_standard_view3(experts) || !is_standard_view3(input)) {
        set_last_error("Tensor layout is not supported by the mulmatid path.");
        return false;
    }
    return true;
}

// (token, slot) pairs go out in launches of at most 65535, the limit of the launch's second grid dimension.
bool run_mul_mat_id(const TSHipTensorView3D& result, const TSHipTensorView3D& experts, const TSHipTensorView3D& input, const int32_t* ids_dev,
                    int ids_cols, hipStream_t stream)
{
    if (ids_cols > 65535) {
        set_last_error("mulmatid: more than 65535 id columns.");
        return false;
    }
    const int T = input.dim0, t_step = std::max(1, 65535 / ids_cols);
    for (int t0 = 0; t0 < T; t0 += t_step) {
        const int tn = std::min(t_step, T - t0);
        const float* x = static_cast<const float*>(input.data) + (size_t)t0 * input.stride0;
        float* y = static_cast<float*>(result.data) + (size_t)t0 * result.stride0;
        if (!launch_mul_mat_id_f32(static_cast<const float*>(experts.data), experts.stride0, experts.stride1, experts.dim0, experts.dim1,
                                   experts.dim2, x, input.stride0, input.stride1, input.dim1, ids_dev + (size_t)t0 * ids_cols, tn, ids_cols, y,
                                   result.stride0, result.stride1, stream))
            return false;
    }
    return true;
}

}  // namespace

int TSHip_MulMatIdF32Device(TSHipTensorView3D result, TSHipTensorView3D expert_weights, TSHipTensorView3D input, const int32_t* ids,
                            int ids_rows, int ids_cols)
{
    return guarded(0, "mulmatid", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_mul_mat_id(result, expert_weights, input, ids, ids_rows, ids_cols)) return 0;
        if (!run_mul_mat_id(result, expert_weights, input, ids, ids_cols, t_stream)) return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_MulMatIdF32(TSHipTensorView3D result, TSHipTensorView3D expert_weights, TSHipTensorView3D input, TSHipContiguousTensor ids,
                      int ids_rows, int ids_cols)
{
    return guarded(0, "mulmatid", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_mul_mat_id(result, expert_weights, input, ids.data, ids_rows, ids_cols)) return 0;
        const int64_t n_ids = (int64_t)ids_rows * ids_cols;
        if (ids.element_count != n_ids || (ids.element_type != 0 && ids.element_type != 3)) {
            set_last_error("mulmatid: ids must hold ids_rows x ids_cols I32 (or F32) values.");
            return 0;
        }
        std::vector<int32_t> id_host((size_t)n_ids);
        if (ids.element_type == 3) {
            std::memcpy(id_host.data(), ids.data, (size_t)n_ids * sizeof(int32_t));
        } else {
            for (int64_t i = 0; i < n_ids; ++i) id_host[(size_t)i] = (int32_t)static_cast<const float*>(ids.data)[i];
        }
        for (int32_t e : id_host)
            if (e < 0 || e >= expert_weights.dim0) {
                set_last_error("mulmatid: expert id out of range.");
                return 0;
            }
        // contiguous device copies: [ids][input T x slots x K][weights E x rows x K][result T x cols x rows]
        auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
        const int T = input.dim0, slots = input.dim1, K = input.dim2, E = expert_weights.dim0, rows = expert_weights.dim1;
        const size_t id_bytes = al((size_t)n_ids * sizeof(int32_t)), x_bytes = al((size_t)T * slots * K * sizeof(float));
        const size_t w_bytes = al((size_t)E * rows * K * sizeof(float)), y_bytes = al((size_t)T * ids_cols * rows * sizeof(float));
        std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
        if (!ws_reserve(id_bytes + x_bytes + w_bytes + y_bytes, std::max(id_bytes + x_bytes, y_bytes))) return 0;
        char* dev = static_cast<char*>(g_ws.dev);
        char* pin = static_cast<char*>(g_ws.pinned);
        std::memcpy(pin, id_host.data(), (size_t)n_ids * sizeof(int32_t));
        float* xs = reinterpret_cast<float*>(pin + id_bytes);
        for (int t = 0; t < T; ++t)
            for (int s = 0; s < slots; ++s)
                std::memcpy(xs + ((size_t)t * slots + s) * K,
                            static_cast<const float*>(input.data) + (size_t)t * input.stride0 + (size_t)s * input.stride1, (size_t)K * sizeof(float));
        hipStream_t stream = nullptr;
        if (!hip_ok(hipMemcpyAsync(dev, pin, id_bytes + x_bytes, hipMemcpyHostToDevice, stream), "hipMemcpy(inputs)")) return 0;
        // the weights go up from the caller's (pageable) memory plane by plane, row by row when rows are padded
        float* w_dev = reinterpret_cast<float*>(dev + id_bytes + x_bytes);
        const float* w_host = static_cast<const float*>(expert_weights.data);
        if (expert_weights.stride1 == K && (E == 1 || expert_weights.stride0 == (int64_t)rows * K)) {
            if (!hip_ok(hipMemcpy(w_dev, w_host, (size_t)E * rows * K * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy(expert weights)")) return 0;
        } else {
            for (int e = 0; e < E; ++e)
                if (!hip_ok(hipMemcpy2D(w_dev + (size_t)e * rows * K, (size_t)K * sizeof(float), w_host + (size_t)e * expert_weights.stride0,
                                        (size_t)expert_weights.stride1 * sizeof(float), (size_t)K * sizeof(float), (size_t)rows,
                                        hipMemcpyHostToDevice),
                            "hipMemcpy2D(expert weights)"))
                    return 0;
        }
        float* y_dev = reinterpret_cast<float*>(dev + id_bytes + x_bytes + w_bytes);
        const TSHipTensorView3D xd{dev + id_bytes, T, slots, K, slots * K, K, 1, (int64_t)((size_t)T * slots * K * sizeof(float))};
        const TSHipTensorView3D wd{w_dev, E, rows, K, rows * K, K, 1, (int64_t)((size_t)E * rows * K * sizeof(float))};
        const TSHipTensorView3D yd{y_dev, T, ids_cols, rows, ids_cols * rows, rows, 1, (int64_t)((size_t)T * ids_cols * rows * sizeof(float))};
        if (!run_mul_mat_id(yd, wd, xd, reinterpret_cast<const int32_t*>(dev), ids_cols, stream)) return 0;
        if (!hip_ok(hipMemcpyAsync(pin, y_dev, (size_t)T * ids_cols * rows * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpy(result)")) return 0;
        if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
        const float* ys = reinterpret_cast<const float*>(pin);
        for (int t = 0; t < T; ++t)
            for (int s = 0; s < ids_cols; ++s)
                std::memcpy(static_cast<float*>(result.data) + (size_t)t * result.stride0 + (size_t)s * result.stride1,
                            ys + ((size_t)t * ids_cols + s) * rows, (size_t)rows * sizeof(float));
        clear_last_error();
        return 1;
    });
}

/* ---- ggml_add_id: per-expert bias rows added to the rows of a mul_mat_id (ggml_ops_matmul.cpp:1123-1290) ---- */
namespace {

bool validate_add_id(const TSHipTensorView3D& result, const TSHipTensorView3D& src, const TSHipTensorView2D& bias, const void* ids,
                     int ids_rows, int ids_cols)
{
    if (!validate_desc3(result, "result") || !validate_desc3(src, "src") || !validate_desc(bias, "bias")) return false;
    if (ids == nullptr) {
        set_last_error("Null pointer passed for ids.");
        return false;
    }
    if (ids_rows <= 0 || ids_cols <= 0) {
        set_last_error("addid requires positive id matrix dimensions.");
        return false;
    }
    if (result.dim0 != src.dim0 || result.dim1 != src.dim1 || result.dim2 != src.dim2) {
        set_last_error("addid expects result and src to have the same shape.");
        return false;
    }
    if (src.dim0 != ids_rows || src.dim1 != ids_cols || src.dim2 != bias.dim1) {
        set_last_error("addid expects src shape [tokens, expert_used, rows], bias shape [experts, rows], and ids shape [tokens, expert_used].");
        return false;
    }
    if (!is_standard_view3(result) || !is_standard_view3(src) || !is_standard_view(bias)) {
        set_last_error("Tensor layout is not supported by the addid path.");
        return false;
    }
    return true;
}

}  // namespace

int TSHip_AddIdF32Device(TSHipTensorView3D result, TSHipTensorView3D src, TSHipTensorView2D bias, const int32_t* ids, int ids_rows,
                         int ids_cols)
{
    return guarded(0, "addid", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_add_id(result, src, bias, ids, ids_rows, ids_cols)) return 0;
        if (!launch_add_id_f32(static_cast<const float*>(src.data), src.stride0, src.stride1, static_cast<const float*>(bias.data), bias.stride0,
                               bias.dim0, ids, ids_rows, ids_cols, src.dim2, static_cast<float*>(result.data), result.stride0, result.stride1,
                               t_stream))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_AddIdF32(TSHipTensorView3D result, TSHipTensorView3D src, TSHipTensorView2D bias, TSHipContiguousTensor ids, int ids_rows,
                   int ids_cols)
{
    return guarded(0, "addid", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!validate_add_id(result, src, bias, ids.data, ids_rows, ids_cols)) return 0;
        const int64_t n_ids = (int64_t)ids_rows * ids_cols;
        if (ids.element_count != n_ids || (ids.element_type != 0 && ids.element_type != 3)) {
            set_last_error("addid: ids must hold ids_rows x ids_cols I32 (or F32) values.");
            return 0;
        }
        const int T = src.dim0, cols = src.dim1, rows = src.dim2, E = bias.dim0;
        auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
        const size_t id_bytes = al((size_t)n_ids * sizeof(int32_t)), x_bytes = al((size_t)n_ids * rows * sizeof(float));
        const size_t b_bytes = al((size_t)E * rows * sizeof(float));
        std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
        if (!ws_reserve(id_bytes + x_bytes + b_bytes, id_bytes + x_bytes + b_bytes)) return 0;
        char* dev = static_cast<char*>(g_ws.dev);
        char* pin = static_cast<char*>(g_ws.pinned);
        int32_t* id_host = reinterpret_cast<int32_t*>(pin);
        for (int64_t i = 0; i < n_ids; ++i) {
            const int32_t e = ids.element_type == 3 ? static_cast<const int32_t*>(ids.data)[i] : (int32_t)static_cast<const float*>(ids.data)[i];
            if (e < 0 || e >= E) {
                set_last_error("addid: expert id out of range.");
                return 0;
            }
            id_host[i] = e;
        }
        float* xs = reinterpret_cast<float*>(pin + id_bytes);
        for (int t = 0; t < T; ++t)
            for (int sl = 0; sl < cols; ++sl)
                std::memcpy(xs + ((size_t)t * cols + sl) * rows, static_cast<const float*>(src.data) + (size_t)t * src.stride0 + (size_t)sl * src.stride1,
                            (size_t)rows * sizeof(float));
        float* bs = reinterpret_cast<float*>(pin + id_bytes + x_bytes);
        for (int e = 0; e < E; ++e)
            std::memcpy(bs + (size_t)e * rows, static_cast<const float*>(bias.data) + (size_t)e * bias.stride0, (size_t)rows * sizeof(float));
        hipStream_t stream = nullptr;
        if (!hip_ok(hipMemcpyAsync(dev, pin, id_bytes + x_bytes + b_bytes, hipMemcpyHostToDevice, stream), "hipMemcpy(inputs)")) return 0;
        float* x_dev = reinterpret_cast<float*>(dev + id_bytes);
        // in place on the packed copy of src
        if (!launch_add_id_f32(x_dev, (int64_t)cols * rows, rows, reinterpret_cast<const float*>(dev + id_bytes + x_bytes), rows, E,
                               reinterpret_cast<const int32_t*>(dev), T, cols, rows, x_dev, (int64_t)cols * rows, rows, stream))
            return 0;
        if (!hip_ok(hipMemcpyAsync(xs, x_dev, (size_t)n_ids * rows * sizeof(float), hipMemcpyDeviceToHost, stream), "hipMemcpy(result)")) return 0;
        if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
        for (int t = 0; t < T; ++t)
            for (int sl = 0; sl < cols; ++sl)
                std::memcpy(static_cast<float*>(result.data) + (size_t)t * result.stride0 + (size_t)sl * result.stride1,
                            xs + ((size_t)t * cols + sl) * rows, (size_t)rows * sizeof(float));
        clear_last_error();
        return 1;
    });
}

}  // extern "C"

namespace {

struct LayerShape {
    int hidden, head_dim, num_heads, num_kv_heads, max_seq_len, intermediate;
    int qkv_type, o_type, gu_type, down_type;
    int64_t qkv_bytes, o_bytes, gu_bytes, down_bytes;
};

bool validate_layer(const LayerShape& L, int64_t qkv_ne0, int64_t qkv_ne1, int64_t o_ne0, int64_t o_ne1, int64_t gu_ne0, int64_t gu_ne1,
                    int64_t down_ne0, int64_t down_ne1, int position)
{
    const int64_t q_dim = (int64_t)L.num_heads * L.head_dim, k_dim = (int64_t)L.num_kv_heads * L.head_dim;
    if (L.hidden <= 0 || L.head_dim <= 0 || L.num_heads <= 0 || L.num_kv_heads <= 0 || L.intermediate <= 0 || L.max_seq_len <= 0 ||
        L.num_heads % L.num_kv_heads != 0) {
        set_last_error("Invalid dimensions for transformer layer decode.");
        return false;
    }
    if (position < 0 || position >= L.max_seq_len) {
        set_last_error("transformer layer decode: position outside the KV cache.");
        return false;
    }
    if (qkv_ne0 != L.hidden || qkv_ne1 != q_dim + 2 * k_dim || o_ne0 != q_dim || o_ne1 != L.hidden || gu_ne0 != L.hidden ||
        gu_ne1 != 2 * (int64_t)L.intermediate || down_ne0 != L.intermediate || down_ne1 != L.hidden) {
        set_last_error("Size mismatch: layer weight dims don't match in transformer layer decode.");
        return false;
    }
    const struct { int type; int64_t ne0, ne1, bytes; } ws[4] = {{L.qkv_type, qkv_ne0, qkv_ne1, L.qkv_bytes}, {L.o_type, o_ne0, o_ne1, L.o_bytes},
                                                                 {L.gu_type, gu_ne0, gu_ne1, L.gu_bytes}, {L.down_type, down_ne0, down_ne1, L.down_bytes}};
    for (const auto& w : ws) {
        const size_t rs = row_size(w.type, w.ne0);
        if (!is_quant_type(w.type) || rs == 0 || (size_t)w.bytes < rs * (size_t)w.ne1) {
            set_last_error("Unsupported quantized weight type, row length or byte span in transformer layer decode.");
            return false;
        }
    }
    return true;
}

// one token through one layer (ggml_ops_transformer.cpp:379-470); every pointer in device memory
bool run_layer_decode(float* hidden, const LayerShape& L, const float* attn_norm, const void* qkv, const float* q_norm,
                      const float* k_norm, const void* o, const float* ffn_norm, const void* gu, const void* down, float* k_cache,
                      float* v_cache, int position, float eps, float rope_base, float rope_freq_scale, int rope_mode, hipStream_t stream,
                      const float* next_attn_norm = nullptr)
{
    const int q_dim = L.num_heads * L.head_dim, k_dim = L.num_kv_heads * L.head_dim, qkv_n = q_dim + 2 * k_dim;
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t b_qkv = al((size_t)qkv_n * 4), b_attn = al((size_t)q_dim * 4);
    const size_t b_part = al(attention_decode_ws_bytes(L.num_heads, position + 1));
    const size_t b_mm = al(std::max(matmul_ws_bytes(L.qkv_type, 1, L.hidden, qkv_n, true, false), matmul_ws_bytes(L.o_type, 1, q_dim, L.hidden, false, true)));
    const size_t b_ffn = ffn_ws_bytes(1, L.gu_type, L.down_type, L.hidden, L.intermediate);
    WsLease lease(stream, b_qkv + b_attn + b_part + b_mm + b_ffn);
    if (!lease.ok()) return false;
    char* ws = lease.ptr();
    float* qkv_out = reinterpret_cast<float*>(ws);
    float* attn = reinterpret_cast<float*>(ws + b_qkv);
    float* part = reinterpret_cast<float*>(ws + b_qkv + b_attn);
    void* mm_ws = ws + b_qkv + b_attn + b_part;
    const TSHipTensorView2D h_view{hidden, 1, L.hidden, L.hidden, 1, (int64_t)L.hidden * 4};
    const TSHipTensorView2D qkv_view{qkv_out, 1, qkv_n, qkv_n, 1, (int64_t)qkv_n * 4};
    const TSHipTensorView2D attn_view{attn, 1, q_dim, q_dim, 1, (int64_t)q_dim * 4};
    if (!run_matmul_device_ws(qkv_view, h_view, qkv, L.qkv_type, L.hidden, qkv_n, stream, mm_ws, b_mm, attn_norm, eps, false)) return false;
    if (!launch_attention_decode(qkv_out, q_norm, k_norm, eps, rope_base, rope_freq_scale, rope_mode, k_cache, v_cache, L.num_heads,
                                 L.num_kv_heads, L.head_dim, L.max_seq_len, position, part, attn, stream, ffn_norm, next_attn_norm, L.hidden))
        return false;
    // hidden += W_o attn
    if (!run_matmul_device_ws(h_view, attn_view, o, L.o_type, q_dim, L.hidden, stream, mm_ws, b_mm, nullptr, 0.f, true)) return false;
    // hidden += W_down(silu(g) * u); the FFN reads hidden (RMSNorm) before its last kernel adds into it
    return run_ffn_swiglu_device(h_view, h_view, ffn_norm, eps, gu, L.gu_type, down, L.down_type, L.hidden, L.intermediate, stream,
                                 ws + b_qkv + b_attn + b_part + b_mm);
}

}  // namespace

// ---- host-pointer forms (the bridge's own argument lists) -------------------------------------
// hidden travels per call; everything else - norm weights, raw weight blocks, the fp32 KV caches - lives in device
// buffers kept under the host pointer the caller passes (uploaded on first use, like the bridge's cacheable buffers,
// ggml_ops_transformer.cpp:244-300).  The device copy of a KV cache is the one that is updated: TSHip_SyncHostBuffer
// brings it back to host memory, TSHip_InvalidateHostBuffer makes the next call upload the host bytes again.
namespace {
struct HostLayer {
    const float* attn_norm;
    const void* qkv;
    const float* q_norm;
    const float* k_norm;
    const void* o;
    const float* ffn_norm;
    const void* gu;
    const void* down;
    float* k_cache;
    float* v_cache;
};

bool resolve_layer(const LayerShape& L, void* attn_norm, void* qkv, void* q_norm, void* k_norm, void* o, void* ffn_norm, void* gu,
                   void* down, void* k_cache, void* v_cache, HostLayer* out)
{
    const size_t kv_bytes = (size_t)L.num_kv_heads * L.max_seq_len * L.head_dim * sizeof(float);
    auto f32 = [](void* p, size_t n) { return p ? static_cast<const float*>(resolve_weight(p, n * sizeof(float))) : nullptr; };
    out->attn_norm = f32(attn_norm, (size_t)L.hidden);
    out->ffn_norm = f32(ffn_norm, (size_t)L.hidden);
    out->q_norm = f32(q_norm, (size_t)L.head_dim);
    out->k_norm = f32(k_norm, (size_t)L.head_dim);
    out->qkv = resolve_weight(qkv, (size_t)L.qkv_bytes);
    out->o = resolve_weight(o, (size_t)L.o_bytes);
    out->gu = resolve_weight(gu, (size_t)L.gu_bytes);
    out->down = resolve_weight(down, (size_t)L.down_bytes);
    out->k_cache = static_cast<float*>(const_cast<void*>(resolve_weight(k_cache, kv_bytes)));
    out->v_cache = static_cast<float*>(const_cast<void*>(resolve_weight(v_cache, kv_bytes)));
    return out->attn_norm && out->ffn_norm && (!q_norm || out->q_norm) && (!k_norm || out->k_norm) && out->qkv && out->o && out->gu &&
           out->down && out->k_cache && out->v_cache;
}

// hidden: host -> device, `layers` layer steps, device -> host
template <typename Layers>
int decode_with_host_hidden(float* hidden, int hidden_size, Layers&& layers)
{
    const size_t h_bytes = ((size_t)hidden_size * sizeof(float) + 255) & ~(size_t)255;
    if (!ws_reserve(h_bytes, h_bytes)) return 0;
    hipStream_t stream = nullptr;
    std::memcpy(g_ws.pinned, hidden, (size_t)hidden_size * sizeof(float));
    if (!hip_ok(hipMemcpyAsync(g_ws.dev, g_ws.pinned, h_bytes, hipMemcpyHostToDevice, stream), "hipMemcpy(hidden)")) return 0;
    if (!layers(static_cast<float*>(g_ws.dev), stream)) return 0;
    if (!hip_ok(hipMemcpyAsync(g_ws.pinned, g_ws.dev, h_bytes, hipMemcpyDeviceToHost, stream), "hipMemcpy(hidden)")) return 0;
    if (!hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize")) return 0;
    std::memcpy(hidden, g_ws.pinned, (size_t)hidden_size * sizeof(float));
    clear_last_error();
    return 1;
}
}  // namespace

extern "C" {

int TSHip_TransformerLayerDecodeDevice(float* hidden, int hidden_size, const float* attn_norm, const void* qkv_data, int qkv_type,
                                       int64_t qkv_ne0, int64_t qkv_ne1, int64_t qkv_bytes, const float* q_norm, const float* k_norm,
                                       int head_dim, const void* o_data, int o_type, int64_t o_ne0, int64_t o_ne1, int64_t o_bytes,
                                       const float* ffn_norm, const void* gu_data, int gu_type, int64_t gu_ne0, int64_t gu_ne1,
                                       int64_t gu_bytes, const void* down_data, int down_type, int64_t down_ne0, int64_t down_ne1,
                                       int64_t down_bytes, float* k_cache, float* v_cache, int num_heads, int num_kv_heads,
                                       int max_seq_len, int position, float eps, float rope_base, float rope_freq_scale,
                                       int intermediate_size, int rope_mode)
{
    return guarded(0, "transformer_layer_decode", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!hidden || !attn_norm || !qkv_data || !o_data || !ffn_norm || !gu_data || !down_data || !k_cache || !v_cache) {
            set_last_error("Invalid arguments for transformer layer decode.");
            return 0;
        }
        const LayerShape L{hidden_size, head_dim, num_heads, num_kv_heads, max_seq_len, intermediate_size, qkv_type, o_type, gu_type,
                           down_type, qkv_bytes, o_bytes, gu_bytes, down_bytes};
        if (!validate_layer(L, qkv_ne0, qkv_ne1, o_ne0, o_ne1, gu_ne0, gu_ne1, down_ne0, down_ne1, position)) return 0;
        if (!run_layer_decode(hidden, L, attn_norm, qkv_data, q_norm, k_norm, o_data, ffn_norm, gu_data, down_data, k_cache, v_cache,
                              position, eps, rope_base, rope_freq_scale, rope_mode, t_stream))
            return 0;
        clear_last_error();
        return 1;
    });
}

int TSHip_TransformerModelDecodeDevice(float* hidden, int hidden_size, int num_layers, const float* const* attn_norm,
                                       const void* const* qkv, const float* const* q_norm, const float* const* k_norm,
                                       const void* const* o, const float* const* ffn_norm, const void* const* gu,
                                       const void* const* down, float* const* k_cache, float* const* v_cache, int qkv_type,
                                       int64_t qkv_ne0, int64_t qkv_ne1, int64_t qkv_bytes, int o_type, int64_t o_ne0, int64_t o_ne1,
                                       int64_t o_bytes, int gu_type, int64_t gu_ne0, int64_t gu_ne1, int64_t gu_bytes, int down_type,
                                       int64_t down_ne0, int64_t down_ne1, int64_t down_bytes, int head_dim, int num_heads,
                                       int num_kv_heads, int max_seq_len, int position, float eps, float rope_base,
                                       float rope_freq_scale, int intermediate_size, int rope_mode)
{
    return guarded(0, "transformer_model_decode", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!hidden || num_layers <= 0 || !attn_norm || !qkv || !o || !ffn_norm || !gu || !down || !k_cache || !v_cache) {
            set_last_error("Invalid arguments for transformer model decode.");
            return 0;
        }
        const LayerShape L{hidden_size, head_dim, num_heads, num_kv_heads, max_seq_len, intermediate_size, qkv_type, o_type, gu_type,
                           down_type, qkv_bytes, o_bytes, gu_bytes, down_bytes};
        if (!validate_layer(L, qkv_ne0, qkv_ne1, o_ne0, o_ne1, gu_ne0, gu_ne1, down_ne0, down_ne1, position)) return 0;
        for (int l = 0; l < num_layers; ++l) {
            if (!attn_norm[l] || !qkv[l] || !o[l] || !ffn_norm[l] || !gu[l] || !down[l] || !k_cache[l] || !v_cache[l]) {
                set_last_error("transformer model decode: a layer pointer is null.");
                return 0;
            }
            if (!run_layer_decode(hidden, L, attn_norm[l], qkv[l], q_norm ? q_norm[l] : nullptr, k_norm ? k_norm[l] : nullptr, o[l],
                                  ffn_norm[l], gu[l], down[l], k_cache[l], v_cache[l], position, eps, rope_base, rope_freq_scale,
                                  rope_mode, t_stream, l + 1 < num_layers ? static_cast<const float*>(attn_norm[l + 1]) : nullptr))
                return 0;
        }
        clear_last_error();
        return 1;
    });
}

int TSHip_TransformerLayerDecode(void* hidden, int hidden_size, void* attn_norm, void* qkv_data, int qkv_type, int64_t qkv_ne0,
                                 int64_t qkv_ne1, int64_t qkv_bytes, void* q_norm, void* k_norm, int head_dim, void* o_data, int o_type,
                                 int64_t o_ne0, int64_t o_ne1, int64_t o_bytes, void* ffn_norm, void* gu_data, int gu_type,
                                 int64_t gu_ne0, int64_t gu_ne1, int64_t gu_bytes, void* down_data, int down_type, int64_t down_ne0,
                                 int64_t down_ne1, int64_t down_bytes, void* k_cache, void* v_cache, int num_heads, int num_kv_heads,
                                 int max_seq_len, int position, float eps, float rope_base, float rope_freq_scale,
                                 int intermediate_size, int rope_mode)
{
    return guarded(0, "transformer_layer_decode", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!hidden || !attn_norm || !qkv_data || !o_data || !ffn_norm || !gu_data || !down_data || !k_cache || !v_cache) {
            set_last_error("Invalid arguments for transformer layer decode.");
            return 0;
        }
        const LayerShape L{hidden_size, head_dim, num_heads, num_kv_heads, max_seq_len, intermediate_size, qkv_type, o_type, gu_type,
                           down_type, qkv_bytes, o_bytes, gu_bytes, down_bytes};
        if (!validate_layer(L, qkv_ne0, qkv_ne1, o_ne0, o_ne1, gu_ne0, gu_ne1, down_ne0, down_ne1, position)) return 0;
        std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
        HostLayer d;
        if (!resolve_layer(L, attn_norm, qkv_data, q_norm, k_norm, o_data, ffn_norm, gu_data, down_data, k_cache, v_cache, &d)) return 0;
        return decode_with_host_hidden(static_cast<float*>(hidden), hidden_size, [&](float* h, hipStream_t stream) {
            return run_layer_decode(h, L, d.attn_norm, d.qkv, d.q_norm, d.k_norm, d.o, d.ffn_norm, d.gu, d.down, d.k_cache, d.v_cache,
                                    position, eps, rope_base, rope_freq_scale, rope_mode, stream);
        });
    });
}

int TSHip_TransformerModelDecode(void* hidden, int hidden_size, int num_layers, void* const* attn_norm, void* const* qkv,
                                 void* const* q_norm, void* const* k_norm, void* const* o, void* const* ffn_norm, void* const* gu,
                                 void* const* down, void* const* k_cache, void* const* v_cache, int qkv_type, int64_t qkv_ne0,
                                 int64_t qkv_ne1, int64_t qkv_bytes, int o_type, int64_t o_ne0, int64_t o_ne1, int64_t o_bytes,
                                 int gu_type, int64_t gu_ne0, int64_t gu_ne1, int64_t gu_bytes, int down_type, int64_t down_ne0,
                                 int64_t down_ne1, int64_t down_bytes, int head_dim, int num_heads, int num_kv_heads, int max_seq_len,
                                 int position, float eps, float rope_base, float rope_freq_scale, int intermediate_size, int rope_mode)
{
    return guarded(0, "transformer_model_decode", [&]() -> int {
        if (!ensure_backend()) return 0;
        if (!hidden || num_layers <= 0 || !attn_norm || !qkv || !o || !ffn_norm || !gu || !down || !k_cache || !v_cache) {
            set_last_error("Invalid arguments for transformer model decode.");
            return 0;
        }
        const LayerShape L{hidden_size, head_dim, num_heads, num_kv_heads, max_seq_len, intermediate_size, qkv_type, o_type, gu_type,
                           down_type, qkv_bytes, o_bytes, gu_bytes, down_bytes};
        if (!validate_layer(L, qkv_ne0, qkv_ne1, o_ne0, o_ne1, gu_ne0, gu_ne1, down_ne0, down_ne1, position)) return 0;
        std::lock_guard<std::recursive_mutex> lock(g_host_call_mutex);
        std::vector<HostLayer> d((size_t)num_layers);
        for (int l = 0; l < num_layers; ++l) {
            if (!attn_norm[l] || !qkv[l] || !o[l] || !ffn_norm[l] || !gu[l] || !down[l] || !k_cache[l] || !v_cache[l]) {
                set_last_error("transformer model decode: a layer pointer is null.");
                return 0;
            }
            if (!resolve_layer(L, attn_norm[l], qkv[l], q_norm ? q_norm[l] : nullptr, k_norm ? k_norm[l] : nullptr, o[l], ffn_norm[l],
                               gu[l], down[l], k_cache[l], v_cache[l], &d[(size_t)l]))
                return 0;
        }
        return decode_with_host_hidden(static_cast<float*>(hidden), hidden_size, [&](float* h, hipStream_t stream) {
            for (size_t l = 0; l < d.size(); ++l) {
                const HostLayer& x = d[l];
                if (!run_layer_decode(h, L, x.attn_norm, x.qkv, x.q_norm, x.k_norm, x.o, x.ffn_norm, x.gu, x.down, x.k_cache, x.v_cache,
                                      position, eps, rope_base, rope_freq_scale, rope_mode, stream,
                                      l + 1 < d.size() ? d[l + 1].attn_norm : nullptr))
                    return false;
            }
            return true;
        });
    });
}

}  // extern "C"
