// C ABI of libvxhip_w8a8 (see include/vxhip_w8a8.h): handle lifetimes, the
// host-side admission proofs, and the choice between the MFMA GEMM and the
// streaming GEMV.  No arithmetic on tensor data happens on the host.
#include "common.h"

#include <limits.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <memory>
#include <sys/syscall.h>
#include <unistd.h>
#include <mutex>
#include <vector>

namespace vxhip {

static thread_local char g_error[512] = "";
static thread_local char g_force[64] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}

VxHipStatus hip_status(hipError_t e, const char* what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    (void)hipGetLastError();
    if (e == hipErrorOutOfMemory) return VXHIP_OUT_OF_MEMORY;
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) return VXHIP_BACKEND_UNAVAILABLE;
    if (e == hipErrorIllegalAddress || e == hipErrorLaunchFailure || e == hipErrorECCNotCorrectable)
        return VXHIP_DEVICE_LOST;
    return VXHIP_EXECUTION_FAILED;
}

const char* forced_variant() { return g_force[0] ? g_force : nullptr; }

static bool byte_dtype(uint32_t d) { return d == VXHIP_DTYPE_I8 || d == VXHIP_DTYPE_U8; }
static bool zero_point_ok(int32_t zp, uint32_t d) {
    return d == VXHIP_DTYPE_I8 ? (zp >= -128 && zp <= 127) : (zp >= 0 && zp <= 255);
}
static bool scale_ok(float v) { return isfinite(v) && v > 0.0f; }

// f32(f32(s_in * s_w) / s_out), each step rounded to f32
// (native/src/backends/qlinear_multiplier.h:12-27).
static bool multiplier_ok(float s_in, float s_w, float s_out) {
    volatile float p = s_in * s_w;
    volatile float m = p / s_out;
    return scale_ok(m);
}

VxHipStatus ensure_scratch(VxHipContext* ctx, size_t bytes) {
    if (bytes <= ctx->scratch_bytes) return VXHIP_OK;
    if (ctx->recording) {
        set_error("the context's scratch would have to grow while its launches are being recorded: run the same "
                  "calls once before recording them");
        return VXHIP_INVALID_ARGUMENT;
    }
    // The outgrown block is retired, not freed: launches in flight may still read it, and a HIP
    // graph captured on this context keeps its address and may be replayed after this call.
    // Growing at least doubles the block, so the retired ones add up to less than the live one.
    if (ctx->scratch && ctx->retired_count == VxHipContext::kRetiredSlots) {
        set_error("context scratch grew more often than %d times", VxHipContext::kRetiredSlots);
        return VXHIP_INTERNAL;
    }
    size_t want = (bytes + (1u << 20)) & ~((size_t)(1u << 20) - 1u);
    if (want < 2 * ctx->scratch_bytes) want = 2 * ctx->scratch_bytes;
    void* fresh = nullptr;
    VXHIP_TRY(hipMalloc(&fresh, want));
    if (ctx->scratch) ctx->retired[ctx->retired_count++] = ctx->scratch;
    ctx->scratch = fresh;
    ctx->scratch_bytes = want;
    return VXHIP_OK;
}

void set_last_variant(VxHipContext* ctx, const char* id) {
    snprintf(ctx->last_variant, sizeof ctx->last_variant, "%s", id ? id : "");
}

struct Carver {
    char* base;
    size_t off = 0;
    template <class T>
    T* take(size_t count) {
        off = (off + 255u) & ~(size_t)255u;
        T* p = base ? reinterpret_cast<T*>(base + off) : nullptr;
        off += count * sizeof(T);
        return p;
    }
};

// ---- scratch of the entry point that allocates nothing ---------------------------------------
// vxhip_packed_linear_forward_f32_noalloc stages its prepared activations (one f32 scale per row,
// then the int8 codes) here instead of in a context's grow-only scratch.  The array lives in every
// device's copy of the code object, at an address of its own on each device: host code never uses
// the array's name as a pointer, only the per-device address looked up once, with that device
// current, when the first context on the device is created.
constexpr size_t kNoAllocScratchBytes = 4u << 20;
static __device__ __align__(256) unsigned char g_no_alloc_scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
static std::mutex g_no_alloc_mutex;
static void* g_no_alloc_ptr[kMaxDevices] = {};
static hipError_t g_no_alloc_status[kMaxDevices] = {};
static bool g_no_alloc_looked_up[kMaxDevices] = {};

// Looks the array's address up on `device`, which must be current.  Returns null on failure (the
// error text is set); the failure is remembered, so the entry point reports it instead of trying
// again at a time when the caller may not allocate.
static void* no_alloc_scratch(int device) {
    if (device < 0 || device >= kMaxDevices) {
        set_error("device ordinal %d is outside the table of %d", device, kMaxDevices);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_no_alloc_mutex);
    if (!g_no_alloc_looked_up[device]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_no_alloc_scratch));
        if (e != hipSuccess) (void)hipGetLastError();
        g_no_alloc_status[device] = e;
        g_no_alloc_ptr[device] = e == hipSuccess ? ptr : nullptr;
        g_no_alloc_looked_up[device] = true;
    }
    if (!g_no_alloc_ptr[device])
        set_error("hipGetSymbolAddress(no-alloc scratch) failed on device %d: %s", device,
                  hipGetErrorString(g_no_alloc_status[device]));
    return g_no_alloc_ptr[device];
}

static bool use_device(int device) {
    if (hipSetDevice(device) != hipSuccess) {
        set_error("hipSetDevice(%d) failed", device);
        return false;
    }
    return true;
}

// The context of the host-pointer entry points: device 0, one per thread.  Its device is made
// current on every use, because the handles those entry points create live on the current device.
// ---- weights of the host-pointer entry points, kept resident --------------------------------------
// vxhip_qlinear_i8u8 and vxhip_packed_linear_f32 receive their weights as host pointers on every call,
// as the VxW8A8Ops slots do.  The reference's device routes keep such immutable inputs resident, keyed
// by the host pointer (graph_ensure_input(ptr, bytes, 1),
// native/src/backends/cuda/host/cuda_graph_quantized_linear_conv_host.inc:74-77); so does this one: the
// prepacked weight with its scales, zero points and bias is built once per (pointers, shape, type) and
// reused.  On top of the reference's rule a fingerprint of the bytes is part of the key (all of the
// per-channel arrays, and of the weight its ends and a few hundred samples), so that a buffer that was
// refilled in place is packed again rather than served stale -- a caller that rewrites single weights
// calls vxhip_resident_weights_clear.  Least recently used entries go when the entry or byte limit is
// reached (VXHIP_RESIDENT_WEIGHT_BYTES, default 4 GiB).  An entry in use by another thread outlives
// its eviction.
struct ResidentWeights {
    VxHipQLinear* qlinear = nullptr;
    VxHipPackedLinear* packed = nullptr;
    ~ResidentWeights() {
        if (qlinear) vxhip_qlinear_destroy(qlinear);
        if (packed) vxhip_packed_linear_destroy(packed);
    }
};
struct ResidentKey {
    const void* pointers[4];
    uint32_t extents[4];
    uint64_t fingerprint;
    bool operator==(const ResidentKey& o) const { return memcmp(this, &o, sizeof(*this)) == 0; }
};
struct ResidentSlot {
    ResidentKey key;
    std::shared_ptr<ResidentWeights> weights;
    uint64_t last_use;
    size_t bytes;
};
static std::mutex g_resident_mutex;
// never destroyed: at process exit the runtime may already be gone when static destructors run
static std::vector<ResidentSlot>& g_resident = *new std::vector<ResidentSlot>();
static uint64_t g_resident_clock = 0;
constexpr size_t kResidentMaxEntries = 256;

static size_t resident_limit_bytes() {
    const char* text = getenv("VXHIP_RESIDENT_WEIGHT_BYTES");
    if (text && *text) return (size_t)strtoull(text, nullptr, 10);
    return (size_t)4 << 30;
}

static uint64_t fnv1a(uint64_t h, const void* data, size_t bytes) {
    const unsigned char* p = (const unsigned char*)data;
    size_t i = 0;
    for (; i + 8u <= bytes; i += 8u) {  // eight bytes a step: this runs on every call
        uint64_t word;
        memcpy(&word, p + i, 8u);
        h = (h ^ word) * 0x100000001b3ull;
        h ^= h >> 29;
    }
    for (; i < bytes; i++) h = (h ^ p[i]) * 0x100000001b3ull;
    return h;
}
// all of a small array; of a large one both ends and 512 samples of 8 bytes spread evenly
static uint64_t fingerprint(uint64_t h, const void* data, size_t bytes) {
    if (!data) return fnv1a(h, "null", 4);
    h = fnv1a(h, &bytes, sizeof bytes);
    if (bytes <= 65536u) return fnv1a(h, data, bytes);
    const unsigned char* p = (const unsigned char*)data;
    h = fnv1a(h, p, 8192u);
    h = fnv1a(h, p + bytes - 8192u, 8192u);
    const size_t stride = (bytes - 16384u) / 512u;
    for (size_t i = 0; i < 512u; i++) h = fnv1a(h, p + 8192u + i * stride, 8u);
    return h;
}

static std::shared_ptr<ResidentWeights> resident_find(const ResidentKey& key) {
    std::lock_guard<std::mutex> lock(g_resident_mutex);
    for (ResidentSlot& slot : g_resident)
        if (slot.key == key) {
            slot.last_use = ++g_resident_clock;
            return slot.weights;
        }
    return nullptr;
}

static void resident_insert(const ResidentKey& key, const std::shared_ptr<ResidentWeights>& weights, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_resident_mutex);
    for (const ResidentSlot& slot : g_resident)
        if (slot.key == key) return;  // another thread packed the same weight meanwhile: this copy serves its call only
    const size_t limit = resident_limit_bytes();
    if (bytes > limit) return;  // used for this call only
    size_t held = bytes;
    for (const ResidentSlot& slot : g_resident) held += slot.bytes;
    while (!g_resident.empty() && (held > limit || g_resident.size() >= kResidentMaxEntries)) {
        size_t oldest = 0;
        for (size_t i = 1; i < g_resident.size(); i++)
            if (g_resident[i].last_use < g_resident[oldest].last_use) oldest = i;
        held -= g_resident[oldest].bytes;
        g_resident.erase(g_resident.begin() + (long)oldest);
    }
    g_resident.push_back(ResidentSlot{key, weights, ++g_resident_clock, bytes});
}

// device staging of a host-pointer call's activations and outputs, grown as needed and kept by the context
static bool io_staging(VxHipContext* ctx, size_t in_bytes, size_t out_bytes) {
    if (in_bytes > ctx->io_in_bytes) {
        (void)hipStreamSynchronize(ctx->stream);
        if (ctx->io_in) (void)hipFree(ctx->io_in);
        ctx->io_in = nullptr;
        ctx->io_in_bytes = 0;
        if (hipMalloc(&ctx->io_in, in_bytes) != hipSuccess) return false;
        ctx->io_in_bytes = in_bytes;
    }
    if (out_bytes > ctx->io_out_bytes) {
        (void)hipStreamSynchronize(ctx->stream);
        if (ctx->io_out) (void)hipFree(ctx->io_out);
        ctx->io_out = nullptr;
        ctx->io_out_bytes = 0;
        if (hipMalloc(&ctx->io_out, out_bytes) != hipSuccess) return false;
        ctx->io_out_bytes = out_bytes;
    }
    return true;
}

// The context of the host-pointer entry points: one per calling thread, released when that thread ends.
// (Not on the main thread, whose thread-local objects die at process exit, when nothing should be
// asked of the runtime any more.)
struct ThreadContext {
    VxHipContext* ctx = nullptr;
    ~ThreadContext() {
        if (ctx && (pid_t)syscall(SYS_gettid) != getpid()) vxhip_context_destroy(ctx);
    }
};
static VxHipContext* default_context() {
    static thread_local ThreadContext holder;
    VxHipContext*& ctx = holder.ctx;
    if (!ctx && vxhip_context_create(0, nullptr, VXHIP_CONTEXT_OWN_STREAM, &ctx) != VXHIP_OK) ctx = nullptr;
    if (ctx && !use_device(ctx->device)) return nullptr;
    return ctx;
}

// Entry points that copy to or from the host or wait for the stream have no place in a recording.
static bool not_recording(const VxHipContext* ctx, const char* who) {
    if (!ctx->recording) return true;
    set_error("%s: the context is recording its launches; host copies and waits cannot be recorded", who);
    return false;
}

// A compiled weight is used on the device it was created on.
static bool same_device(const VxHipContext* ctx, int handle_device, const char* who) {
    if (ctx->device == handle_device) return true;
    set_error("%s: the handle lives on device %d, the context on device %d", who, handle_device, ctx->device);
    return false;
}

// Picks the kernel family for the shape and launches it.
static const char* run_linear(VxHipContext* ctx, const LinearArgs& a) {
    const char* force = forced_variant();
    const bool force_gemm = force && strstr(force, "mfma-i8") != nullptr && !strstr(force, "gemv");
    const bool force_gemm_f = force && strstr(force, "a8-mfma") != nullptr;
    const bool force_gemv = force && strstr(force, "gemv") != nullptr;
    const char* id = nullptr;
    if (force_gemv) return launch_gemv_stream(ctx->stream, a, ctx->cu_count, force);
    if (force_gemm || force_gemm_f) return launch_gemm_mfma(ctx->stream, a, ctx->cu_count, force);
    if (a.rows <= kMaxGemvRows) id = launch_gemv_stream(ctx->stream, a, ctx->cu_count, force);
    if (!id) id = launch_gemm_mfma(ctx->stream, a, ctx->cu_count, force);
    return id;
}

}  // namespace vxhip

using namespace vxhip;

extern "C" {

uint32_t vxhip_abi_version(void) { return VXHIP_ABI_VERSION; }

const char* vxhip_last_error(void) { return g_error; }

int32_t vxhip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int ok = 0;
    for (int i = 0; i < n; i++) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, i) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0)
            ok++;
    }
    return ok;
}

VxHipStatus vxhip_device_name(int32_t device, char* buffer, size_t capacity) {
    if (!buffer || !capacity) return VXHIP_INVALID_ARGUMENT;
    hipDeviceProp_t prop;
    VXHIP_TRY(hipGetDeviceProperties(&prop, device));
    snprintf(buffer, capacity, "%s (%s), %d CU, %.0f GiB", prop.name, prop.gcnArchName,
             prop.multiProcessorCount, (double)prop.totalGlobalMem / (1024.0 * 1024.0 * 1024.0));
    return VXHIP_OK;
}

void vxhip_force_variant(const char* id_prefix) {
    snprintf(g_force, sizeof g_force, "%s", id_prefix ? id_prefix : "");
}

// ---- context -----------------------------------------------------------------

VxHipStatus vxhip_context_create(int32_t device, void* stream, uint32_t flags, VxHipContext** out) {
    if (!out || flags > VXHIP_CONTEXT_BORROW_STREAM) return VXHIP_INVALID_ARGUMENT;
    *out = nullptr;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) {
        (void)hipGetLastError();
        set_error("no HIP device %d", device);
        return VXHIP_BACKEND_UNAVAILABLE;
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
        return VXHIP_BACKEND_UNAVAILABLE;
    }
    VXHIP_TRY(hipSetDevice(device));
    VxHipContext* ctx = new (std::nothrow) VxHipContext();
    if (!ctx) return VXHIP_OUT_OF_MEMORY;
    ctx->device = device;
    // set-up of the entry point that allocates nothing: this device's address of its scratch array
    // (a failure is reported by that entry point, not here)
    ctx->no_alloc_scratch = no_alloc_scratch(device);
    ctx->cu_count = prop.multiProcessorCount;
    if (flags == VXHIP_CONTEXT_BORROW_STREAM) {
        ctx->stream = (hipStream_t)stream;
    } else {
        hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            delete ctx;
            return hip_status(e, "hipStreamCreateWithFlags");
        }
        ctx->own_stream = true;
    }
    hipError_t e = hipMalloc((void**)&ctx->fault_dev, 256);
    if (e == hipSuccess) e = hipMemset(ctx->fault_dev, 0, 256);
    if (e == hipSuccess)
        e = hipMalloc((void**)&ctx->div_proof_dev, VxHipContext::kDivisorSlots * 2 * sizeof(uint32_t));
    if (e != hipSuccess) {
        vxhip_context_destroy(ctx);
        return hip_status(e, "fault word");
    }
    *out = ctx;
    return VXHIP_OK;
}

void vxhip_context_destroy(VxHipContext* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->recording) {  // an open recording is abandoned
        hipGraph_t graph = nullptr;
        if (hipStreamEndCapture(ctx->stream, &graph) == hipSuccess && graph) (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
    }
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    for (int i = 0; i < ctx->retired_count; i++) (void)hipFree(ctx->retired[i]);
    if (ctx->fault_dev) (void)hipFree(ctx->fault_dev);
    if (ctx->div_proof_dev) (void)hipFree(ctx->div_proof_dev);
    if (ctx->io_in) (void)hipFree(ctx->io_in);
    if (ctx->io_out) (void)hipFree(ctx->io_out);
    if (ctx->own_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

VxHipStatus vxhip_context_synchronize(VxHipContext* ctx) {
    if (!ctx) return VXHIP_INVALID_ARGUMENT;
    if (!not_recording(ctx, "context_synchronize")) return VXHIP_INVALID_ARGUMENT;
    VXHIP_TRY(hipStreamSynchronize(ctx->stream));
    return VXHIP_OK;
}

// Recording and replay of a context's launches: the reference's device route captures a forward pass
// on its stream and replays the instantiated graph on later passes
// (native/src/backends/cuda/host/cuda_graph_lifecycle_host.inc:184-188 cuStreamBeginCapture, :236-262
// instantiate and first launch, :285-290 replay).
VxHipStatus vxhip_context_begin_recording(VxHipContext* ctx) {
    if (!ctx || ctx->recording) {
        set_error("context_begin_recording: null context, or a recording is already open");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!use_device(ctx->device)) return VXHIP_BACKEND_UNAVAILABLE;
    VXHIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->recording = true;
    return VXHIP_OK;
}

VxHipStatus vxhip_context_end_recording(VxHipContext* ctx, VxHipReplay** out) {
    if (out) *out = nullptr;
    if (!ctx || !ctx->recording) {
        set_error("context_end_recording: null context, or no recording is open");
        return VXHIP_INVALID_ARGUMENT;
    }
    ctx->recording = false;
    hipGraph_t graph = nullptr;
    const hipError_t ended = hipStreamEndCapture(ctx->stream, &graph);
    if (ended != hipSuccess || !graph) {
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        set_error("context_end_recording: the stream did not yield a graph (%s)", hipGetErrorString(ended));
        return VXHIP_EXECUTION_FAILED;
    }
    if (!out) {  // the caller abandons the recording
        (void)hipGraphDestroy(graph);
        return VXHIP_OK;
    }
    hipGraphExec_t executable = nullptr;
    const hipError_t made = hipGraphInstantiate(&executable, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (made != hipSuccess || !executable) {
        (void)hipGetLastError();
        set_error("context_end_recording: the recorded launches could not be instantiated (%s)", hipGetErrorString(made));
        return VXHIP_EXECUTION_FAILED;
    }
    VxHipReplay* replay = new (std::nothrow) VxHipReplay();
    if (!replay) {
        (void)hipGraphExecDestroy(executable);
        return VXHIP_OUT_OF_MEMORY;
    }
    replay->device = ctx->device;
    replay->executable = executable;
    *out = replay;
    return VXHIP_OK;
}

VxHipStatus vxhip_replay_launch(VxHipContext* ctx, const VxHipReplay* replay) {
    if (!ctx || !replay || !replay->executable || ctx->recording) {
        set_error("replay_launch: null handle, or the context is recording");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!same_device(ctx, replay->device, "replay_launch") || !use_device(ctx->device)) return VXHIP_INVALID_ARGUMENT;
    VXHIP_TRY(hipGraphLaunch(replay->executable, ctx->stream));
    return VXHIP_OK;
}

void vxhip_replay_destroy(VxHipReplay* replay) {
    if (!replay) return;
    (void)hipSetDevice(replay->device);
    if (replay->executable) (void)hipGraphExecDestroy(replay->executable);
    delete replay;
}

const char* vxhip_context_last_variant(const VxHipContext* ctx) { return ctx ? ctx->last_variant : ""; }

VxHipStatus vxhip_context_fault_flags(VxHipContext* ctx, uint32_t* flags) {
    if (!ctx || !flags || !not_recording(ctx, "context_fault_flags")) return VXHIP_INVALID_ARGUMENT;
    VXHIP_TRY(hipMemcpyAsync(flags, ctx->fault_dev, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    VXHIP_TRY(hipStreamSynchronize(ctx->stream));
    return VXHIP_OK;
}

VxHipStatus vxhip_context_clear_fault_flags(VxHipContext* ctx) {
    if (!ctx) return VXHIP_INVALID_ARGUMENT;
    if (!use_device(ctx->device)) return VXHIP_BACKEND_UNAVAILABLE;
    // a fill kernel on the context's stream: ordered after the launches that may still raise bits
    return launch_fill_u32(ctx->stream, ctx->fault_dev, 1u, 0u);
}

VxHipStatus vxhip_context_reserve_scratch(VxHipContext* ctx, size_t bytes) {
    if (!ctx) return VXHIP_INVALID_ARGUMENT;
    if (!use_device(ctx->device)) return VXHIP_BACKEND_UNAVAILABLE;
    return ensure_scratch(ctx, bytes);
}

VxHipStatus vxhip_context_set_activation_layout(VxHipContext* ctx, uint32_t layout) {
    if (!ctx || layout > VXHIP_ACTIVATIONS_OPERAND32) return VXHIP_INVALID_ARGUMENT;
    ctx->activation_layout = layout;
    return VXHIP_OK;
}

size_t vxhip_context_prepared_bytes(const VxHipContext* ctx, uint32_t rows, uint32_t k) {
    if (ctx && ctx->activation_layout == VXHIP_ACTIVATIONS_OPERAND32 && rows <= kOperandOrderRows)
        return (size_t)kOperandOrderRows * ((k + 15u) / 16u * 16u);
    return (size_t)rows * k;
}

VxHipStatus vxhip_device_malloc(size_t bytes, void** out) {
    if (!out) return VXHIP_INVALID_ARGUMENT;
    *out = nullptr;
    VXHIP_TRY(hipMalloc(out, bytes ? bytes : 1));
    return VXHIP_OK;
}

void vxhip_device_free(void* p) {
    if (p) (void)hipFree(p);
}

VxHipStatus vxhip_memcpy_to_device(VxHipContext* ctx, void* dst, const void* src, size_t bytes) {
    if (!ctx || (bytes && (!dst || !src)) || !not_recording(ctx, "memcpy_to_device")) return VXHIP_INVALID_ARGUMENT;
    if (!bytes) return VXHIP_OK;
    VXHIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    VXHIP_TRY(hipStreamSynchronize(ctx->stream));
    return VXHIP_OK;
}

VxHipStatus vxhip_memcpy_to_host(VxHipContext* ctx, void* dst, const void* src, size_t bytes) {
    if (!ctx || (bytes && (!dst || !src)) || !not_recording(ctx, "memcpy_to_host")) return VXHIP_INVALID_ARGUMENT;
    if (!bytes) return VXHIP_OK;
    VXHIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    VXHIP_TRY(hipStreamSynchronize(ctx->stream));
    return VXHIP_OK;
}

// ---- QLinear ------------------------------------------------------------------

void vxhip_qlinear_destroy(VxHipQLinear* lin) {
    if (!lin) return;
    (void)hipSetDevice(lin->device);
    (void)hipDeviceSynchronize();
    if (lin->w.data) (void)hipFree(lin->w.data);
    if (lin->scales) (void)hipFree(lin->scales);
    if (lin->zero_points) (void)hipFree(lin->zero_points);
    if (lin->bias) (void)hipFree(lin->bias);
    if (lin->weight_sums) (void)hipFree(lin->weight_sums);
    delete lin;
}

uint64_t vxhip_qlinear_resident_bytes(const VxHipQLinear* lin) { return lin ? lin->resident : 0; }

VxHipStatus vxhip_qlinear_create(const void* weight, const float* weight_scales,
                                 const int32_t* weight_zero_points, const int32_t* bias,
                                 uint32_t d_in, uint32_t d_out, uint32_t weight_dtype,
                                 VxHipQLinear** out) {
    if (!out) return VXHIP_INVALID_ARGUMENT;
    *out = nullptr;
    if (!weight || !weight_scales || !weight_zero_points || !d_in || !d_out ||
        !byte_dtype(weight_dtype)) {
        set_error("qlinear_create: null tensor, zero extent or non-byte weight dtype");
        return VXHIP_INVALID_ARGUMENT;
    }
    if ((uint64_t)d_in * d_out > (uint64_t)1 << 40) return VXHIP_INVALID_ARGUMENT;
    int device = 0;
    VXHIP_TRY(hipGetDevice(&device));
    const bool flip = weight_dtype == VXHIP_DTYPE_U8;
    float smin = INFINITY, smax = 0.f;
    bool any_zp = false;
    int64_t bias_abs = 0;
    const uint32_t n_pad = ((d_out + 31u) / 32u + kPanelPad - 1) / kPanelPad * kPanelPad * 32u;
    std::vector<int32_t> zps(n_pad, 0), hbias(n_pad, 0);
    std::vector<float> hscale(n_pad, 1.0f);
    for (uint32_t i = 0; i < d_out; i++) {
        if (!scale_ok(weight_scales[i]) || !zero_point_ok(weight_zero_points[i], weight_dtype)) {
            set_error("qlinear_create: channel %u has an invalid scale or zero point", i);
            return VXHIP_INVALID_ARGUMENT;
        }
        hscale[i] = weight_scales[i];
        smin = fminf(smin, weight_scales[i]);
        smax = fmaxf(smax, weight_scales[i]);
        zps[i] = weight_zero_points[i] - (flip ? 128 : 0);
        any_zp |= zps[i] != 0;
        if (bias) {
            hbias[i] = bias[i];
            const int64_t b = bias[i] < 0 ? -(int64_t)bias[i] : (int64_t)bias[i];
            if (b > bias_abs) bias_abs = b;
        }
    }
    VxHipQLinear* lin = new (std::nothrow) VxHipQLinear();
    if (!lin) return VXHIP_OUT_OF_MEMORY;
    lin->device = device;
    lin->weight_dtype = weight_dtype;
    lin->any_zero_point = any_zp;
    lin->scale_min = smin;
    lin->scale_max = smax;
    lin->bias_abs_max = bias_abs;
    uint8_t* raw = nullptr;
    int32_t* absmax_dev = nullptr;
    const size_t raw_bytes = (size_t)d_in * d_out;
    VxHipStatus st = VXHIP_OK;
    auto fail = [&](VxHipStatus s) {
        if (raw) (void)hipFree(raw);
        if (absmax_dev) (void)hipFree(absmax_dev);
        vxhip_qlinear_destroy(lin);
        return s;
    };
#define TRY_OR_FAIL(expr)                                        \
    do {                                                         \
        hipError_t e_ = (expr);                                  \
        if (e_ != hipSuccess) return fail(hip_status(e_, #expr)); \
    } while (0)
    TRY_OR_FAIL(hipMalloc((void**)&raw, raw_bytes));
    TRY_OR_FAIL(hipMalloc((void**)&absmax_dev, 256));
    TRY_OR_FAIL(hipMalloc((void**)&lin->scales, n_pad * sizeof(float)));
    TRY_OR_FAIL(hipMalloc((void**)&lin->zero_points, n_pad * sizeof(int32_t)));
    TRY_OR_FAIL(hipMalloc((void**)&lin->bias, n_pad * sizeof(int32_t)));
    TRY_OR_FAIL(hipMalloc((void**)&lin->weight_sums, n_pad * sizeof(int32_t)));
    TRY_OR_FAIL(hipMemcpy(raw, weight, raw_bytes, hipMemcpyHostToDevice));
    TRY_OR_FAIL(hipMemcpy(lin->scales, hscale.data(), n_pad * sizeof(float), hipMemcpyHostToDevice));
    TRY_OR_FAIL(hipMemcpy(lin->zero_points, zps.data(), n_pad * sizeof(int32_t), hipMemcpyHostToDevice));
    TRY_OR_FAIL(hipMemcpy(lin->bias, hbias.data(), n_pad * sizeof(int32_t), hipMemcpyHostToDevice));
    TRY_OR_FAIL(hipMemset(lin->weight_sums, 0, n_pad * sizeof(int32_t)));
    st = weight_row_stats(nullptr, raw, d_in, d_out, d_in, flip, lin->zero_points, lin->weight_sums,
                          absmax_dev);
    if (st != VXHIP_OK) return fail(st);
    st = pack_weight(nullptr, raw, d_in, d_out, d_in, flip, &lin->w);
    if (st != VXHIP_OK) return fail(st);
    int32_t absmax = 0;
    TRY_OR_FAIL(hipMemcpy(&absmax, absmax_dev, sizeof absmax, hipMemcpyDeviceToHost));
    TRY_OR_FAIL(hipDeviceSynchronize());
#undef TRY_OR_FAIL
    lin->weight_abs_max = absmax;
    (void)hipFree(raw);
    (void)hipFree(absmax_dev);
    lin->resident = lin->w.bytes() + (uint64_t)n_pad * 16u;
    *out = lin;
    return VXHIP_OK;
}

// Mismatch counters of the short divisions by `divisor`, proved on the context's stream the
// first time the divisor is seen (a few microseconds; later calls find the slot).  The kernels
// that read them are ordered after the proof by the stream.  Null if the launch failed.
static const uint32_t* division_proof(VxHipContext* ctx, float divisor, float recip) {
    uint32_t bits;
    memcpy(&bits, &divisor, sizeof bits);
    for (int i = 0; i < ctx->div_used; i++)
        if (ctx->div_bits[i] == bits) return ctx->div_proof_dev + 2 * i;
    // (a proof recorded rather than run would not have happened for the calls that find its slot later:
    // a divisor first seen while recording stays unproved, and its launches divide the long way)
    if (ctx->recording) return nullptr;
    const int slot = ctx->div_next;
    uint32_t* counters = ctx->div_proof_dev + 2 * slot;
    ctx->div_bits[slot] = 0;  // +0.0 is never a divisor: the slot matches nothing until the launch succeeded
    if (launch_division_proof(ctx->stream, divisor, recip, counters) != VXHIP_OK) return nullptr;
    ctx->div_bits[slot] = bits;
    ctx->div_next = (slot + 1) % VxHipContext::kDivisorSlots;
    if (ctx->div_used < VxHipContext::kDivisorSlots) ctx->div_used++;
    return counters;
}

// Everything a QLinear call must satisfy before anything is launched; shared by the forward
// entry points and by vxhip_qlinear_admits.
static bool qlinear_admission(const VxHipQLinear* lin, bool per_row, float input_scale, int32_t input_zp,
                              float output_scale, int32_t output_zp, uint32_t input_dtype,
                              uint32_t output_dtype) {
    if (!byte_dtype(input_dtype) || !byte_dtype(output_dtype) || !scale_ok(output_scale) ||
        !zero_point_ok(input_zp, input_dtype) || !zero_point_ok(output_zp, output_dtype)) {
        set_error("qlinear_forward: invalid dtype, scale or zero point");
        return false;
    }
    const uint32_t k = lin->w.k;
    if (!per_row) {
        // product and quotient are monotone in s_w, so the extremes decide for every channel
        if (!scale_ok(input_scale) || !multiplier_ok(input_scale, lin->scale_min, output_scale) ||
            !multiplier_ok(input_scale, lin->scale_max, output_scale)) {
            set_error("qlinear_forward: a requantization multiplier is not a positive finite f32");
            return false;
        }
    }
    // int32 admission: no partial sum can leave int32 when
    //   K * max|x - zx| * max|w - zw| + max|bias| <= INT32_MAX
    // (the proof the reference's vector route demands, native/src/kernels/qlinear_w8a8_x86.c:80,92-99)
    const int64_t lo = input_dtype == VXHIP_DTYPE_I8 ? -128 : 0, hi = input_dtype == VXHIP_DTYPE_I8 ? 127 : 255;
    const int64_t xmax = llabs(lo - input_zp) > llabs(hi - input_zp) ? llabs(lo - input_zp) : llabs(hi - input_zp);
    if ((int64_t)k * xmax * lin->weight_abs_max + lin->bias_abs_max > (int64_t)INT32_MAX) {
        set_error("qlinear_forward: int32 accumulator bound not provable for K=%u", k);
        return false;
    }
    return true;
}

static bool per_row_ok(bool per_row, const float* row_scales_dev) {
    if (per_row && !row_scales_dev) {
        set_error("qlinear_forward_rowscale: row scales are required");
        return false;
    }
    return true;
}

int vxhip_qlinear_admits(const VxHipQLinear* lin, float input_scale, int32_t input_zp, float output_scale,
                         int32_t output_zp, uint32_t input_dtype, uint32_t output_dtype) {
    if (!lin) {
        set_error("qlinear_admits: null handle");
        return 0;
    }
    return qlinear_admission(lin, false, input_scale, input_zp, output_scale, output_zp, input_dtype, output_dtype) ? 1 : 0;
}

// Shared by the per-tensor and the per-row entry points.
static int qlinear_run(VxHipContext* ctx, const VxHipQLinear* lin, const void* input_dev,
                       const float* row_scales_dev, const float* bias_f32_dev, void* output_dev,
                       int32_t* acc_dev, uint32_t rows, float input_scale, int32_t input_zp,
                       float output_scale, int32_t output_zp, uint32_t input_dtype,
                       uint32_t output_dtype, bool per_row, float* dq_dev = nullptr, float dq_scale = 0.0f,
                       int32_t dq_zp = 0, const float* input_f32_dev = nullptr) {
    // input_f32_dev (instead of input_dev): the rows before the QuantizeLinear that feeds this QLinear
    if (!ctx || !lin || (!input_dev && !input_f32_dev) || (!output_dev && !acc_dev && !dq_dev) || !rows) {
        set_error("qlinear_forward: null handle/tensor or zero rows");
        return 0;
    }
    if (!per_row_ok(per_row, row_scales_dev) ||
        !qlinear_admission(lin, per_row, input_scale, input_zp, output_scale, output_zp, input_dtype, output_dtype))
        return 0;
    const uint32_t k = lin->w.k, n = lin->w.n;
    if (!same_device(ctx, lin->device, "qlinear_forward") || !use_device(ctx->device)) return 0;

    const bool flip = input_dtype == VXHIP_DTYPE_U8;
    const char* force = forced_variant();
    // One or two f32 rows and weights without zero points: the streaming kernel quantizes the rows
    // itself (gemv_stream.hip, PREP) and the QuantizeLinear costs no launch.  Otherwise, or when no such
    // kernel takes the shape, it runs first, into the scratch.
    bool quantize_inside = input_f32_dev && !per_row && rows <= kMaxPrepRows && !lin->any_zero_point && !acc_dev &&
                           !(force && (!strstr(force, "gemv") || strstr(force, "noprep")));
    if (input_f32_dev && (uint64_t)rows * k > UINT32_MAX) {
        set_error("qlinear_forward: rows * k beyond 2^32 elements");
        return 0;
    }
    // bytes are staged when they need flipping, padding to whole 16-byte chunks, or alignment
    const bool stage = flip || (k % 16u) != 0u || (!input_f32_dev && ((uintptr_t)input_dev % 16u) != 0u);
    const uint32_t ld = stage ? (k + 15u) / 16u * 16u : k;
    const uint32_t n_pad = lin->w.panels * 32u;
    Carver sizes{nullptr};
    sizes.take<int32_t>(rows);
    sizes.take<int8_t>(stage ? (size_t)rows * ld : 0);
    sizes.take<int8_t>(input_f32_dev ? (size_t)rows * k : 0);
    if (ensure_scratch(ctx, sizes.off + 256u) != VXHIP_OK) return 0;
    Carver c{(char*)ctx->scratch};
    int32_t* rowsum = c.take<int32_t>(rows);
    int8_t* staged = c.take<int8_t>(stage ? (size_t)rows * ld : 0);
    int8_t* quantized = c.take<int8_t>(input_f32_dev ? (size_t)rows * k : 0);

    LinearArgs a{};
    a.mode = per_row ? Epilogue::RequantRow : Epilogue::RequantTensor;
    a.rows = rows;
    a.n = n;
    a.k = k;
    a.w = lin->w.data;
    a.panels = lin->w.panels;
    a.ksteps = lin->w.ksteps;
    a.weight_bits = 8u;
    a.wscale = lin->scales;
    a.bias_i32 = lin->bias;
    a.wsum = lin->weight_sums;
    a.zw = lin->any_zero_point ? lin->zero_points : nullptr;
    a.rowsum = rowsum;
    a.row_scale = row_scales_dev;
    a.bias_row = bias_f32_dev;
    a.input_scale = input_scale;
    a.input_zp = input_zp - (flip ? 128 : 0);
    a.output_scale = output_scale;
    // 1/s in double is within 2^-53 of the true quotient, which can never sit that close to
    // an f32 rounding boundary, so the second rounding gives the correctly rounded f32
    a.output_scale_recip = (float)(1.0 / (double)output_scale);
    a.div_proof = per_row ? division_proof(ctx, output_scale, a.output_scale_recip) : nullptr;
    a.int_bias_zero = lin->bias_abs_max == 0;
    a.wscale_min = lin->scale_min;
    a.wscale_max = lin->scale_max;
    a.out_zp = output_zp;
    a.out_lo = output_dtype == VXHIP_DTYPE_I8 ? -128 : 0;
    a.out_hi = output_dtype == VXHIP_DTYPE_I8 ? 127 : 255;
    a.n_pad = n_pad;
    a.y = output_dev;
    a.acc_out = acc_dev;
    a.dq_out = dq_dev;
    a.dq_scale = dq_scale;
    a.dq_zp = dq_zp;
    a.fault = ctx->fault_dev;

    const char* id = nullptr;
    if (quantize_inside) {
        a.x_f32 = input_f32_dev;
        a.x_f32_unsigned = flip ? 1u : 0u;
        a.ldx = k;
        id = launch_gemv_stream(ctx->stream, a, ctx->cu_count, force);
        a.x_f32 = nullptr;
    }
    // Unsigned bytes in whole aligned 16-byte chunks, few rows, no row sums wanted: the streaming kernel
    // flips the top bits itself and the staging launch is saved.
    if (!id && !input_f32_dev && flip && rows <= kMaxGemvRows && (k % 16u) == 0u && ((uintptr_t)input_dev % 16u) == 0u &&
        !lin->any_zero_point && !(force && !strstr(force, "gemv"))) {
        a.x = (const int8_t*)input_dev;
        a.ldx = k;
        a.x_flip_mask = 0x80808080u;
        id = launch_gemv_stream(ctx->stream, a, ctx->cu_count, force);
        a.x_flip_mask = 0u;
    }
    // ... and so do the large-tile GEMM kernels (gemm_k64.hip, FLIP) for more rows
    if (!id && !input_f32_dev && flip && rows > kMaxGemvRows && (k % 16u) == 0u && ((uintptr_t)input_dev % 16u) == 0u &&
        !lin->any_zero_point && !per_row && !(force && strstr(force, "gemv"))) {
        a.x = (const int8_t*)input_dev;
        a.ldx = k;
        a.x_flip_mask = 0x80808080u;
        id = launch_gemm_mfma(ctx->stream, a, ctx->cu_count, force);
        a.x_flip_mask = 0u;
    }
    if (!id) {
        if (input_f32_dev) {
            if (launch_quantize(ctx->stream, input_f32_dev, rows * k, quantized, input_scale, input_zp,
                                input_dtype == VXHIP_DTYPE_I8) != VXHIP_OK)
                return 0;
            input_dev = quantized;
        }
        if (stage || lin->any_zero_point) {
            if (launch_stage_activations(ctx->stream, input_dev, rows, k, flip, stage ? staged : nullptr, ld,
                                         lin->any_zero_point ? rowsum : nullptr) != VXHIP_OK)
                return 0;
        }
        a.x = stage ? staged : (const int8_t*)input_dev;
        a.ldx = ld;
        id = run_linear(ctx, a);
    }
    if (!id) {
        set_error("qlinear_forward: no kernel variant accepts rows=%u k=%u n=%u", rows, k, n);
        return 0;
    }
    set_last_variant(ctx, id);
    return 1;
}

int vxhip_qlinear_forward(VxHipContext* ctx, const VxHipQLinear* lin, const void* input_dev,
                          void* output_dev, int32_t* acc_dev, uint32_t rows, float input_scale,
                          int32_t input_zp, float output_scale, int32_t output_zp,
                          uint32_t input_dtype, uint32_t output_dtype) {
    return qlinear_run(ctx, lin, input_dev, nullptr, nullptr, output_dev, acc_dev, rows, input_scale,
                       input_zp, output_scale, output_zp, input_dtype, output_dtype, false);
}

int vxhip_qlinear_forward_dequantized(VxHipContext* ctx, const VxHipQLinear* lin, const void* input_dev,
                                      float* output_f32_dev, void* output_dev, uint32_t rows, float input_scale,
                                      int32_t input_zp, float output_scale, int32_t output_zp, uint32_t input_dtype,
                                      uint32_t output_dtype, float dequant_scale, int32_t dequant_zp) {
    if (!output_f32_dev) {
        set_error("qlinear_forward_dequantized: null f32 output");
        return 0;
    }
    // the parameters a typed DequantizeLinear is given (native/src/kernels/w8a8_affine.h:46-65): a finite positive scale and a
    // zero point inside the byte type it reads; then q - zero_point is exact in f32 as well
    if (!byte_dtype(output_dtype) || !scale_ok(dequant_scale) || !zero_point_ok(dequant_zp, output_dtype)) {
        set_error("qlinear_forward_dequantized: dequantization scale %g / zero point %d not admissible", (double)dequant_scale,
                  dequant_zp);
        return 0;
    }
    return qlinear_run(ctx, lin, input_dev, nullptr, nullptr, output_dev, nullptr, rows, input_scale, input_zp,
                       output_scale, output_zp, input_dtype, output_dtype, false, output_f32_dev, dequant_scale,
                       dequant_zp);
}

int vxhip_qlinear_forward_f32(VxHipContext* ctx, const VxHipQLinear* lin, const float* input_f32_dev,
                              float* output_f32_dev, void* output_dev, uint32_t rows, float input_scale,
                              int32_t input_zp, float output_scale, int32_t output_zp, uint32_t input_dtype,
                              uint32_t output_dtype, float dequant_scale, int32_t dequant_zp) {
    if (!input_f32_dev || (!output_f32_dev && !output_dev)) {
        set_error("qlinear_forward_f32: null input, or neither output");
        return 0;
    }
    if (output_f32_dev &&
        (!byte_dtype(output_dtype) || !scale_ok(dequant_scale) || !zero_point_ok(dequant_zp, output_dtype))) {
        set_error("qlinear_forward_f32: dequantization scale %g / zero point %d not admissible", (double)dequant_scale,
                  dequant_zp);
        return 0;
    }
    // (the QuantizeLinear's own parameters are the QLinear's input scale and zero point, which its admission checks)
    return qlinear_run(ctx, lin, nullptr, nullptr, nullptr, output_dev, nullptr, rows, input_scale, input_zp,
                       output_scale, output_zp, input_dtype, output_dtype, false, output_f32_dev, dequant_scale,
                       dequant_zp, input_f32_dev);
}

int vxhip_qlinear_forward_rowscale(VxHipContext* ctx, const VxHipQLinear* lin, const int8_t* input_dev,
                                   const float* row_scales_dev, const float* bias_f32_dev,
                                   void* output_dev, int32_t* acc_dev, uint32_t rows,
                                   float output_scale, int32_t output_zp, uint32_t output_dtype) {
    return qlinear_run(ctx, lin, input_dev, row_scales_dev, bias_f32_dev, output_dev, acc_dev, rows,
                       1.0f, 0, output_scale, output_zp, VXHIP_DTYPE_I8, output_dtype, true);
}

int vxhip_qlinear_i8u8(const void* input, const void* weight, const float* weight_scales,
                       const int32_t* weight_zero_points, const int32_t* bias, void* output,
                       uint32_t rows, uint32_t d_in, uint32_t d_out, float input_scale,
                       int32_t input_zp, float output_scale, int32_t output_zp, uint32_t input_dtype,
                       uint32_t weight_dtype, uint32_t output_dtype) {
    // the reference declines a null bias (portable_inference_kernels.inc:978)
    if (!input || !weight || !bias || !weight_scales || !weight_zero_points || !output || !rows ||
        !d_in || !d_out || !byte_dtype(input_dtype) || !byte_dtype(weight_dtype) ||
        !byte_dtype(output_dtype)) {
        set_error("qlinear_i8u8: null tensor, zero extent or non-byte dtype");
        return 0;
    }
    VxHipContext* ctx = default_context();
    if (!ctx) return 0;
    ResidentKey key{};
    key.pointers[0] = weight;
    key.pointers[1] = weight_scales;
    key.pointers[2] = weight_zero_points;
    key.pointers[3] = bias;
    key.extents[0] = d_in;
    key.extents[1] = d_out;
    key.extents[2] = weight_dtype;
    key.extents[3] = 1u;  // a QLinear
    key.fingerprint = fingerprint(0xcbf29ce484222325ull, weight, (size_t)d_in * d_out);
    key.fingerprint = fingerprint(key.fingerprint, weight_scales, (size_t)d_out * 4u);
    key.fingerprint = fingerprint(key.fingerprint, weight_zero_points, (size_t)d_out * 4u);
    key.fingerprint = fingerprint(key.fingerprint, bias, (size_t)d_out * 4u);
    std::shared_ptr<ResidentWeights> held = resident_find(key);
    if (!held) {
        held = std::make_shared<ResidentWeights>();
        if (vxhip_qlinear_create(weight, weight_scales, weight_zero_points, bias, d_in, d_out, weight_dtype,
                                 &held->qlinear) != VXHIP_OK)
            return 0;
        resident_insert(key, held, (size_t)vxhip_qlinear_resident_bytes(held->qlinear));
    }
    const size_t in_bytes = (size_t)rows * d_in, out_bytes = (size_t)rows * d_out;
    int ok = 0;
    if (io_staging(ctx, in_bytes, out_bytes) && vxhip_memcpy_to_device(ctx, ctx->io_in, input, in_bytes) == VXHIP_OK) {
        ok = vxhip_qlinear_forward(ctx, held->qlinear, ctx->io_in, ctx->io_out, nullptr, rows, input_scale, input_zp,
                                   output_scale, output_zp, input_dtype, output_dtype);
        // the caller's output is written only after the whole launch succeeded
        if (ok && vxhip_memcpy_to_host(ctx, output, ctx->io_out, out_bytes) != VXHIP_OK) ok = 0;
    }
    (void)hipStreamSynchronize(ctx->stream);
    return ok;
}

// ---- PackedLinear ---------------------------------------------------------------

void vxhip_packed_linear_destroy(VxHipPackedLinear* pl) {
    if (!pl) return;
    (void)hipSetDevice(pl->device);
    (void)hipDeviceSynchronize();
    if (pl->w.data) (void)hipFree(pl->w.data);
    if (pl->scales_t) (void)hipFree(pl->scales_t);
    if (pl->bias) (void)hipFree(pl->bias);
    delete pl;
}

uint64_t vxhip_packed_linear_resident_bytes(const VxHipPackedLinear* pl) { return pl ? pl->resident : 0; }

VxHipStatus vxhip_packed_linear_create(const uint32_t* packed_words, const float* scales,
                                       const float* bias, uint32_t k, uint32_t n, uint32_t group_size,
                                       uint32_t weight_bits, VxHipPackedLinear** out) {
    if (!out) return VXHIP_INVALID_ARGUMENT;
    *out = nullptr;
    if (!packed_words || !scales || !k || !n) {
        set_error("packed_linear_create: null tensor or zero extent");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (weight_bits != 8u && weight_bits != 4u && weight_bits != 3u && weight_bits != 2u) {
        set_error("packed_linear_create: weight_bits must be 2, 3, 4 or 8 (got %u)", weight_bits);
        return VXHIP_BACKEND_UNSUPPORTED;
    }
    if (group_size != 32u && group_size != 64u && group_size != 128u && group_size != 256u) {
        set_error("packed_linear_create: group size %u is not 32/64/128/256", group_size);
        return VXHIP_INVALID_ARGUMENT;
    }
    if ((uint64_t)k * n > (uint64_t)1 << 40) return VXHIP_INVALID_ARGUMENT;
    int device = 0;
    VXHIP_TRY(hipGetDevice(&device));
    // vx_packed_words (packed_linear_ops.inc:246-248)
    const uint32_t words = (k / 32u) * weight_bits + ((k % 32u) * weight_bits + 31u) / 32u;
    const uint32_t groups = (k + group_size - 1u) / group_size;
    const uint32_t n_pad = ((n + 31u) / 32u + kPanelPad - 1) / kPanelPad * kPanelPad * 32u;
    std::vector<float> st((size_t)groups * n_pad, 1.0f), hb(n_pad, 0.0f);
    bool uniform_scales = true;
    for (uint32_t o = 0; o < n; o++) {
        for (uint32_t g = 0; g < groups; g++) {
            const float s = scales[(size_t)o * groups + g];
            if (memcmp(&s, &scales[(size_t)o * groups], sizeof s) != 0) uniform_scales = false;
            if (!isfinite(s)) {
                set_error("packed_linear_create: scale [%u][%u] is not finite", o, g);
                return VXHIP_INVALID_ARGUMENT;
            }
            st[(size_t)g * n_pad + o] = s;
        }
        if (bias) hb[o] = bias[o];
    }
    VxHipPackedLinear* pl = new (std::nothrow) VxHipPackedLinear();
    if (!pl) return VXHIP_OUT_OF_MEMORY;
    pl->device = device;
    pl->group_size = group_size;
    pl->groups = groups;
    pl->uniform_scales = uniform_scales;
    uint8_t* raw = nullptr;
    const size_t raw_bytes = (size_t)n * words * 4u;
    auto fail = [&](VxHipStatus s) {
        if (raw) (void)hipFree(raw);
        vxhip_packed_linear_destroy(pl);
        return s;
    };
#define TRY_OR_FAIL(expr)                                        \
    do {                                                         \
        hipError_t e_ = (expr);                                  \
        if (e_ != hipSuccess) return fail(hip_status(e_, #expr)); \
    } while (0)
    TRY_OR_FAIL(hipMalloc((void**)&raw, raw_bytes));
    TRY_OR_FAIL(hipMalloc((void**)&pl->scales_t, st.size() * sizeof(float)));
    TRY_OR_FAIL(hipMalloc((void**)&pl->bias, n_pad * sizeof(float)));
    TRY_OR_FAIL(hipMemcpy(raw, packed_words, raw_bytes, hipMemcpyHostToDevice));
    TRY_OR_FAIL(hipMemcpy(pl->scales_t, st.data(), st.size() * sizeof(float), hipMemcpyHostToDevice));
    TRY_OR_FAIL(hipMemcpy(pl->bias, hb.data(), n_pad * sizeof(float), hipMemcpyHostToDevice));
    // offset-binary codes: value = code - 128, i.e. the byte with its top bit flipped
    VxHipStatus s2 = weight_bits != 8u
                         ? pack_weight_nibbles(nullptr, (const uint32_t*)raw, words, n, k, weight_bits, &pl->w)
                         : pack_weight(nullptr, raw, (size_t)words * 4u, n, k, true, &pl->w);
    if (s2 != VXHIP_OK) return fail(s2);
    TRY_OR_FAIL(hipDeviceSynchronize());
#undef TRY_OR_FAIL
    (void)hipFree(raw);
    pl->resident = pl->w.bytes() + st.size() * sizeof(float) + n_pad * sizeof(float);
    *out = pl;
    return VXHIP_OK;
}

VxHipStatus vxhip_packed_prepare_i8(VxHipContext* ctx, const float* input_dev, uint32_t rows, uint32_t k,
                                    int8_t* prepared_dev, float* row_scales_dev) {
    if (!ctx || !input_dev || !prepared_dev || !row_scales_dev || !k) return VXHIP_INVALID_ARGUMENT;
    if (!rows) return VXHIP_OK;
    if (!use_device(ctx->device)) return VXHIP_BACKEND_UNAVAILABLE;
    set_last_variant(ctx, "hip.packed-linear.prepare-i8");
    const bool operand_order = ctx->activation_layout == VXHIP_ACTIVATIONS_OPERAND32 && rows <= kOperandOrderRows;
    return launch_prepare_i8(ctx->stream, input_dev, rows, k, prepared_dev,
                             operand_order ? ActivationLayout{(k + 15u) / 16u * 16u, 1u} : ActivationLayout{k, 0u},
                             row_scales_dev);
}

// operand_order: a8 is in operand order (rows <= 32), which only the GEMV reads; -2 then says that
// no GEMV takes the shape and the caller has to come back with row-major activations.
static int packed_run_a8(VxHipContext* ctx, const VxHipPackedLinear* pl, const int8_t* a8, uint32_t lda,
                         bool operand_order, const float* row_scales, float* y, int32_t* acc,
                         const int32_t* zeros, uint32_t rows) {
    LinearArgs a{};
    a.mode = Epilogue::DequantF32;
    a.x = a8;
    a.ldx = lda;
    a.x_operand_order = operand_order ? 1u : 0u;
    a.rows = rows;
    a.n = pl->w.n;
    a.k = pl->w.k;
    a.w = pl->w.data;
    a.panels = pl->w.panels;
    a.ksteps = pl->w.ksteps;
    a.weight_bits = pl->w.bits;
    a.row_scale = row_scales;
    a.scales_t = pl->scales_t;
    a.bias_f32 = pl->bias;
    a.group_size = pl->group_size;
    a.groups = pl->groups;
    a.uniform_group_scales = pl->uniform_scales;
    a.n_pad = pl->w.panels * 32u;
    a.y = y;
    a.fault = ctx->fault_dev;
    const char* id = nullptr;
    if (y) {
        id = run_linear(ctx, a);
        if (!id) return operand_order ? -2 : -1;
    }
    if (acc) {
        // exact full-K int32 sums: the same kernels in requantizing mode with the byte output
        // off; unit scales and the zero array stand in for the unused per-channel inputs
        LinearArgs b = a;
        b.mode = Epilogue::RequantTensor;
        b.y = nullptr;
        b.acc_out = acc;
        b.wscale = pl->bias;
        b.bias_i32 = zeros;
        b.wsum = zeros;
        b.zw = nullptr;
        b.input_scale = 1.0f;
        b.input_zp = 0;
        b.output_scale = 1.0f;
        b.output_scale_recip = 1.0f;
        b.wscale_min = b.wscale_max = 1.0f;
        b.fault = ctx->fault_dev + 1;  // multipliers are meaningless here: keep them off the real word
        b.out_lo = -128;
        b.out_hi = 127;
        const char* id2 = run_linear(ctx, b);
        if (!id2) return operand_order && !y ? -2 : -1;
        if (!id) id = id2;
    }
    set_last_variant(ctx, id);
    return 0;
}

int vxhip_packed_linear_forward_a8(VxHipContext* ctx, const VxHipPackedLinear* pl,
                                   const int8_t* activation_dev, const float* row_scales_dev,
                                   float* output_dev, int32_t* acc_dev, uint32_t rows) {
    if (!ctx || !pl || !activation_dev || !row_scales_dev || (!output_dev && !acc_dev)) {
        set_error("packed_linear_forward_a8: null handle or tensor");
        return -1;
    }
    if (!rows) return 0;
    if (!same_device(ctx, pl->device, "packed_linear_forward_a8") || !use_device(ctx->device)) return -1;
    const uint32_t k = pl->w.k, n_pad = pl->w.panels * 32u;
    if (acc_dev && pl->w.bits != 8u) {
        set_error("packed_linear_forward_a8: the int32 sums are produced for 8-bit weights only");
        return -1;
    }
    if (acc_dev && (uint64_t)k * 127u * 128u > (uint64_t)INT32_MAX) {
        set_error("packed_linear_forward_a8: full-K int32 sums are not provable for K=%u", k);
        return -1;
    }
    const bool operand_order = ctx->activation_layout == VXHIP_ACTIVATIONS_OPERAND32 && rows <= kOperandOrderRows;
    if (operand_order && ((uintptr_t)activation_dev % 16u) != 0u) {
        set_error("packed_linear_forward_a8: operand-order activations must be 16-byte aligned");
        return -1;
    }
    // row-major rows are used in place when they are aligned whole chunks; operand order is
    // used in place by the GEMV and copied out to rows only if the call ends up on the GEMM
    const bool stage = operand_order || (k % 16u) != 0u || ((uintptr_t)activation_dev % 16u) != 0u;
    const uint32_t ld = stage ? (k + 15u) / 16u * 16u : k;
    Carver sizes{nullptr};
    sizes.take<int32_t>(acc_dev ? n_pad : 0);
    sizes.take<int8_t>(stage ? (size_t)rows * ld : 0);
    if (ensure_scratch(ctx, sizes.off + 256u) != VXHIP_OK) return -1;
    Carver c{(char*)ctx->scratch};
    int32_t* zeros = c.take<int32_t>(acc_dev ? n_pad : 0);
    int8_t* staged = c.take<int8_t>(stage ? (size_t)rows * ld : 0);
    // a fill kernel rather than a memset node, so the call stays graph-capturable
    if (acc_dev && launch_fill_u32(ctx->stream, (uint32_t*)zeros, n_pad, 0u) != VXHIP_OK) return -1;
    if (operand_order) {
        const int st = packed_run_a8(ctx, pl, activation_dev, ld, true, row_scales_dev, output_dev, acc_dev, zeros, rows);
        if (st != -2) return st;
        if (launch_unblock_activations(ctx->stream, activation_dev, rows, k, staged, ld) != VXHIP_OK) return -1;
        return packed_run_a8(ctx, pl, staged, ld, false, row_scales_dev, output_dev, acc_dev, zeros, rows);
    }
    if (stage && launch_stage_activations(ctx->stream, activation_dev, rows, k, false, staged, ld, nullptr) !=
                     VXHIP_OK)
        return -1;
    return packed_run_a8(ctx, pl, stage ? staged : activation_dev, ld, false, row_scales_dev, output_dev, acc_dev,
                         zeros, rows);
}

// Few f32 rows: one launch, the GEMV preparing the rows itself (gemv_stream.hip, PREP).  0: ran; -2: no
// such kernel takes the call (shape, forced variant) and nothing was launched.
struct RowOps {
    const float* gain = nullptr;  // RMSNorm in front of the preparation
    double eps = 0.0;
    bool swiglu = false;          // the rows are [gate | up]
    const float* add_to = nullptr;
};
static int packed_run_f32_rows(VxHipContext* ctx, const VxHipPackedLinear* pl, const float* x, float* y, uint32_t rows,
                               const RowOps& ops = RowOps{}) {
    const char* force = forced_variant();
    if (rows > kMaxPrepRows || (force && (!strstr(force, "gemv") || strstr(force, "noprep")))) return -2;
    LinearArgs a{};
    a.mode = Epilogue::DequantF32;
    a.x_f32 = x;
    a.ldx = ops.swiglu ? 2u * pl->w.k : pl->w.k;
    a.row_gain = ops.gain;
    a.row_eps = ops.eps;
    a.row_swiglu = ops.swiglu ? 1u : 0u;
    a.add_to = ops.add_to;
    a.rows = rows;
    a.n = pl->w.n;
    a.k = pl->w.k;
    a.w = pl->w.data;
    a.panels = pl->w.panels;
    a.ksteps = pl->w.ksteps;
    a.weight_bits = pl->w.bits;
    a.scales_t = pl->scales_t;
    a.bias_f32 = pl->bias;
    a.group_size = pl->group_size;
    a.groups = pl->groups;
    a.uniform_group_scales = pl->uniform_scales;
    a.n_pad = pl->w.panels * 32u;
    a.y = y;
    a.fault = ctx->fault_dev;
    const char* id = launch_gemv_stream(ctx->stream, a, ctx->cu_count, force);
    if (!id) return -2;
    set_last_variant(ctx, id);
    return 0;
}

int vxhip_packed_linear_forward_f32(VxHipContext* ctx, const VxHipPackedLinear* pl, const float* input_dev,
                                    float* output_dev, uint32_t rows) {
    if (!ctx || !pl || !input_dev || !output_dev) {
        set_error("packed_linear_forward_f32: null handle or tensor");
        return -1;
    }
    if (!rows) return 0;
    if (!same_device(ctx, pl->device, "packed_linear_forward_f32") || !use_device(ctx->device)) return -1;
    const uint32_t k = pl->w.k;
    if (packed_run_f32_rows(ctx, pl, input_dev, output_dev, rows) == 0) return 0;
    const uint32_t ld = (k + 15u) / 16u * 16u;
    // the prepared rows never leave this call: up to 32 rows go to the GEMV in its operand order
    const bool operand_order = rows <= kOperandOrderRows;
    const size_t prepared_rows = operand_order ? kOperandOrderRows : rows;
    Carver sizes{nullptr};
    sizes.take<float>(rows);
    sizes.take<int8_t>(prepared_rows * ld);
    if (ensure_scratch(ctx, sizes.off + 256u) != VXHIP_OK) return -1;
    Carver c{(char*)ctx->scratch};
    float* row_scales = c.take<float>(rows);
    int8_t* prepared = c.take<int8_t>(prepared_rows * ld);
    if (launch_prepare_i8(ctx->stream, input_dev, rows, k, prepared, ActivationLayout{ld, operand_order ? 1u : 0u},
                          row_scales) != VXHIP_OK)
        return -1;
    const int st = packed_run_a8(ctx, pl, prepared, ld, operand_order, row_scales, output_dev, nullptr, nullptr, rows);
    if (st != -2) return st;
    // no GEMV takes the shape (or a GEMM tile is forced): once more, as rows, for the GEMM
    if (launch_prepare_i8(ctx->stream, input_dev, rows, k, prepared, ActivationLayout{ld, 0u}, row_scales) != VXHIP_OK)
        return -1;
    return packed_run_a8(ctx, pl, prepared, ld, false, row_scales, output_dev, nullptr, nullptr, rows);
}

int vxhip_packed_linear_forward_fused(VxHipContext* ctx, const VxHipPackedLinear* pl, const float* input_dev,
                                      uint32_t rows, uint32_t row_op, const float* gain_dev, double eps,
                                      const float* add_to_dev, float* output_dev) {
    if (!ctx || !pl || !input_dev || !output_dev || row_op > VXHIP_ROW_OP_SWIGLU ||
        (row_op == VXHIP_ROW_OP_RMSNORM && (!gain_dev || !(eps >= 0.0)))) {
        set_error("packed_linear_forward_fused: null handle or tensor, unknown row operation, or RMSNorm without gain");
        return -1;
    }
    if (!rows) return 1;
    if (!same_device(ctx, pl->device, "packed_linear_forward_fused") || !use_device(ctx->device)) return -1;
    // Every workgroup reads the whole input rows while others already store their channels: an input that
    // overlaps the output (or the residual it is added to, which may itself be the output) would be read
    // half updated.
    {
        const uintptr_t x0 = (uintptr_t)input_dev;
        const uintptr_t x1 = x0 + (size_t)rows * (row_op == VXHIP_ROW_OP_SWIGLU ? 2u : 1u) * pl->w.k * 4u;
        const size_t out_bytes = (size_t)rows * pl->w.n * 4u;
        const uintptr_t y0 = (uintptr_t)output_dev, a0 = (uintptr_t)add_to_dev;
        if ((x0 < y0 + out_bytes && y0 < x1) || (add_to_dev && x0 < a0 + out_bytes && a0 < x1)) {
            set_error("packed_linear_forward_fused: the input rows overlap the output or the residual");
            return -1;
        }
    }
    RowOps ops;
    ops.gain = row_op == VXHIP_ROW_OP_RMSNORM ? gain_dev : nullptr;
    ops.eps = eps;
    ops.swiglu = row_op == VXHIP_ROW_OP_SWIGLU;
    ops.add_to = add_to_dev;
    return packed_run_f32_rows(ctx, pl, input_dev, output_dev, rows, ops) == 0 ? 1 : 0;
}

int vxhip_packed_linear_fused_takes(VxHipContext* ctx, const VxHipPackedLinear* pl, uint32_t rows, uint32_t row_op,
                                    int with_residual) {
    if (!ctx || !pl || !rows || row_op > VXHIP_ROW_OP_SWIGLU) return 0;
    // the launcher's own decision, with nothing launched: stand-in addresses that are never dereferenced
    static const float stand_in[4] = {0.f, 0.f, 0.f, 0.f};
    static float stand_out[4];
    RowOps ops;
    ops.gain = row_op == VXHIP_ROW_OP_RMSNORM ? stand_in : nullptr;
    ops.eps = 1e-6;
    ops.swiglu = row_op == VXHIP_ROW_OP_SWIGLU;
    ops.add_to = with_residual ? stand_out : nullptr;
    char kept[sizeof ctx->last_variant];
    memcpy(kept, ctx->last_variant, sizeof kept);
    set_gemv_dry_run(true);
    const int st = packed_run_f32_rows(ctx, pl, stand_in, stand_out, rows, ops);
    set_gemv_dry_run(false);
    memcpy(ctx->last_variant, kept, sizeof kept);
    return st == 0 ? 1 : 0;
}

int vxhip_packed_linear_forward_f32_noalloc(VxHipContext* ctx, const VxHipPackedLinear* pl, const float* input_dev,
                                            float* output_dev, uint32_t rows) {
    if (!ctx || !pl || !input_dev || !output_dev) {
        set_error("packed_linear_forward_f32_noalloc: null handle or tensor");
        return -1;
    }
    if (!rows) return 0;
    if (!same_device(ctx, pl->device, "packed_linear_forward_f32_noalloc") || !use_device(ctx->device)) return -1;
    if (!ctx->no_alloc_scratch) {
        (void)no_alloc_scratch(ctx->device);  // sets the error text of the failed set-up
        return -1;
    }
    if (packed_run_f32_rows(ctx, pl, input_dev, output_dev, rows) == 0) return 0;
    const uint32_t k = pl->w.k;
    const uint32_t ld = (k + 15u) / 16u * 16u;
    const bool operand_order = rows <= kOperandOrderRows;
    const size_t prepared_rows = operand_order ? kOperandOrderRows : rows;
    // the same carving as vxhip_packed_linear_forward_f32, out of the fixed array
    Carver sizes{nullptr};
    sizes.take<float>(rows);
    sizes.take<int8_t>(prepared_rows * ld);
    if (sizes.off > kNoAllocScratchBytes) {
        set_error("packed_linear_forward_f32_noalloc: rows=%u k=%u need %zu bytes of staging, the fixed scratch "
                  "holds %zu (use vxhip_packed_linear_forward_f32, which sizes its own)",
                  rows, k, sizes.off, kNoAllocScratchBytes);
        return -1;
    }
    Carver c{(char*)ctx->no_alloc_scratch};
    float* row_scales = c.take<float>(rows);
    int8_t* prepared = c.take<int8_t>(prepared_rows * ld);
    // every byte the linear reads is written by the preparation first: nothing has to start at zero
    if (launch_prepare_i8(ctx->stream, input_dev, rows, k, prepared, ActivationLayout{ld, operand_order ? 1u : 0u},
                          row_scales) != VXHIP_OK)
        return -1;
    const int st = packed_run_a8(ctx, pl, prepared, ld, operand_order, row_scales, output_dev, nullptr, nullptr, rows);
    if (st != -2) return st;
    if (launch_prepare_i8(ctx->stream, input_dev, rows, k, prepared, ActivationLayout{ld, 0u}, row_scales) != VXHIP_OK)
        return -1;
    return packed_run_a8(ctx, pl, prepared, ld, false, row_scales, output_dev, nullptr, nullptr, rows);
}

// The output window of vx_packed_linear_forward (packed_linear_ops.inc:1550-1553): units are elements of
// the row-major output, [first, first + count); a count of 0 stands for the whole output (and then only
// first = 0 fits).  False for a window the reference refuses.
static bool unit_window(uint64_t rows, uint32_t n, uint64_t first_unit, uint64_t unit_count, uint64_t* first,
                        uint64_t* units) {
    const uint64_t all = rows * n;
    *first = first_unit;
    *units = unit_count ? unit_count : all;
    return first_unit <= all && *units <= all - first_unit;
}

int vxhip_packed_linear_forward_f32_window(VxHipContext* ctx, const VxHipPackedLinear* pl, const float* input_dev,
                                           float* output_dev, uint32_t rows, uint64_t first_unit, uint64_t unit_count) {
    if (!ctx || !pl || !input_dev || !output_dev) {
        set_error("packed_linear_forward_f32_window: null handle or tensor");
        return -1;
    }
    const uint32_t n = pl->w.n, k = pl->w.k;
    uint64_t first = 0, units = 0;
    if (!unit_window(rows, n, first_unit, unit_count, &first, &units)) {
        set_error("packed_linear_forward_f32_window: units [%llu, +%llu) do not fit %u rows of %u", (unsigned long long)first_unit,
                  (unsigned long long)unit_count, rows, n);
        return -1;
    }
    if (!units) return 0;
    // the rows the window touches; whole rows are computed, the window's elements are what gets written
    const uint64_t r0 = first / n, r1 = (first + units + n - 1u) / n;
    const float* x = input_dev + r0 * k;
    if (first % n == 0u && (first + units) % n == 0u)
        return vxhip_packed_linear_forward_f32(ctx, pl, x, output_dev + first, (uint32_t)(r1 - r0));
    if (!use_device(ctx->device)) return -1;
    if (ctx->recording && (size_t)(r1 - r0) * n * 4u > ctx->io_out_bytes) {
        set_error("packed_linear_forward_f32_window: a recording cannot grow the staging buffer");
        return -1;
    }
    if (!io_staging(ctx, 0, (size_t)(r1 - r0) * n * 4u)) return -1;
    float* staged = (float*)ctx->io_out;
    const int st = vxhip_packed_linear_forward_f32(ctx, pl, x, staged, (uint32_t)(r1 - r0));
    if (st != 0) return st;
    if (hipMemcpyAsync(output_dev + first, staged + (first - r0 * n), (size_t)units * 4u, hipMemcpyDeviceToDevice,
                       ctx->stream) != hipSuccess)
        return -1;
    return 0;
}

int vxhip_packed_linear_f32(const float* input, const uint32_t* packed_weight, const float* scale,
                            const float* bias, float* output, uint64_t rows, int32_t key_dim,
                            int32_t value_dim, int32_t rate, int32_t groups, int32_t normalize,
                            uint64_t first_unit, uint64_t unit_count) {
    // descriptor checks of vx_packed_linear_forward (packed_linear_ops.inc:1545-1554)
    if (!input || !packed_weight || !scale || !output || key_dim <= 0 || value_dim <= 0 || !rows ||
        rows > 0x7fffffffull)
        return -1;
    uint64_t first = 0, units = 0;
    if (!unit_window(rows, (uint32_t)value_dim, first_unit, unit_count, &first, &units)) return -1;
    const uint32_t bits = groups ? (uint32_t)groups : 4u;
    if ((bits != 8u && bits != 4u && bits != 3u && bits != 2u) || normalize != 8) {
        set_error("packed_linear_f32: this backend runs weight_bits 2, 3, 4 and 8 under DYNAMIC_I8 only");
        return -1;
    }
    VxHipContext* ctx = default_context();
    if (!ctx) return -1;
    if (rate <= 0) return -1;
    const uint32_t k = (uint32_t)key_dim, n = (uint32_t)value_dim;
    const size_t row_words = (size_t)(k / 32u) * bits + ((size_t)(k % 32u) * bits + 31u) / 32u;
    const size_t group_count = ((size_t)k + (size_t)rate - 1u) / (size_t)rate;
    ResidentKey key{};
    key.pointers[0] = packed_weight;
    key.pointers[1] = scale;
    key.pointers[2] = bias;
    key.extents[0] = k;
    key.extents[1] = n;
    key.extents[2] = (uint32_t)rate * 16u + bits;
    key.extents[3] = 2u;  // a PackedLinear
    key.fingerprint = fingerprint(0xcbf29ce484222325ull, packed_weight, (size_t)n * row_words * 4u);
    key.fingerprint = fingerprint(key.fingerprint, scale, (size_t)n * group_count * 4u);
    key.fingerprint = fingerprint(key.fingerprint, bias, (size_t)n * 4u);
    std::shared_ptr<ResidentWeights> held = resident_find(key);
    if (!held) {
        held = std::make_shared<ResidentWeights>();
        if (vxhip_packed_linear_create(packed_weight, scale, bias, k, n, (uint32_t)rate, bits, &held->packed) != VXHIP_OK)
            return -1;
        resident_insert(key, held, (size_t)vxhip_packed_linear_resident_bytes(held->packed));
    }
    if (!units) return 0;
    // Only the rows the window touches travel; they are computed whole and the window's elements, which
    // are one run of the row-major output, are what is copied back: everything else in `output` stays
    // as it was (the reference writes columns [begin, end) of the first and last row, :1593-1596).
    const uint64_t r0 = first / n, r1 = (first + units + n - 1u) / n;
    const size_t in_bytes = (size_t)(r1 - r0) * k * 4u, out_bytes = (size_t)(r1 - r0) * n * 4u;
    int st = -1;
    if (io_staging(ctx, in_bytes, out_bytes) && vxhip_memcpy_to_device(ctx, ctx->io_in, input + r0 * k, in_bytes) == VXHIP_OK) {
        st = vxhip_packed_linear_forward_f32(ctx, held->packed, (const float*)ctx->io_in, (float*)ctx->io_out,
                                             (uint32_t)(r1 - r0));
        if (st == 0 && vxhip_memcpy_to_host(ctx, output + first, (const float*)ctx->io_out + (first - r0 * n),
                                            (size_t)units * 4u) != VXHIP_OK)
            st = -1;
    }
    (void)hipStreamSynchronize(ctx->stream);
    return st;
}

// ---- boundaries -------------------------------------------------------------------

int vxhip_quantize_forward(VxHipContext* ctx, const float* input_dev, uint32_t elements, void* output_dev,
                           float scale, int32_t zp, uint32_t dtype) {
    if (!ctx || !input_dev || !output_dev || !byte_dtype(dtype) || !scale_ok(scale) ||
        !zero_point_ok(zp, dtype))
        return 0;
    if (!use_device(ctx->device)) return 0;
    set_last_variant(ctx, "hip.quantize-linear.elementwise");
    return launch_quantize(ctx->stream, input_dev, elements, output_dev, scale, zp,
                           dtype == VXHIP_DTYPE_I8) == VXHIP_OK;
}

int vxhip_dequantize_forward(VxHipContext* ctx, const void* input_dev, uint32_t elements, float scale,
                             int32_t zp, uint32_t dtype, float* output_dev) {
    if (!ctx || !input_dev || !output_dev || !byte_dtype(dtype)) return 0;
    if (!use_device(ctx->device)) return 0;
    set_last_variant(ctx, "hip.dequantize-linear.elementwise");
    return launch_dequantize(ctx->stream, input_dev, elements, scale, zp, dtype == VXHIP_DTYPE_I8,
                             output_dev) == VXHIP_OK;
}

// the descriptor checks of requantize_linear_i8u8 (portable_inference_kernels.inc:2441-2449); the multiplier on success
static bool requantize_admission(float input_scale, int32_t input_zp, float output_scale, int32_t output_zp,
                                 uint32_t input_dtype, uint32_t output_dtype, float* multiplier) {
    if (!byte_dtype(input_dtype) || !byte_dtype(output_dtype) || !scale_ok(input_scale) || !scale_ok(output_scale) ||
        !zero_point_ok(input_zp, input_dtype) || !zero_point_ok(output_zp, output_dtype))
        return false;
    volatile float m = input_scale / output_scale;
    *multiplier = m;
    return scale_ok(m);
}

int vxhip_requantize_forward(VxHipContext* ctx, const void* input_dev, uint32_t elements, void* output_dev,
                             float input_scale, int32_t input_zp, float output_scale, int32_t output_zp,
                             uint32_t input_dtype, uint32_t output_dtype) {
    float multiplier = 0.0f;
    if (!ctx || !input_dev || !output_dev || !elements ||
        !requantize_admission(input_scale, input_zp, output_scale, output_zp, input_dtype, output_dtype, &multiplier))
        return 0;
    if (!use_device(ctx->device)) return 0;
    set_last_variant(ctx, "hip.requantize-linear.elementwise");
    return launch_requantize(ctx->stream, input_dev, elements, output_dev, multiplier, input_zp, output_zp,
                             input_dtype == VXHIP_DTYPE_I8, output_dtype == VXHIP_DTYPE_I8) == VXHIP_OK;
}

int vxhip_requantize_linear_i8u8(const void* input, uint32_t input_elements, void* output, uint32_t output_elements,
                                 float input_scale, int32_t input_zp, float output_scale, int32_t output_zp,
                                 uint32_t input_dtype, uint32_t output_dtype) {
    float multiplier = 0.0f;
    // (the device form's own refusals as well: equal counts, no overlap --
    // cuda_graph_quantized_boundary_shape_host.inc:257-265)
    if (!input || !output || !input_elements || input_elements != output_elements ||
        !requantize_admission(input_scale, input_zp, output_scale, output_zp, input_dtype, output_dtype, &multiplier))
        return 0;
    const uintptr_t a = (uintptr_t)input, b = (uintptr_t)output;
    if (a < b + output_elements && b < a + input_elements) return 0;
    VxHipContext* ctx = default_context();
    if (!ctx) return 0;
    int ok = 0;
    // (the context's grow-only staging buffers, like the other host-pointer entry points)
    if (io_staging(ctx, input_elements, output_elements) &&
        vxhip_memcpy_to_device(ctx, ctx->io_in, input, input_elements) == VXHIP_OK) {
        ok = vxhip_requantize_forward(ctx, ctx->io_in, input_elements, ctx->io_out, input_scale, input_zp, output_scale,
                                      output_zp, input_dtype, output_dtype);
        if (ok && vxhip_memcpy_to_host(ctx, output, ctx->io_out, output_elements) != VXHIP_OK) ok = 0;
    }
    (void)hipStreamSynchronize(ctx->stream);
    return ok;
}

int vxhip_quantize_typed_f32_i8u8(const float* input, uint32_t elements, void* output, float scale,
                                  int32_t zp, uint32_t dtype) {
    if (!input || !output || !byte_dtype(dtype) || !scale_ok(scale) || !zero_point_ok(zp, dtype)) return 0;
    if (!elements) return 1;
    VxHipContext* ctx = default_context();
    if (!ctx) return 0;
    int ok = 0;
    if (io_staging(ctx, (size_t)elements * 4u, elements) &&
        vxhip_memcpy_to_device(ctx, ctx->io_in, input, (size_t)elements * 4u) == VXHIP_OK) {
        ok = vxhip_quantize_forward(ctx, (const float*)ctx->io_in, elements, ctx->io_out, scale, zp, dtype);
        if (ok && vxhip_memcpy_to_host(ctx, output, ctx->io_out, elements) != VXHIP_OK) ok = 0;
    }
    (void)hipStreamSynchronize(ctx->stream);
    return ok;
}

int vxhip_dequantize_typed_i8u8_f32(const void* input, uint32_t elements, float scale, int32_t zp,
                                    uint32_t dtype, float* output) {
    if (!input || !output || !byte_dtype(dtype)) return 0;
    if (!elements) return 1;
    VxHipContext* ctx = default_context();
    if (!ctx) return 0;
    int ok = 0;
    if (io_staging(ctx, elements, (size_t)elements * 4u) &&
        vxhip_memcpy_to_device(ctx, ctx->io_in, input, elements) == VXHIP_OK) {
        ok = vxhip_dequantize_forward(ctx, ctx->io_in, elements, scale, zp, dtype, (float*)ctx->io_out);
        if (ok && vxhip_memcpy_to_host(ctx, output, ctx->io_out, (size_t)elements * 4u) != VXHIP_OK) ok = 0;
    }
    (void)hipStreamSynchronize(ctx->stream);
    return ok;
}

void vxhip_resident_weights_clear(void) {
    std::lock_guard<std::mutex> lock(g_resident_mutex);
    g_resident.clear();
}

uint64_t vxhip_resident_weights_bytes(void) {
    std::lock_guard<std::mutex> lock(g_resident_mutex);
    uint64_t held = 0;
    for (const ResidentSlot& slot : g_resident) held += slot.bytes;
    return held;
}

}  // extern "C"
