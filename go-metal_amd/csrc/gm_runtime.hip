// Device, queue and buffer entry points of the C ABI (the HIP counterpart of
// cgo_bridge/bridge_memory.m and the device / queue part of bridge_device.m),
// plus the measurement helpers.
#include "gm_context.hpp"
#include "gm_plan.hpp"

#include "../../include/gometal_hip.h"

#include <hip/hip_fp16.h>

#include <cstring>
#include <exception>
#include <thread>

namespace gm {

// ---------------------------------------------------------------- errors ----
static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}

void clear_error() { g_error[0] = '\0'; }

void note_exception() noexcept
{
    try {
        throw;
    } catch (const std::exception &e) {
        set_error("exception: %s", e.what());
    } catch (...) {
        set_error("unknown exception");
    }
}

bool hip_ok(hipError_t e, const char *what)
{
    if (e == hipSuccess) return true;
    set_error("%s: %s", what, hipGetErrorString(e));
    return false;
}

// --------------------------------------------------------------- context ----
Context::~Context() = default;

static Context *g_ctx = nullptr;
static std::once_flag g_ctx_once;

Context *default_context()
{
    std::call_once(g_ctx_once, [] {
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess || count < 1) {
            set_error("no HIP device is visible");
            return;
        }
        auto *ctx = new Context();   // lives until the process ends
        ctx->device_id = 0;
        if (!hip_ok(hipSetDevice(0), "hipSetDevice") ||
            !hip_ok(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking), "hipStreamCreate") ||
            !hip_ok(hipEventCreate(&ctx->ev_start), "hipEventCreate") ||
            !hip_ok(hipEventCreate(&ctx->ev_stop), "hipEventCreate") ||
            !noalloc_bind_scratch(ctx)) {
            delete ctx;
            return;
        }
        ctx->usable = true;
        g_ctx = ctx;
    });
    return g_ctx;
}

Context *resolve_device(uintptr_t device)
{
    if (device == 0) return nullptr;
    return default_context();
}

bool make_current(Context *ctx) { return hip_ok(hipSetDevice(ctx->device_id), "hipSetDevice"); }

// -------------------------------------------------------------- registry ----
struct Allocation {
    size_t bytes;        // usable length from the handle on
    uintptr_t base;      // what hipMalloc returned (the handle itself unless the buffer is phased)
};
static std::mutex g_reg_mu;
static std::unordered_map<uintptr_t, Allocation> g_reg;

void registry_add(uintptr_t buffer, size_t bytes, uintptr_t base)
{
    std::lock_guard<std::mutex> lk(g_reg_mu);
    g_reg[buffer] = Allocation{bytes, base ? base : buffer};
}

uintptr_t registry_remove(uintptr_t buffer)
{
    std::lock_guard<std::mutex> lk(g_reg_mu);
    auto it = g_reg.find(buffer);
    if (it == g_reg.end()) return 0;
    const uintptr_t base = it->second.base;
    g_reg.erase(it);
    return base;
}

size_t registry_length(uintptr_t buffer)
{
    std::lock_guard<std::mutex> lk(g_reg_mu);
    auto it = g_reg.find(buffer);
    return it == g_reg.end() ? 0 : it->second.bytes;
}

// --------------------------------------------------------------- kernels ----
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
#define GM_GLOBAL __attribute__((address_space(1)))

// Launch shapes of the kernels below, measured on MI355X over 2^28 elements (1 GiB of fp32): with one
// or two streams the memory system prefers 16-byte accesses from single-wavefront workgroups, the
// opposite of the seven-stream optimizer update.  Conversion: 4 elements per lane (16-byte side +
// 8-byte side, non-temporal), 64 lanes: 85-87 % of the 8 TB/s peak, against 75-78 % for a grid-stride
// loop of 256-lane workgroups and 35-60 % for 1 or 2 elements per lane.  Copy: one 16-byte vector per
// lane, 64 lanes, 83 % (hipMemcpyAsync device-to-device: 63 %).  Zero fill: one 16-byte store per
// lane, 256 lanes, ordinary stores, 85 % (64 lanes: 59 %; grid-stride loop: 74 %).
constexpr int kConvertBlock = 64;
constexpr int kCopyBlock = 64;
constexpr int kZeroBlock = 256;

// fp32 -> fp16, round to nearest even (v_cvt_f16_f32).  GROUPED: lane i converts elements
// [4 i, 4 i + 4); the last n % 4 elements go to the first lanes of workgroup 0.  Otherwise
// (a view that is not aligned for 16-byte / 8-byte accesses) one element per lane.
template <bool GROUPED>
__global__ void __launch_bounds__(kConvertBlock)
convert_f32_to_f16_kernel(const float *__restrict__ src, _Float16 *__restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * kConvertBlock + threadIdx.x;
    if (!GROUPED) {
        if (i < n) dst[i] = (_Float16)src[i];
        return;
    }
    const size_t n4 = n / 4;
    if (i < n4) {
        const floatx4 x = __builtin_nontemporal_load(((const GM_GLOBAL floatx4 *)(src)) + i);
        halfx4 y;
#pragma unroll
        for (int c = 0; c < 4; c++) y[c] = (_Float16)x[c];
        __builtin_nontemporal_store(y, ((GM_GLOBAL halfx4 *)(dst)) + i);
    }
    if (blockIdx.x == 0 && n4 * 4 + threadIdx.x < n) dst[n4 * 4 + threadIdx.x] = (_Float16)src[n4 * 4 + threadIdx.x];
}

template <bool GROUPED>
__global__ void __launch_bounds__(kConvertBlock)
convert_f16_to_f32_kernel(const _Float16 *__restrict__ src, float *__restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * kConvertBlock + threadIdx.x;
    if (!GROUPED) {
        if (i < n) dst[i] = (float)src[i];
        return;
    }
    const size_t n4 = n / 4;
    if (i < n4) {
        const halfx4 x = __builtin_nontemporal_load(((const GM_GLOBAL halfx4 *)(src)) + i);
        floatx4 y;
#pragma unroll
        for (int c = 0; c < 4; c++) y[c] = (float)x[c];
        __builtin_nontemporal_store(y, ((GM_GLOBAL floatx4 *)(dst)) + i);
    }
    if (blockIdx.x == 0 && n4 * 4 + threadIdx.x < n) dst[n4 * 4 + threadIdx.x] = (float)src[n4 * 4 + threadIdx.x];
}

// Zero fill: bytes up to the first 16-byte boundary and after the last one by workgroup 0, one
// 16-byte store per lane between them.  (A kernel rather than hipMemsetAsync, so the entry point
// stays safe to record into a HIP graph.)
__global__ void __launch_bounds__(kZeroBlock)
zero_kernel(unsigned char *__restrict__ dst, size_t bytes, size_t head, size_t n16)
{
    const size_t i = (size_t)blockIdx.x * kZeroBlock + threadIdx.x;
    const uintx4 z = {0u, 0u, 0u, 0u};
    if (i < n16) ((GM_GLOBAL uintx4 *)(dst + head))[i] = z;
    if (blockIdx.x == 0) {
        for (size_t k = threadIdx.x; k < head; k += kZeroBlock) dst[k] = 0;
        for (size_t k = head + n16 * 16 + threadIdx.x; k < bytes; k += kZeroBlock) dst[k] = 0;
    }
}

// Plain copy, one 16-byte vector per lane, one wavefront per workgroup; the last bytes % 16 bytes
// go to the first lanes of workgroup 0.  Both addresses are 16-byte aligned.
__global__ void __launch_bounds__(kCopyBlock)
copy_kernel(const unsigned char *__restrict__ src, unsigned char *__restrict__ dst, size_t bytes)
{
    const size_t n16 = bytes / 16;
    const size_t i = (size_t)blockIdx.x * kCopyBlock + threadIdx.x;
    if (i < n16)
        __builtin_nontemporal_store(__builtin_nontemporal_load(((const GM_GLOBAL uintx4 *)(src)) + i),
                                    ((GM_GLOBAL uintx4 *)(dst)) + i);
    if (blockIdx.x == 0 && n16 * 16 + threadIdx.x < bytes) dst[n16 * 16 + threadIdx.x] = src[n16 * 16 + threadIdx.x];
}

__device__ inline uint64_t splitmix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// One Box-Muller pair per two consecutive elements.
__device__ inline void normal_pair(uint64_t seed, size_t pair_index, float &a, float &b)
{
    uint64_t r = splitmix64(seed ^ (0xD1B54A32D192ED03ull * (uint64_t)(pair_index + 1)));
    float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);   // (0, 1]
    float u2 = (float)(uint32_t)((r >> 8) & 0xFFFFFFu) * (1.0f / 16777216.0f);
    float rad = sqrtf(-2.0f * logf(u1));
    float s, c;
    sincosf(6.28318530717958647692f * u2, &s, &c);
    a = rad * c;
    b = rad * s;
}

template <bool HALF>
__global__ void __launch_bounds__(256)
fill_normal_kernel(void *__restrict__ dst, size_t n, uint64_t seed, float mean, float std, float scale)
{
    const size_t pairs = (n + 1) / 2;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x; p < pairs; p += stride) {
        float a, b;
        normal_pair(seed, p, a, b);
        a = a * std + mean;
        b = b * std + mean;
        const size_t i = 2 * p;
        if (HALF) {
            __half *d = reinterpret_cast<__half *>(dst);
            d[i] = __float2half_rn(a * scale);
            if (i + 1 < n) d[i + 1] = __float2half_rn(b * scale);
        } else {
            float *d = reinterpret_cast<float *>(dst);
            d[i] = a;
            if (i + 1 < n) d[i + 1] = b;
        }
    }
}

// ------------------------------------------------------- staged host copies ----
// Measured on MI355X hosts over 1 GiB of pageable memory: the runtime's own copy 18 GB/s device to
// host and 21-30 GB/s host to device; this pipeline 50 GB/s both ways with two lanes (no gain from
// four or eight); pinned memory end to end 57 GB/s.
constexpr size_t kStagedCopyMinBytes = 8u << 20;

static bool ensure_staging(Context *ctx)
{
    if (ctx->stage_ready) return true;
    for (StageLane &lane : ctx->stage) {
        if (!lane.stream &&
            !hip_ok(hipStreamCreateWithFlags(&lane.stream, hipStreamNonBlocking), "hipStreamCreate(staging)"))
            return false;
        for (int k = 0; k < 2; k++) {
            if (!lane.slot[k] && !hip_ok(hipHostMalloc(reinterpret_cast<void **>(&lane.slot[k]), kStageSlotBytes,
                                                      hipHostMallocDefault), "hipHostMalloc(staging)"))
                return false;
            if (!lane.ev[k] && !hip_ok(hipEventCreateWithFlags(&lane.ev[k], hipEventDisableTiming),
                                       "hipEventCreate(staging)"))
                return false;
        }
    }
    ctx->stage_ready = true;
    return true;
}

// One lane's share, device to host: the DMA of chunk k into one slot runs while chunk k - 1 is
// copied out of the other.
static hipError_t stage_to_host(StageLane &lane, char *dst, const char *src, size_t bytes)
{
    hipError_t e = hipSuccess;
    size_t off = 0, prev_off = 0, prev_len = 0;
    int k = 0;
    while (off < bytes && e == hipSuccess) {
        const size_t len = bytes - off < kStageSlotBytes ? bytes - off : kStageSlotBytes;
        const int slot = k & 1;
        e = hipMemcpyAsync(lane.slot[slot], src + off, len, hipMemcpyDeviceToHost, lane.stream);
        if (e == hipSuccess) e = hipEventRecord(lane.ev[slot], lane.stream);
        if (e == hipSuccess && k > 0) {
            e = hipEventSynchronize(lane.ev[slot ^ 1]);
            if (e == hipSuccess) std::memcpy(dst + prev_off, lane.slot[slot ^ 1], prev_len);
        }
        prev_off = off;
        prev_len = len;
        off += len;
        k++;
    }
    if (e == hipSuccess && k > 0) {
        e = hipEventSynchronize(lane.ev[(k - 1) & 1]);
        if (e == hipSuccess) std::memcpy(dst + prev_off, lane.slot[(k - 1) & 1], prev_len);
    }
    if (e != hipSuccess) (void)hipStreamSynchronize(lane.stream);   // nothing of this call stays in flight
    return e;
}

// Host to device: a slot is refilled once the DMA that last read it has finished.
static hipError_t stage_to_device(StageLane &lane, char *dst, const char *src, size_t bytes)
{
    hipError_t e = hipSuccess;
    size_t off = 0;
    int k = 0;
    while (off < bytes && e == hipSuccess) {
        const size_t len = bytes - off < kStageSlotBytes ? bytes - off : kStageSlotBytes;
        const int slot = k & 1;
        if (k >= 2) e = hipEventSynchronize(lane.ev[slot]);
        if (e == hipSuccess) {
            std::memcpy(lane.slot[slot], src + off, len);
            e = hipMemcpyAsync(dst + off, lane.slot[slot], len, hipMemcpyHostToDevice, lane.stream);
        }
        if (e == hipSuccess) e = hipEventRecord(lane.ev[slot], lane.stream);
        off += len;
        k++;
    }
    const hipError_t drained = hipStreamSynchronize(lane.stream);
    return e != hipSuccess ? e : drained;
}

// Copies bytes between a device range and pageable host memory through the staging lanes; the
// calling thread drives lane 0 and a helper thread lane 1.  Returns after the data has arrived.
// The caller has already ordered the copy after earlier work (the context's stream is idle).
static bool staged_copy(Context *ctx, char *device_ptr, char *host_ptr, size_t bytes, bool to_device)
{
    std::lock_guard<std::mutex> lk(ctx->stage_mu);
    if (!ensure_staging(ctx)) return false;
    const size_t first = ((bytes / kStageLanes) + 4095) / 4096 * 4096;      // lane 0's share, page aligned
    const size_t share[kStageLanes] = {first < bytes ? first : bytes, first < bytes ? bytes - first : 0};
    hipError_t result[kStageLanes] = {hipSuccess, hipSuccess};
    auto run = [&](int lane) {
        const size_t off = lane == 0 ? 0 : share[0];
        result[lane] = to_device ? stage_to_device(ctx->stage[lane], device_ptr + off, host_ptr + off, share[lane])
                                 : stage_to_host(ctx->stage[lane], host_ptr + off, device_ptr + off, share[lane]);
    };
    std::thread helper;
    bool helper_runs = false;
    if (share[1] > 0) {
        try {
            helper = std::thread([&] {
                if (hipSetDevice(ctx->device_id) != hipSuccess) {
                    result[1] = hipErrorInvalidDevice;
                    return;
                }
                run(1);
            });
            helper_runs = true;
        } catch (...) {
            helper_runs = false;      // no thread to be had: the calling thread takes both shares
        }
    }
    run(0);
    if (helper_runs) helper.join();
    else if (share[1] > 0) run(1);
    for (int lane = 0; lane < kStageLanes; lane++)
        if (!hip_ok(result[lane], to_device ? "staged copy to the device" : "staged copy to the host")) return false;
    return true;
}

static unsigned int grid_for(size_t work_items, unsigned int block, unsigned int max_blocks)
{
    size_t blocks = (work_items + block - 1) / block;
    if (blocks < 1) blocks = 1;
    if (blocks > max_blocks) blocks = max_blocks;
    return (unsigned int)blocks;
}

}  // namespace gm

using namespace gm;

// ================================================================= C ABI ====
extern "C" {

const char *gm_last_error(void) { return g_error; }

uintptr_t create_metal_device(void)
try {
    Context *ctx = default_context();
    if (!ctx) return 0;
    ctx->refs.fetch_add(1);
    return reinterpret_cast<uintptr_t>(ctx);
} catch (...) {
    note_exception();
    return 0;
}

void destroy_metal_device(uintptr_t device)
{
    Context *ctx = g_ctx;
    if (device == 0 || !ctx || reinterpret_cast<uintptr_t>(ctx) != device) return;
    // The context outlives every handle: pooled buffers and cached plans reached
    // through another handle must stay valid.  Only the count is dropped.
    if (ctx->refs.load() > 0) ctx->refs.fetch_sub(1);
}

struct CommandQueue {
    uint64_t magic;
    Context *ctx;
};
static const uint64_t kQueueMagic = 0x676D5F7175657565ull;   // "gm_queue"

uintptr_t create_command_queue(uintptr_t device)
try {
    if (device == 0) return 0;
    Context *ctx = resolve_device(device);
    if (!ctx) return 0;
    return reinterpret_cast<uintptr_t>(new CommandQueue{kQueueMagic, ctx});
} catch (...) {
    note_exception();
    return 0;
}

void release_command_queue(uintptr_t command_queue)
{
    if (command_queue == 0) return;
    auto *q = reinterpret_cast<CommandQueue *>(command_queue);
    if (q->magic != kQueueMagic) return;
    q->magic = 0;
    delete q;
}

uintptr_t allocate_metal_buffer(uintptr_t device, int size, int device_type)
try {
    (void)device_type;
    if (device == 0 || size <= 0) return 0;
    Context *ctx = resolve_device(device);
    if (!ctx || !make_current(ctx)) return 0;
    const size_t aligned = ((size_t)size + 15) / 16 * 16;
    void *p = nullptr;
    if (!hip_ok(hipMalloc(&p, aligned), "hipMalloc")) return 0;
    registry_add(reinterpret_cast<uintptr_t>(p), aligned);
    return reinterpret_cast<uintptr_t>(p);
} catch (...) {
    note_exception();
    return 0;
}

void deallocate_metal_buffer(uintptr_t buffer)
try {
    if (buffer == 0) return;
    const size_t len = registry_length(buffer);
    if (len == 0) return;   // not ours (or already freed): leave it alone
    Context *ctx = default_context();
    if (ctx) {
        make_current(ctx);
        // plans validated against this allocation go before the address can be handed out again
        std::lock_guard<std::mutex> lk(ctx->mu);
        plans_forget_range(ctx, buffer, len);
        lbfgs_forget_range(buffer, len);
    }
    const uintptr_t base = registry_remove(buffer);
    if (base) (void)hipFree(reinterpret_cast<void *>(base));   // hipFree waits for work in flight
} catch (...) {
    note_exception();
}

// Where a buffer starts decides which HBM channels and banks its elements fall into.  Buffers from
// hipMalloc share their low address bits (large ones are 2 MiB aligned), so element i of a
// tensor's weight, gradient and state buffers all land on the same channel at the same moment
// and a workgroup's four loads queue up behind each other.  Measured on MI355X, Adam over the
// 1.012B-parameter list: 82.0 % of peak with every stream at the same phase, 83.1 % with the two
// state streams 512 KiB and 1.5 MiB off (mod 2 MiB); 78.9 % to 84.4 % over flat arrays depending
// on the spacing alone (address bits 12, 19 and 20 separate streams, bits 13 and 21 set them
// against each other).  The optimizers own their state buffers and ask for them here.
constexpr size_t kPhasePeriod = 2u << 20;
constexpr size_t kPhasedMinBytes = 1u << 20;      // below this the phase is ignored: nothing to gain, 2 MiB to lose

uintptr_t gm_allocate_buffer_phased(uintptr_t device, int size, int device_type, int phase_bytes)
try {
    if (phase_bytes < 0 || (size_t)phase_bytes >= kPhasePeriod || phase_bytes % 256 != 0) {
        set_error("a phase is a multiple of 256 bytes below %zu (got %d)", kPhasePeriod, phase_bytes);
        return 0;
    }
    if (device == 0 || size <= 0) return 0;
    if ((size_t)size < kPhasedMinBytes) return allocate_metal_buffer(device, size, device_type);
    Context *ctx = resolve_device(device);
    if (!ctx || !make_current(ctx)) return 0;
    const size_t aligned = ((size_t)size + 15) / 16 * 16;
    void *p = nullptr;
    if (!hip_ok(hipMalloc(&p, aligned + kPhasePeriod), "hipMalloc")) return 0;
    const uintptr_t base = reinterpret_cast<uintptr_t>(p);
    const uintptr_t handle = base + (((uintptr_t)phase_bytes + kPhasePeriod - base % kPhasePeriod) % kPhasePeriod);
    registry_add(handle, aligned, base);
    return handle;
} catch (...) {
    note_exception();
    return 0;
}

size_t gm_buffer_length(uintptr_t buffer) { return registry_length(buffer); }

int zero_metal_buffer(uintptr_t device, uintptr_t buffer, int size)
try {
    if (device == 0 || buffer == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx || !make_current(ctx)) return -5;
    if (size <= 0) return 0;
    const size_t len = registry_length(buffer);
    if (len != 0 && (size_t)size > len) {
        set_error("zero of %d bytes exceeds the %zu-byte buffer", size, len);
        return -5;
    }
    size_t head = (16 - buffer % 16) % 16;
    if (head > (size_t)size) head = (size_t)size;
    const size_t n16 = ((size_t)size - head) / 16;
    const unsigned int grid = grid_for(n16, kZeroBlock, 0x7FFFFFFFu);
    zero_kernel<<<grid, kZeroBlock, 0, ctx->stream>>>(reinterpret_cast<unsigned char *>(buffer), (size_t)size, head,
                                                      n16);
    if (!hip_ok(hipGetLastError(), "zero kernel launch")) return -5;
    return 0;
} catch (...) {
    note_exception();
    return -5;
}

int zero_metal_buffer_mpsgraph(uintptr_t device, uintptr_t buffer, int size)
{
    return zero_metal_buffer(device, buffer, size);
}

int copy_data_to_metal_buffer(uintptr_t buffer, void *data, int size)
try {
    if (buffer == 0 || data == nullptr || size <= 0) return -1;
    const size_t len = registry_length(buffer);
    if (len != 0 && (size_t)size > len) {
        set_error("copy of %d bytes exceeds the %zu-byte buffer", size, len);
        return -3;
    }
    Context *ctx = default_context();
    if (!ctx || !make_current(ctx)) return -4;
    // The copy is ordered after earlier work on the stream and the call returns once the data
    // is on the device.
    if ((size_t)size >= kStagedCopyMinBytes) {
        if (!hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize") ||
            !staged_copy(ctx, reinterpret_cast<char *>(buffer), static_cast<char *>(data), (size_t)size, true))
            return -4;
        return 0;
    }
    if (!hip_ok(hipMemcpyAsync(reinterpret_cast<void *>(buffer), data, (size_t)size,
                               hipMemcpyHostToDevice, ctx->stream), "hipMemcpyAsync(H2D)") ||
        !hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))
        return -4;
    return 0;
} catch (...) {
    note_exception();
    return -4;
}

int copy_float32_array_to_metal_buffer(uintptr_t buffer, float *data, int num_elements)
{
    if (buffer == 0 || data == nullptr || num_elements <= 0) return -1;
    if ((size_t)num_elements * sizeof(float) > 0x7FFFFFFFull) return -1;
    return copy_data_to_metal_buffer(buffer, data, num_elements * (int)sizeof(float));
}

int copy_int32_array_to_metal_buffer(uintptr_t buffer, int *data, int num_elements)
{
    if (buffer == 0 || data == nullptr || num_elements <= 0) return -1;
    if ((size_t)num_elements * sizeof(int) > 0x7FFFFFFFull) return -1;
    return copy_data_to_metal_buffer(buffer, data, num_elements * (int)sizeof(int));
}

static int copy_from_buffer(uintptr_t buffer, void *data, size_t bytes)
{
    const size_t len = registry_length(buffer);
    if (len != 0 && bytes > len) {
        set_error("read of %zu bytes exceeds the %zu-byte buffer", bytes, len);
        return -3;
    }
    Context *ctx = default_context();
    if (!ctx || !make_current(ctx)) return -4;
    if (bytes >= kStagedCopyMinBytes) {
        if (!hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize") ||
            !staged_copy(ctx, reinterpret_cast<char *>(buffer), static_cast<char *>(data), bytes, false))
            return -4;
        return 0;
    }
    if (!hip_ok(hipMemcpyAsync(data, reinterpret_cast<void *>(buffer), bytes, hipMemcpyDeviceToHost,
                               ctx->stream), "hipMemcpyAsync(D2H)") ||
        !hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))
        return -4;
    return 0;
}

int copy_metal_buffer_to_float32_array(uintptr_t buffer, float *data, int num_elements)
{
    if (buffer == 0 || data == nullptr || num_elements <= 0) return -1;
    return copy_from_buffer(buffer, data, (size_t)num_elements * sizeof(float));
}

int copy_metal_buffer_to_int32_array(uintptr_t buffer, int *data, int num_elements)
{
    if (buffer == 0 || data == nullptr || num_elements <= 0) return -1;
    return copy_from_buffer(buffer, data, (size_t)num_elements * sizeof(int));
}

int convert_tensor_type(uintptr_t src_buffer, uintptr_t dst_buffer, int *shape, int num_dims,
                        int src_type, int dst_type, uintptr_t device)
try {
    if (src_buffer == 0 || dst_buffer == 0 || shape == nullptr || num_dims <= 0) return -1;
    if (device == 0) return -2;
    size_t total = 1;
    for (int i = 0; i < num_dims; i++) {
        if (shape[i] < 0) return -1;
        total *= (size_t)shape[i];
    }
    const bool to_half = (src_type == 0 && dst_type == 2);
    const bool to_float = (src_type == 2 && dst_type == 0);
    if (!to_half && !to_float) return -3;
    Context *ctx = resolve_device(device);
    if (!ctx || !make_current(ctx)) return -4;
    if (total == 0) return 0;
    const size_t src_len = registry_length(src_buffer), dst_len = registry_length(dst_buffer);
    if ((src_len != 0 && total * (to_half ? 4 : 2) > src_len) ||
        (dst_len != 0 && total * (to_half ? 2 : 4) > dst_len)) {
        set_error("conversion of %zu elements exceeds a buffer (src %zu bytes, dst %zu bytes)", total, src_len,
                  dst_len);
        return -5;
    }
    // 4-element groups only when both views are aligned for them (handles may be offset addresses)
    const bool grouped = src_buffer % (to_half ? 16 : 8) == 0 && dst_buffer % (to_half ? 8 : 16) == 0;
    const size_t lanes = grouped ? (total / 4 > 0 ? total / 4 : 1) : total;
    if ((lanes + kConvertBlock - 1) / kConvertBlock > 0x7FFFFFFFull) {
        set_error("conversion of %zu elements needs more workgroups than one launch can address", total);
        return -5;
    }
    const unsigned int grid = grid_for(lanes, kConvertBlock, 0x7FFFFFFFu);
    const float *f_src = reinterpret_cast<const float *>(src_buffer);
    const _Float16 *h_src = reinterpret_cast<const _Float16 *>(src_buffer);
    float *f_dst = reinterpret_cast<float *>(dst_buffer);
    _Float16 *h_dst = reinterpret_cast<_Float16 *>(dst_buffer);
    if (to_half && grouped) convert_f32_to_f16_kernel<true><<<grid, kConvertBlock, 0, ctx->stream>>>(f_src, h_dst, total);
    else if (to_half) convert_f32_to_f16_kernel<false><<<grid, kConvertBlock, 0, ctx->stream>>>(f_src, h_dst, total);
    else if (grouped) convert_f16_to_f32_kernel<true><<<grid, kConvertBlock, 0, ctx->stream>>>(h_src, f_dst, total);
    else convert_f16_to_f32_kernel<false><<<grid, kConvertBlock, 0, ctx->stream>>>(h_src, f_dst, total);
    if (!hip_ok(hipGetLastError(), "convert kernel launch")) return -4;
    return 0;
} catch (...) {
    note_exception();
    return -4;
}

int copy_buffer_to_buffer_sync(uintptr_t src_buffer, uintptr_t dst_buffer, int src_offset,
                               int dst_offset, int size)
try {
    if (src_buffer == 0 || dst_buffer == 0) return -1;
    if (size <= 0 || src_offset < 0 || dst_offset < 0) return -2;
    const size_t src_len = registry_length(src_buffer);
    const size_t dst_len = registry_length(dst_buffer);
    if (src_len != 0 && (size_t)src_offset + (size_t)size > src_len) return -4;
    if (dst_len != 0 && (size_t)dst_offset + (size_t)size > dst_len) return -5;
    Context *ctx = default_context();
    if (!ctx || !make_current(ctx)) return -10;
    const uintptr_t from = src_buffer + (uintptr_t)src_offset, to = dst_buffer + (uintptr_t)dst_offset;
    const bool overlap = from < to + (uintptr_t)size && to < from + (uintptr_t)size;
    if (from % 16 == 0 && to % 16 == 0 && !overlap) {
        // the library's own copy kernel: faster than the runtime's device-to-device copy
        const unsigned int grid = grid_for((size_t)size / 16, kCopyBlock, 0x7FFFFFFFu);
        copy_kernel<<<grid, kCopyBlock, 0, ctx->stream>>>(reinterpret_cast<const unsigned char *>(from),
                                                          reinterpret_cast<unsigned char *>(to), (size_t)size);
        if (!hip_ok(hipGetLastError(), "copy kernel launch")) return -10;
    } else if (!hip_ok(hipMemcpyAsync(reinterpret_cast<void *>(to), reinterpret_cast<const void *>(from),
                                      (size_t)size, hipMemcpyDeviceToDevice, ctx->stream), "hipMemcpyAsync(D2D)")) {
        return -10;
    }
    if (!hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize")) return -10;
    return 0;
} catch (...) {
    note_exception();
    return -11;
}

int gm_synchronize(uintptr_t device)
try {
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (!make_current(ctx) || !hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))
        return -10;
    return 0;
} catch (...) {
    note_exception();
    return -10;
}

// Cross-stream ordering without a host wait: an event recorded on one stream, waited for by
// the other.  The event is created per call and destroyed once recorded and enqueued (HIP keeps
// it alive until the wait has been satisfied).
static int order_streams(uintptr_t device, void *caller_stream, bool library_waits)
{
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (!make_current(ctx)) return -10;
    hipStream_t theirs = reinterpret_cast<hipStream_t>(caller_stream);
    hipStream_t first = library_waits ? theirs : ctx->stream;
    hipStream_t second = library_waits ? ctx->stream : theirs;
    hipEvent_t ev = nullptr;
    if (!hip_ok(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "hipEventCreate")) return -10;
    const bool ok = hip_ok(hipEventRecord(ev, first), "hipEventRecord") &&
                    hip_ok(hipStreamWaitEvent(second, ev, 0), "hipStreamWaitEvent");
    (void)hipEventDestroy(ev);
    return ok ? 0 : -10;
}

int gm_wait_for_stream(uintptr_t device, void *hip_stream) { return order_streams(device, hip_stream, true); }
int gm_signal_stream(uintptr_t device, void *hip_stream) { return order_streams(device, hip_stream, false); }

int gm_timer_start(uintptr_t device)
try {
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (!make_current(ctx) || !hip_ok(hipEventRecord(ctx->ev_start, ctx->stream), "hipEventRecord"))
        return -10;
    return 0;
} catch (...) {
    note_exception();
    return -10;
}

float gm_timer_stop(uintptr_t device)
try {
    if (device == 0) return -1.0f;
    Context *ctx = resolve_device(device);
    if (!ctx || !make_current(ctx)) return -1.0f;
    float ms = -1.0f;
    if (!hip_ok(hipEventRecord(ctx->ev_stop, ctx->stream), "hipEventRecord") ||
        !hip_ok(hipEventSynchronize(ctx->ev_stop), "hipEventSynchronize") ||
        !hip_ok(hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop), "hipEventElapsedTime"))
        return -1.0f;
    return ms;
} catch (...) {
    note_exception();
    return -1.0f;
}

static int fill_normal(uintptr_t device, uintptr_t buffer, size_t n, uint64_t seed, float mean,
                       float std, float scale, bool half)
{
    if (device == 0) return -1;
    if (buffer == 0) return -4;
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (!make_current(ctx)) return -10;
    if (n == 0) return 0;
    const size_t len = registry_length(buffer);
    if (len != 0 && n * (half ? 2 : 4) > len) {
        set_error("fill of %zu elements exceeds the %zu-byte buffer", n, len);
        return -5;
    }
    const unsigned int grid = grid_for((n + 1) / 2, 256, 1u << 16);
    if (half)
        fill_normal_kernel<true><<<grid, 256, 0, ctx->stream>>>(reinterpret_cast<void *>(buffer), n,
                                                                 seed, mean, std, scale);
    else
        fill_normal_kernel<false><<<grid, 256, 0, ctx->stream>>>(reinterpret_cast<void *>(buffer), n,
                                                                  seed, mean, std, scale);
    return hip_ok(hipGetLastError(), "fill kernel launch") ? 0 : -10;
}

int gm_fill_normal_f32(uintptr_t device, uintptr_t buffer, size_t num_elements, uint64_t seed,
                       float mean, float std)
{
    return fill_normal(device, buffer, num_elements, seed, mean, std, 1.0f, false);
}

int gm_fill_normal_f16(uintptr_t device, uintptr_t buffer, size_t num_elements, uint64_t seed,
                       float mean, float std, float scale)
{
    return fill_normal(device, buffer, num_elements, seed, mean, std, scale, true);
}

int gm_copy_probe(uintptr_t device, uintptr_t dst_buffer, uintptr_t src_buffer, size_t bytes)
try {
    if (device == 0) return -1;
    if (dst_buffer == 0 || src_buffer == 0) return -4;
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (!make_current(ctx)) return -10;
    const size_t src_len = registry_length(src_buffer), dst_len = registry_length(dst_buffer);
    if ((src_len != 0 && bytes > src_len) || (dst_len != 0 && bytes > dst_len) || bytes % 16 != 0 ||
        src_buffer % 16 != 0 || dst_buffer % 16 != 0) {
        set_error("copy probe of %zu bytes does not fit (src %zu, dst %zu) or is not 16-byte aligned and sized",
                  bytes, src_len, dst_len);
        return -5;
    }
    const size_t n16 = bytes / 16;
    if (n16 == 0) return 0;
    const size_t blocks = (n16 + kCopyBlock - 1) / kCopyBlock;
    if (blocks > 0x7FFFFFFFull) return -5;
    copy_kernel<<<(unsigned int)blocks, kCopyBlock, 0, ctx->stream>>>(
        reinterpret_cast<const unsigned char *>(src_buffer), reinterpret_cast<unsigned char *>(dst_buffer), bytes);
    return hip_ok(hipGetLastError(), "copy probe launch") ? 0 : -10;
} catch (...) {
    note_exception();
    return -10;
}

}  // extern "C"
