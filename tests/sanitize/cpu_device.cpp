// A CPU stand-in for the device half of the C ABI (include/gometal_hip.h), for ONE purpose: to
// let the host-side mirror of the Go packages (go-metal_amd/host/*.cpp) be built and exercised
// under -fsanitize=address,undefined on a machine without a GPU.  Test infrastructure only; it is
// never part of libgometal_hip.so.
//
// Buffers are exact-length heap blocks, so the address sanitizer sees every byte the host code or
// a step touches.  A "step" computes no optimizer arithmetic (the GPU parity tests do that): it lays
// the request out with the library's own planner (csrc/gm_planner.cpp), walks every descriptor the
// way the kernels' grid does and increments every element of every written stream by one, so that
// a caller can still observe that a step happened and which buffers it covered.  The request
// masks restate those of the real entry points (csrc/gm_multi_tensor.hip, csrc/gm_amp.hip).
#include "../../go-metal_amd/csrc/gm_planner.hpp"
#include "../../include/gometal_hip.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

using namespace gm;

namespace {

std::mutex g_mu;
std::map<uintptr_t, size_t> g_buffers;
char g_error[256] = "";
int g_device_token;

size_t length_of(uintptr_t h)
{
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_buffers.find(h);
    return it == g_buffers.end() ? 0 : it->second;
}

// fp16 <-> fp32 with round to nearest even (what the device's conversion instructions do)
uint16_t f32_to_f16(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (x > 0x7F800000u ? 0x200u : 0));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);                 // rounds to infinity
    if (x < 0x33000001u) return (uint16_t)sign;                              // rounds to zero
    int e = (int)(x >> 23) - 127;
    uint32_t man = (x & 0x7FFFFFu) | 0x800000u;
    int shift = 13;
    if (e < -14) {
        shift += -14 - e;
        e = -15;
    }
    uint32_t half = man >> shift;
    const uint32_t rest = man & ((1u << shift) - 1), mid = 1u << (shift - 1);
    if (rest > mid || (rest == mid && (half & 1))) half++;
    return (uint16_t)(sign | (uint32_t)(((e + 15) << 10) + (int)half - (e == -15 ? 0 : 0x400)));
}

float f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t x;
    if (e == 0x1F) x = sign | 0x7F800000u | (man << 13);
    else if (e != 0) x = sign | ((e + 112) << 23) | (man << 13);
    else if (man == 0) x = sign;
    else {
        float f = std::ldexp((float)man, -24);
        std::memcpy(&x, &f, 4);
        x |= sign;
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// Walks the plan in the library's default launch shape and bumps every element of the written
// streams (reads the read-only ones): the accesses a step's kernel makes.
int walk(const PlanRequest &req, uint32_t written_mask, int streams)
{
    PlanLayout L;
    layout_plan(req, 0, length_of, L);
    if (L.status != 0) return L.status;
    const int vec = streams <= 5 ? 2 : 1, block = streams <= 5 ? 128 : 256;
    for (int s = 0; s < L.num_segments; s++) {
        const PlanSegment &seg = L.segment[s];
        uint32_t grid = 0, shift = 0;
        if (seg.num_chunks == 0) continue;
        if (!segment_grid(seg, vec, block, grid, shift)) return -6;
        for (uint32_t b = 0; b < grid; b++) {
            const Chunk &ch = L.chunks[seg.first_chunk + (b >> shift)];
            const uint32_t slice = b & ((1u << shift) - 1u);
            for (uint32_t lane = 0; lane < (uint32_t)block; lane++) {
                const LaneShare sh = lane_share(ch.count, ch.flags, slice, lane, vec, block);
                for (uint32_t e = 0; e < sh.count; e++) {
                    for (int k = 0; k < kNumSlots; k++) {
                        if (!ch.p[k]) continue;
                        const bool half = (req.half_mask >> k) & 1;
                        if (half) {
                            uint16_t *p = static_cast<uint16_t *>(ch.p[k]) + sh.first + e;
                            if ((written_mask >> k) & 1) *p = f32_to_f16(f16_to_f32(*p) + 1.0f);
                            else (void)*(volatile uint16_t *)p;
                        } else {
                            float *p = static_cast<float *>(ch.p[k]) + sh.first + e;
                            if ((written_mask >> k) & 1) *p = *p + 1.0f;
                            else (void)*(volatile float *)p;
                        }
                    }
                }
            }
        }
    }
    return 0;
}

constexpr uint32_t bit(int k) { return 1u << k; }

int adam_like(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *m, uintptr_t *v, int n, int *sizes, int kind)
{
    if (device == 0) return -1;
    PlanRequest req{};
    req.kind = kind;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g;
    req.slot[kSlotState0] = m;
    req.slot[kSlotState1] = v;
    req.sizes = sizes;
    req.required_mask = bit(kSlotWeight) | bit(kSlotGrad) | bit(kSlotState0) | bit(kSlotState1);
    req.missing_code = -4;
    return walk(req, bit(kSlotWeight) | bit(kSlotState0) | bit(kSlotState1), 7);
}

struct AmpState {
    float scale, growth, backoff;
    int interval, tracker, applied, skipped;
    int current_set;
};

}  // namespace

extern "C" {

const char *gm_last_error(void) { return g_error; }

uintptr_t create_metal_device(void) { return reinterpret_cast<uintptr_t>(&g_device_token); }
void destroy_metal_device(uintptr_t) {}
uintptr_t create_command_queue(uintptr_t device) { return device ? reinterpret_cast<uintptr_t>(std::malloc(8)) : 0; }
void release_command_queue(uintptr_t q) { std::free(reinterpret_cast<void *>(q)); }

uintptr_t allocate_metal_buffer(uintptr_t device, int size, int)
{
    if (device == 0 || size <= 0) return 0;
    const size_t bytes = ((size_t)size + 15) / 16 * 16;
    void *p = std::malloc(bytes);                    // exact length: overruns land in a red zone
    if (!p) return 0;
    std::memset(p, 0xA5, bytes);
    std::lock_guard<std::mutex> lk(g_mu);
    g_buffers[reinterpret_cast<uintptr_t>(p)] = bytes;
    return reinterpret_cast<uintptr_t>(p);
}

// The stand-in keeps exact-length heap blocks (so that overruns land in a red zone) and therefore cannot
// place a buffer at a phase; it checks the argument as the library does and remembers what was asked for.
std::map<uintptr_t, int> g_requested_phase;
uintptr_t gm_allocate_buffer_phased(uintptr_t device, int size, int device_type, int phase_bytes)
{
    if (phase_bytes < 0 || phase_bytes >= (2 << 20) || phase_bytes % 256 != 0) return 0;
    const uintptr_t h = allocate_metal_buffer(device, size, device_type);
    if (h != 0 && size >= (1 << 20)) {
        std::lock_guard<std::mutex> lk(g_mu);
        g_requested_phase[h] = phase_bytes;
    }
    return h;
}
int cpu_device_requested_phase(uintptr_t buffer)
{
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_requested_phase.find(buffer);
    return it == g_requested_phase.end() ? -1 : it->second;
}

void deallocate_metal_buffer(uintptr_t buffer)
{
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (g_buffers.erase(buffer) == 0) return;
        g_requested_phase.erase(buffer);
    }
    std::free(reinterpret_cast<void *>(buffer));
}

size_t gm_buffer_length(uintptr_t buffer) { return length_of(buffer); }

int zero_metal_buffer(uintptr_t device, uintptr_t buffer, int size)
{
    if (device == 0 || buffer == 0) return -1;
    if (size <= 0) return 0;
    const size_t len = length_of(buffer);
    if (len != 0 && (size_t)size > len) return -5;
    std::memset(reinterpret_cast<void *>(buffer), 0, (size_t)size);
    return 0;
}

int copy_data_to_metal_buffer(uintptr_t buffer, void *data, int size)
{
    if (buffer == 0 || data == nullptr || size <= 0) return -1;
    const size_t len = length_of(buffer);
    if (len != 0 && (size_t)size > len) return -3;
    std::memcpy(reinterpret_cast<void *>(buffer), data, (size_t)size);
    return 0;
}

int copy_float32_array_to_metal_buffer(uintptr_t buffer, float *data, int n)
{
    if (buffer == 0 || data == nullptr || n <= 0) return -1;
    return copy_data_to_metal_buffer(buffer, data, n * 4);
}

int copy_int32_array_to_metal_buffer(uintptr_t buffer, int *data, int n)
{
    if (buffer == 0 || data == nullptr || n <= 0) return -1;
    return copy_data_to_metal_buffer(buffer, data, n * 4);
}

int copy_metal_buffer_to_float32_array(uintptr_t buffer, float *data, int n)
{
    if (buffer == 0 || data == nullptr || n <= 0) return -1;
    const size_t len = length_of(buffer);
    if (len != 0 && (size_t)n * 4 > len) return -3;
    std::memcpy(data, reinterpret_cast<void *>(buffer), (size_t)n * 4);
    return 0;
}

int convert_tensor_type(uintptr_t src, uintptr_t dst, int *shape, int num_dims, int src_type, int dst_type,
                        uintptr_t device)
{
    if (src == 0 || dst == 0 || shape == nullptr || num_dims <= 0) return -1;
    if (device == 0) return -2;
    size_t total = 1;
    for (int i = 0; i < num_dims; i++) total *= (size_t)shape[i];
    if (src_type == 0 && dst_type == 2) {
        for (size_t i = 0; i < total; i++) reinterpret_cast<uint16_t *>(dst)[i] = f32_to_f16(reinterpret_cast<float *>(src)[i]);
        return 0;
    }
    if (src_type == 2 && dst_type == 0) {
        for (size_t i = 0; i < total; i++) reinterpret_cast<float *>(dst)[i] = f16_to_f32(reinterpret_cast<uint16_t *>(src)[i]);
        return 0;
    }
    return -3;
}

int copy_buffer_to_buffer_sync(uintptr_t src, uintptr_t dst, int src_offset, int dst_offset, int size)
{
    if (src == 0 || dst == 0) return -1;
    if (size <= 0 || src_offset < 0 || dst_offset < 0) return -2;
    const size_t sl = length_of(src), dl = length_of(dst);
    if (sl != 0 && (size_t)src_offset + (size_t)size > sl) return -4;
    if (dl != 0 && (size_t)dst_offset + (size_t)size > dl) return -5;
    std::memmove(reinterpret_cast<char *>(dst) + dst_offset, reinterpret_cast<char *>(src) + src_offset, (size_t)size);
    return 0;
}

int execute_sgd_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *m, int n, int *sizes, float,
                              float momentum, float, int, int)
{
    if (device == 0) return -1;
    PlanRequest req{};
    req.kind = kRuleSGD;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g;
    req.slot[kSlotState0] = momentum > 0.0f ? m : nullptr;
    req.sizes = sizes;
    req.skip_if_zero_mask = bit(kSlotWeight) | bit(kSlotGrad);
    return walk(req, bit(kSlotWeight) | bit(kSlotState0), 5);
}

int execute_adam_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *m, uintptr_t *v, int n,
                               int *sizes, float, float, float, float, float, int)
{
    return adam_like(device, w, g, m, v, n, sizes, kRuleAdam);
}

int execute_nadam_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *m, uintptr_t *v, int n,
                                int *sizes, float, float, float, float, float, int)
{
    return adam_like(device, w, g, m, v, n, sizes, kRuleNAdam);
}

int execute_rmsprop_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *s, uintptr_t *mom,
                                  uintptr_t *gavg, int n, int *sizes, float, float, float, float, float momentum,
                                  bool centered, int)
{
    if (device == 0) return -1;
    PlanRequest req{};
    req.kind = kRuleRMSProp;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g;
    req.slot[kSlotState0] = s;
    int next = kSlotState1;
    uint32_t written = bit(kSlotWeight) | bit(kSlotState0);
    if (momentum > 0.0f) {
        if (!mom) return -5;
        written |= bit(next);
        req.slot[next++] = mom;
    }
    if (centered) {
        if (!gavg) return -6;
        written |= bit(next);
        req.slot[next++] = gavg;
    }
    req.sizes = sizes;
    req.required_mask = bit(kSlotWeight) | bit(kSlotGrad) | bit(kSlotState0);
    req.missing_code = -4;
    return walk(req, written, 5 + 2 * (next - kSlotState1));
}

int execute_adagrad_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *s, int n, int *sizes,
                                  float, float, float)
{
    if (device == 0) return -1;
    PlanRequest req{};
    req.kind = kRuleAdaGrad;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g;
    req.slot[kSlotState0] = s;
    req.sizes = sizes;
    req.skip_if_zero_mask = bit(kSlotWeight) | bit(kSlotGrad) | bit(kSlotState0);
    return walk(req, bit(kSlotWeight) | bit(kSlotState0), 5);
}

int execute_adagrad_step_mpsgraph_pooled(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *s, int n,
                                         int *sizes, float lr, float eps, float wd, uintptr_t)
{
    return execute_adagrad_step_mpsgraph(device, w, g, s, n, sizes, lr, eps, wd);
}

int execute_adadelta_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *s, uintptr_t *a, int n,
                                   int *sizes, float, float, float)
{
    if (device == 0) return -1;
    PlanRequest req{};
    req.kind = kRuleAdaDelta;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g;
    req.slot[kSlotState0] = s;
    req.slot[kSlotState1] = a;
    req.sizes = sizes;
    req.skip_if_zero_mask = bit(kSlotWeight) | bit(kSlotGrad) | bit(kSlotState0) | bit(kSlotState1);
    return walk(req, bit(kSlotWeight) | bit(kSlotState0) | bit(kSlotState1), 7);
}

int execute_adadelta_step_mpsgraph_pooled(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *s, uintptr_t *a,
                                          int n, int *sizes, float rho, float eps, float wd, uintptr_t)
{
    return execute_adadelta_step_mpsgraph(device, w, g, s, a, n, sizes, rho, eps, wd);
}

// L-BFGS: every buffer of the step is read and the written ones bumped, over their full sizes.
int execute_lbfgs_step_mpsgraph(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *old_g, uintptr_t *dir,
                                uintptr_t *s, uintptr_t *y, uintptr_t *rho, uintptr_t alpha, int n, int *sizes,
                                int history_size, int history_count, int history_index, float initial_step, float,
                                float, int, float, float, float *step_size)
{
    if (device == 0) return -1;
    if (history_size <= 0 || history_count < 0 || history_count > history_size || history_index < 0 ||
        history_index >= history_size)
        return -5;
    if (!w || !g || !old_g || !dir || !s || !y || !rho || !alpha) return -8;
    for (int i = 0; i < n; i++) {
        const size_t numel = sizes[i] > 0 ? (size_t)sizes[i] / 4 : 0;
        uintptr_t rows[4] = {w[i], g[i], old_g[i], dir[i]};
        for (uintptr_t h : rows) {
            if (!h) return -8;
            float *p = reinterpret_cast<float *>(h);
            for (size_t e = 0; e < numel; e++) p[e] = p[e] + (h == g[i] ? 0.0f : 1.0f);
        }
        for (int h = 0; h < history_size; h++) {
            float *sp = reinterpret_cast<float *>(s[(size_t)h * n + i]), *yp = reinterpret_cast<float *>(y[(size_t)h * n + i]);
            if (!sp || !yp) return -8;
            for (size_t e = 0; e < numel; e++) sp[e] = yp[e] + 0.0f * sp[e];
        }
    }
    for (int h = 0; h < history_size; h++) {
        if (!rho[h]) return -8;
        *reinterpret_cast<float *>(rho[h]) = 0.0f;
    }
    for (int h = 0; h < history_size; h++) reinterpret_cast<float *>(alpha)[h] = 0.0f;
    if (step_size) *step_size = initial_step;
    return 0;
}

int execute_lbfgs_step_mpsgraph_pooled(uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *old_g, uintptr_t *dir,
                                       uintptr_t *s, uintptr_t *y, uintptr_t *rho, uintptr_t alpha, int n, int *sizes,
                                       int history_size, int history_count, int history_index, float initial_step,
                                       float c1, float c2, int max_ls, float cur, float prev, uintptr_t,
                                       float *step_size)
{
    return execute_lbfgs_step_mpsgraph(device, w, g, old_g, dir, s, y, rho, alpha, n, sizes, history_size,
                                       history_count, history_index, initial_step, c1, c2, max_ls, cur, prev, step_size);
}

// ---- loss-scale state and the mixed-precision step (the state machine of csrc/gm_amp.hip) ----
uintptr_t gm_amp_state_create(uintptr_t device, float init_scale, float growth, float backoff, int interval)
{
    if (device == 0) return 0;
    return reinterpret_cast<uintptr_t>(new AmpState{init_scale, growth, backoff, interval, 0, 0, 0, 0});
}
void gm_amp_state_destroy(uintptr_t h) { delete reinterpret_cast<AmpState *>(h); }

int gm_amp_state_query(uintptr_t h, float *scale, int *tracker, int *applied, int *skipped)
{
    if (!h) return -16;
    const AmpState *s = reinterpret_cast<AmpState *>(h);
    if (scale) *scale = s->scale;
    if (tracker) *tracker = s->tracker;
    if (applied) *applied = s->applied;
    if (skipped) *skipped = s->skipped;
    return 0;
}
int gm_amp_state_get(uintptr_t h, float *scale, int *tracker) { return gm_amp_state_query(h, scale, tracker, nullptr, nullptr); }
int gm_amp_state_set(uintptr_t h, float scale, int tracker)
{
    if (!h) return -16;
    reinterpret_cast<AmpState *>(h)->scale = scale;
    reinterpret_cast<AmpState *>(h)->tracker = tracker;
    return 0;
}
int gm_amp_state_set_step_count(uintptr_t h, int applied)
{
    if (!h) return -16;
    if (applied < 0) return -5;
    reinterpret_cast<AmpState *>(h)->applied = applied;
    return 0;
}
int gm_amp_state_max_in_flight(uintptr_t h) { return h ? 0 : -16; }

int execute_adam_amp_step(uintptr_t device, uintptr_t *w, uintptr_t *g16, uintptr_t *m, uintptr_t *v, uintptr_t *w16,
                          int n, int *sizes, float, float, float, float, float, int, uintptr_t amp, int *skipped,
                          float *scale_out, int *tracker_out)
{
    if (device == 0) return -1;
    if (!amp) return -16;
    AmpState *st = reinterpret_cast<AmpState *>(amp);
    PlanRequest req{};
    req.kind = kRuleAdamAMP;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g16;
    req.slot[kSlotState0] = m;
    req.slot[kSlotState1] = v;
    req.slot[kSlotWeight16] = w16;
    req.sizes = sizes;
    req.required_mask = bit(kSlotWeight) | bit(kSlotGrad) | bit(kSlotState0) | bit(kSlotState1);
    req.missing_code = -4;
    req.half_mask = bit(kSlotGrad) | bit(kSlotWeight16);
    bool found = false;
    for (int i = 0; i < n && g16 && !found; i++) {
        if (!w || !m || !v || !w[i] || !g16[i] || !m[i] || !v[i]) return -4;
        const uint16_t *g = reinterpret_cast<const uint16_t *>(g16[i]);
        const size_t numel = sizes[i] > 0 ? (size_t)sizes[i] / 4 : 0;
        for (size_t e = 0; e < numel; e++)
            if ((g[e] & 0x7C00u) == 0x7C00u) found = true;
    }
    if (found) {
        const float next = st->scale * st->backoff;
        if (next >= 1.17549435e-38f) st->scale = next;
        st->tracker = 0;
        st->skipped++;
    } else {
        const int rc = walk(req, bit(kSlotWeight) | bit(kSlotState0) | bit(kSlotState1) | bit(kSlotWeight16), 8);
        if (rc != 0) return rc;
        st->applied++;
        if (++st->tracker == st->interval) {
            const float next = st->scale * st->growth;
            if (next <= 3.40282347e+38f) st->scale = next;
            st->tracker = 0;
        }
    }
    if (skipped) *skipped = found ? 1 : 0;
    if (scale_out) *scale_out = st->scale;
    if (tracker_out) *tracker_out = st->tracker;
    return 0;
}

int execute_adam_amp_step_async(uintptr_t device, uintptr_t *w, uintptr_t *g16, uintptr_t *m, uintptr_t *v,
                                uintptr_t *w16, int n, int *sizes, float lr, float b1, float b2, float eps, float wd,
                                uintptr_t amp)
{
    return execute_adam_amp_step(device, w, g16, m, v, w16, n, sizes, lr, b1, b2, eps, wd, 0, amp, nullptr, nullptr,
                                 nullptr);
}

int gm_amp_state_current_set(uintptr_t h) { return h ? reinterpret_cast<AmpState *>(h)->current_set : -16; }
int gm_amp_state_set_current_set(uintptr_t h, int set)
{
    if (!h) return -16;
    if (set != 0 && set != 1) return -5;
    reinterpret_cast<AmpState *>(h)->current_set = set;
    return 0;
}

// The one-pass step over ping-pong state: the current set is read, the other one written.
int execute_adam_amp_step_fused(uintptr_t device, uintptr_t *wa, uintptr_t *ma, uintptr_t *va, uintptr_t *wb,
                                uintptr_t *mb, uintptr_t *vb, uintptr_t *g16, uintptr_t *w16, int n, int *sizes, float,
                                float, float, float, float, int, uintptr_t amp, int *skipped, float *scale_out,
                                int *tracker_out, int *current_set_out)
{
    if (device == 0) return -1;
    if (!amp) return -16;
    if (!wa || !ma || !va || !wb || !mb || !vb) return -4;
    AmpState *st = reinterpret_cast<AmpState *>(amp);
    const bool b_current = st->current_set != 0;
    uintptr_t *set_a[3] = {wa, ma, va}, *set_b[3] = {wb, mb, vb};
    uintptr_t **in = b_current ? set_b : set_a;
    uintptr_t **out = b_current ? set_a : set_b;
    bool found = false;
    for (int i = 0; i < n; i++) {
        for (int k = 0; k < 3; k++)
            if (!in[k][i] || !out[k][i]) return -4;
        if (!g16 || !g16[i]) return -4;
        const size_t numel = sizes[i] > 0 ? (size_t)sizes[i] / 4 : 0;
        const uint16_t *g = reinterpret_cast<const uint16_t *>(g16[i]);
        for (size_t e = 0; e < numel; e++) {
            if ((g[e] & 0x7C00u) == 0x7C00u) found = true;
            for (int k = 0; k < 3; k++)
                reinterpret_cast<float *>(out[k][i])[e] = reinterpret_cast<const float *>(in[k][i])[e] + 1.0f;
            if (w16 && w16[i]) reinterpret_cast<uint16_t *>(w16[i])[e] = f32_to_f16(reinterpret_cast<float *>(out[0][i])[e]);
        }
    }
    if (found) {
        const float next = st->scale * st->backoff;
        if (next >= 1.17549435e-38f) st->scale = next;
        st->tracker = 0;
        st->skipped++;
        for (int i = 0; i < n && w16; i++) {                    // the repair pass
            if (!w16[i]) continue;
            const size_t numel = sizes[i] > 0 ? (size_t)sizes[i] / 4 : 0;
            for (size_t e = 0; e < numel; e++)
                reinterpret_cast<uint16_t *>(w16[i])[e] = f32_to_f16(reinterpret_cast<float *>(in[0][i])[e]);
        }
    } else {
        st->applied++;
        st->current_set ^= 1;
        if (++st->tracker == st->interval) {
            const float next = st->scale * st->growth;
            if (next <= 3.40282347e+38f) st->scale = next;
            st->tracker = 0;
        }
    }
    if (skipped) *skipped = found ? 1 : 0;
    if (scale_out) *scale_out = st->scale;
    if (tracker_out) *tracker_out = st->tracker;
    if (current_set_out) *current_set_out = st->current_set;
    return 0;
}

int execute_adam_amp_step_fused_async(uintptr_t device, uintptr_t *wa, uintptr_t *ma, uintptr_t *va, uintptr_t *wb,
                                      uintptr_t *mb, uintptr_t *vb, uintptr_t *g16, uintptr_t *w16, int n, int *sizes,
                                      float lr, float b1, float b2, float eps, float wd, uintptr_t amp)
{
    return execute_adam_amp_step_fused(device, wa, ma, va, wb, mb, vb, g16, w16, n, sizes, lr, b1, b2, eps, wd, 0, amp,
                                       nullptr, nullptr, nullptr, nullptr);
}

int gm_synchronize(uintptr_t device) { return device ? 0 : -1; }

}  // extern "C"
