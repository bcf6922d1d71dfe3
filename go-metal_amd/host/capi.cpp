// Flat C view of the host-side mirror (include/gometal_optimizer.h).
#include "lbfgs.hpp"
#include "optimizer.hpp"
#include "scheduler.hpp"
#include "tensor.hpp"

#include "../../include/gometal_optimizer.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <exception>

using namespace gometal;
using namespace gometal::optimizer;

namespace {

thread_local std::string g_error;

int fail(const Error &e)
{
    g_error = e;
    return -1;
}

int ok()
{
    g_error.clear();
    return 0;
}

struct Handle {
    int kind;
    std::unique_ptr<Optimizer> opt;
};

Handle *H(uintptr_t h) { return reinterpret_cast<Handle *>(h); }
memory::MemoryManager *MM(uintptr_t h) { return reinterpret_cast<memory::MemoryManager *>(h); }

std::vector<Pointer> pointers(const uintptr_t *p, int n)
{
    std::vector<Pointer> v;
    if (p && n > 0) {
        v.reserve((size_t)n);
        for (int i = 0; i < n; i++) v.push_back(reinterpret_cast<Pointer>(p[i]));
    }
    return v;
}

// The parameters object of an OptimizerState document, decoded as encoding/json would.
std::map<std::string, ParamValue> parametersFrom(const char *parameters_json)
{
    const std::string doc = std::string("{\"type\":\"\",\"parameters\":") + (parameters_json ? parameters_json : "{}") + "}";
    auto [state, err] = OptimizerState::FromJSON(doc);
    if (!err.empty()) {
        fail(err);
        return {};
    }
    ok();
    return state.Parameters;
}

// No exception may cross the C boundary (the caller is C, Go or Python): a failed allocation or a
// standard-library error inside an entry point becomes that entry point's failure value, with the
// reason in gmo_last_error().
void note_exception() noexcept
{
    try {
        try {
            throw;
        } catch (const std::exception &e) {
            g_error = std::string("exception: ") + e.what();
        } catch (...) {
            g_error = "unknown exception";
        }
    } catch (...) {
    }
}

}  // namespace

extern "C" {

const char *gmo_last_error(void) { return g_error.c_str(); }
void gmo_free_string(char *s) { std::free(s); }

uintptr_t gmo_memory_manager_new(uintptr_t device)
try {
    return reinterpret_cast<uintptr_t>(new memory::MemoryManager(reinterpret_cast<Pointer>(device)));
} catch (...) {
    note_exception();
    return 0;
}

void gmo_memory_manager_free(uintptr_t mm) { delete MM(mm); }

void gmo_initialize_global_memory_manager(uintptr_t device)
try {
    memory::InitializeGlobalMemoryManager(reinterpret_cast<Pointer>(device));
} catch (...) {
    note_exception();
}

uintptr_t gmo_get_global_memory_manager(void)
try {
    return reinterpret_cast<uintptr_t>(memory::GetGlobalMemoryManager());
} catch (...) {
    note_exception();
    return 0;
}

uintptr_t gmo_allocate_buffer(uintptr_t mm, int size)
try {
    if (!mm) return 0;
    return reinterpret_cast<uintptr_t>(MM(mm)->AllocateBuffer(size));
} catch (...) {
    note_exception();
    return 0;
}

void gmo_release_buffer(uintptr_t mm, uintptr_t buffer)
try {
    if (mm) MM(mm)->ReleaseBuffer(reinterpret_cast<Pointer>(buffer));
} catch (...) {
    note_exception();
}

int gmo_find_pool_size(uintptr_t mm, int size) { return mm ? MM(mm)->findPoolSize(size) : -1; }
int gmo_calculate_max_pool_size(int buffer_size) { return memory::calculateMaxPoolSize(buffer_size); }
int gmo_reference_max_pool_size(int buffer_size) { return memory::referenceMaxPoolSize(buffer_size); }
void gmo_set_pool_byte_budget(size_t bytes) { memory::SetPoolByteBudget(bytes); }

int gmo_pool_stats(uintptr_t mm, int pool_size, int *available, int *allocated, int *max_size)
try {
    if (!mm) return -1;
    // buffers of one size are pooled apart by the phase they start at: the figures are summed over those pools
    auto stats = MM(mm)->Stats();
    int a = 0, b = 0, c = 0;
    bool found = false;
    for (const auto &kv : stats) {
        if (kv.first.Size != pool_size || kv.first.Device != memory::GPU) continue;
        int pa = 0, pb = 0, pc = 0;
        if (std::sscanf(kv.second.c_str(), "available=%d, allocated=%d, max=%d", &pa, &pb, &pc) != 3) return -1;
        a += pa;
        b += pb;
        c = pc > c ? pc : c;
        found = true;
    }
    if (!found) return -1;
    if (available) *available = a;
    if (allocated) *allocated = b;
    if (max_size) *max_size = c;
    return 0;
} catch (...) {
    note_exception();
    return -1;
}

int gmo_default_config(int kind, float c[6])
try {
    switch (kind) {
    case GMO_SGD: {
        auto d = DefaultSGDConfig();
        c[0] = d.LearningRate; c[1] = d.Momentum; c[2] = d.WeightDecay; c[3] = d.Nesterov ? 1.0f : 0.0f;
        return 4;
    }
    case GMO_ADAM: {
        auto d = DefaultAdamConfig();
        c[0] = d.LearningRate; c[1] = d.Beta1; c[2] = d.Beta2; c[3] = d.Epsilon; c[4] = d.WeightDecay;
        return 5;
    }
    case GMO_RMSPROP: {
        auto d = DefaultRMSPropConfig();
        c[0] = d.LearningRate; c[1] = d.Alpha; c[2] = d.Epsilon; c[3] = d.WeightDecay; c[4] = d.Momentum;
        c[5] = d.Centered ? 1.0f : 0.0f;
        return 6;
    }
    case GMO_ADAGRAD: {
        auto d = DefaultAdaGradConfig();
        c[0] = d.LearningRate; c[1] = d.Epsilon; c[2] = d.WeightDecay;
        return 3;
    }
    case GMO_ADADELTA: {
        auto d = DefaultAdaDeltaConfig();
        c[0] = d.Rho; c[1] = d.Epsilon; c[2] = d.WeightDecay;
        return 3;
    }
    case GMO_NADAM: {
        auto d = DefaultNadamConfig();
        c[0] = d.LearningRate; c[1] = d.Beta1; c[2] = d.Beta2; c[3] = d.Epsilon; c[4] = d.WeightDecay;
        return 5;
    }
    }
    return -1;
} catch (...) {
    note_exception();
    return -1;
}

uintptr_t gmo_optimizer_new(int kind, const float *c, const int *shape_dims, const int *shape_ndims,
                            int num_weights, uintptr_t memory_manager, uintptr_t device)
try {
    Shapes shapes;
    const int *d = shape_dims;
    for (int i = 0; i < num_weights; i++) {
        shapes.emplace_back(d, d + shape_ndims[i]);
        d += shape_ndims[i];
    }
    auto *mm = MM(memory_manager);
    Pointer dev = reinterpret_cast<Pointer>(device);
    std::unique_ptr<Optimizer> opt;
    Error err;
    switch (kind) {
    case GMO_SGD: {
        auto r = NewSGDOptimizer(SGDConfig{c[0], c[1], c[2], c[3] != 0.0f}, shapes, mm, dev);
        opt = std::move(r.first); err = r.second; break;
    }
    case GMO_ADAM: {
        auto r = NewAdamOptimizer(AdamConfig{c[0], c[1], c[2], c[3], c[4]}, shapes, mm, dev);
        opt = std::move(r.first); err = r.second; break;
    }
    case GMO_RMSPROP: {
        auto r = NewRMSPropOptimizer(RMSPropConfig{c[0], c[1], c[2], c[3], c[4], c[5] != 0.0f}, shapes, mm, dev);
        opt = std::move(r.first); err = r.second; break;
    }
    case GMO_ADAGRAD: {
        auto r = NewAdaGradOptimizer(AdaGradConfig{c[0], c[1], c[2]}, shapes, mm, dev);
        opt = std::move(r.first); err = r.second; break;
    }
    case GMO_ADADELTA: {
        auto r = NewAdaDeltaOptimizer(AdaDeltaConfig{c[0], c[1], c[2]}, shapes, mm, dev);
        opt = std::move(r.first); err = r.second; break;
    }
    case GMO_NADAM: {
        auto r = NewNadamOptimizer(NadamConfig{c[0], c[1], c[2], c[3], c[4]}, shapes, mm, dev);
        opt = std::move(r.first); err = r.second; break;
    }
    default: err = Errorf("unknown optimizer kind %d", kind);
    }
    if (!err.empty() || !opt) {
        fail(err);
        return 0;
    }
    ok();
    return reinterpret_cast<uintptr_t>(new Handle{kind, std::move(opt)});
} catch (...) {
    note_exception();
    return 0;
}

void gmo_optimizer_free(uintptr_t opt) { delete H(opt); }

int gmo_set_weight_buffers(uintptr_t opt, const uintptr_t *weight_buffers, int n)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    Error e = H(opt)->opt->SetWeightBuffers(pointers(weight_buffers, n));
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_step(uintptr_t opt, const uintptr_t *gradient_buffers, int n)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    Error e = H(opt)->opt->Step(pointers(gradient_buffers, n));
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

uint64_t gmo_get_step_count(uintptr_t opt)
try {
    if (!opt) {
        fail(Errorf("object handle is nil"));
        return 0;
    }
    return H(opt)->opt->GetStepCount();
} catch (...) {
    note_exception();
    return 0;
}

void gmo_update_learning_rate(uintptr_t opt, float lr)
try {
    if (!opt) return;
    H(opt)->opt->UpdateLearningRate(lr);
} catch (...) {
    note_exception();
}

void gmo_set_command_pool(uintptr_t opt, uintptr_t pool)
try {
    if (!opt) return;
    H(opt)->opt->SetCommandPool(reinterpret_cast<Pointer>(pool));
} catch (...) {
    note_exception();
}

void gmo_cleanup(uintptr_t opt)
try {
    if (!opt) return;
    H(opt)->opt->Cleanup();
} catch (...) {
    note_exception();
}


char *gmo_get_state_json(uintptr_t opt)
try {
    if (!opt) { fail(Errorf("object handle is nil")); return nullptr; }
    auto [state, err] = H(opt)->opt->GetState();
    if (!err.empty() || !state) {
        fail(err);
        return nullptr;
    }
    auto [js, jerr] = state->ToJSON();
    if (!jerr.empty()) {
        fail(jerr);
        return nullptr;
    }
    ok();
    char *out = (char *)std::malloc(js.size() + 1);
    if (out) std::memcpy(out, js.c_str(), js.size() + 1);
    return out;
} catch (...) {
    note_exception();
    return nullptr;
}

int gmo_load_state_json(uintptr_t opt, const char *json)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto [state, perr] = OptimizerState::FromJSON(json ? json : "");
    if (!perr.empty()) return fail(perr);
    Error e = H(opt)->opt->LoadState(&state);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

char *gmo_state_json_normalize(const char *json)
try {
    auto [state, perr] = OptimizerState::FromJSON(json ? json : "");
    if (!perr.empty()) {
        fail(perr);
        return nullptr;
    }
    auto [js, jerr] = state.ToJSON();
    if (!jerr.empty()) {
        fail(jerr);
        return nullptr;
    }
    ok();
    char *out = (char *)std::malloc(js.size() + 1);
    if (out) std::memcpy(out, js.c_str(), js.size() + 1);
    return out;
} catch (...) {
    note_exception();
    return nullptr;
}

char *gmo_get_checkpoint_json(uintptr_t opt)
try {
    if (!opt) { fail(Errorf("object handle is nil")); return nullptr; }
    auto [state, err] = H(opt)->opt->GetState();
    if (!err.empty() || !state) {
        fail(err);
        return nullptr;
    }
    auto [js, jerr] = state->ToCheckpointJSON();
    if (!jerr.empty()) {
        fail(jerr);
        return nullptr;
    }
    ok();
    char *out = (char *)std::malloc(js.size() + 1);
    if (out) std::memcpy(out, js.c_str(), js.size() + 1);
    return out;
} catch (...) {
    note_exception();
    return nullptr;
}

int gmo_load_checkpoint_json(uintptr_t opt, const char *json)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto [state, perr] = OptimizerState::FromCheckpointJSON(json ? json : "");
    if (!perr.empty()) return fail(perr);
    Error e = H(opt)->opt->LoadState(&state);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

float gmo_get_field(uintptr_t opt, const char *name)
try {
    if (!opt) return std::nanf("");
    Handle *h = H(opt);
    const std::string n = name ? name : "";
    auto b = [](bool v) { return v ? 1.0f : 0.0f; };
    switch (h->kind) {
    case GMO_SGD: {
        auto *o = static_cast<SGDOptimizerState *>(h->opt.get());
        if (n == "LearningRate") return o->LearningRate;
        if (n == "Momentum") return o->Momentum;
        if (n == "WeightDecay") return o->WeightDecay;
        if (n == "Nesterov") return b(o->Nesterov);
        break;
    }
    case GMO_ADAM: {
        auto *o = static_cast<AdamOptimizerState *>(h->opt.get());
        if (n == "LearningRate") return o->LearningRate;
        if (n == "Beta1") return o->Beta1;
        if (n == "Beta2") return o->Beta2;
        if (n == "Epsilon") return o->Epsilon;
        if (n == "WeightDecay") return o->WeightDecay;
        break;
    }
    case GMO_RMSPROP: {
        auto *o = static_cast<RMSPropOptimizerState *>(h->opt.get());
        if (n == "LearningRate") return o->LearningRate;
        if (n == "Alpha") return o->Alpha;
        if (n == "Epsilon") return o->Epsilon;
        if (n == "WeightDecay") return o->WeightDecay;
        if (n == "Momentum") return o->Momentum;
        if (n == "Centered") return b(o->Centered);
        break;
    }
    case GMO_ADAGRAD: {
        auto *o = static_cast<AdaGradOptimizerState *>(h->opt.get());
        if (n == "LearningRate") return o->config.LearningRate;
        if (n == "Epsilon") return o->config.Epsilon;
        if (n == "WeightDecay") return o->config.WeightDecay;
        break;
    }
    case GMO_ADADELTA: {
        auto *o = static_cast<AdaDeltaOptimizerState *>(h->opt.get());
        if (n == "Rho") return o->config.Rho;
        if (n == "Epsilon") return o->config.Epsilon;
        if (n == "WeightDecay") return o->config.WeightDecay;
        break;
    }
    case GMO_NADAM: {
        auto *o = static_cast<NadamOptimizerState *>(h->opt.get());
        if (n == "LearningRate") return o->config.LearningRate;
        if (n == "Beta1") return o->config.Beta1;
        if (n == "Beta2") return o->config.Beta2;
        if (n == "Epsilon") return o->config.Epsilon;
        if (n == "WeightDecay") return o->config.WeightDecay;
        break;
    }
    }
    return std::nanf("");
} catch (...) {
    note_exception();
    return NAN;
}

uintptr_t gmo_state_buffer(uintptr_t opt, const char *state_type, int index)
try {
    if (!opt) { fail(Errorf("object handle is nil")); return 0; }
    Handle *h = H(opt);
    const std::string t = state_type ? state_type : "";
    const std::vector<Pointer> *v = nullptr;
    switch (h->kind) {
    case GMO_SGD:
        if (t == "momentum") v = &static_cast<SGDOptimizerState *>(h->opt.get())->MomentumBuffers;
        break;
    case GMO_ADAM: {
        auto *o = static_cast<AdamOptimizerState *>(h->opt.get());
        if (t == "momentum") v = &o->CurrentMomentumBuffers();
        if (t == "variance") v = &o->CurrentVarianceBuffers();
        if (t == "weight") v = &o->CurrentWeightBuffers();       // ping-pong mode: where the fp32 weights are now
        break;
    }
    case GMO_RMSPROP: {
        auto *o = static_cast<RMSPropOptimizerState *>(h->opt.get());
        if (t == "squared_grad_avg") v = &o->SquaredGradAvgBuffers;
        if (t == "momentum") v = &o->MomentumBuffers;
        if (t == "gradient_avg") v = &o->GradientAvgBuffers;
        break;
    }
    case GMO_ADAGRAD:
        if (t == "squared_grad_avg") v = &static_cast<AdaGradOptimizerState *>(h->opt.get())->squaredGradAvgBuffers;
        break;
    case GMO_ADADELTA: {
        auto *o = static_cast<AdaDeltaOptimizerState *>(h->opt.get());
        if (t == "squared_grad_avg") v = &o->squaredGradAvgBuffers;
        if (t == "squared_update_avg") v = &o->squaredUpdateAvgBuffers;
        break;
    }
    case GMO_NADAM: {
        auto *o = static_cast<NadamOptimizerState *>(h->opt.get());
        if (t == "momentum") v = &o->momentumBuffers;
        if (t == "variance") v = &o->varianceBuffers;
        break;
    }
    }
    if (!v || index < 0 || index >= (int)v->size()) return 0;
    return reinterpret_cast<uintptr_t>((*v)[index]);
} catch (...) {
    note_exception();
    return 0;
}

int gmo_uses_pooling(uintptr_t opt)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    Handle *h = H(opt);
    switch (h->kind) {
    case GMO_SGD: return static_cast<SGDOptimizerState *>(h->opt.get())->usePooling;
    case GMO_ADAM: return static_cast<AdamOptimizerState *>(h->opt.get())->usePooling;
    case GMO_RMSPROP: return static_cast<RMSPropOptimizerState *>(h->opt.get())->usePooling;
    case GMO_ADAGRAD: return static_cast<AdaGradOptimizerState *>(h->opt.get())->usePooling;
    case GMO_ADADELTA: return static_cast<AdaDeltaOptimizerState *>(h->opt.get())->usePooling;
    case GMO_NADAM: return static_cast<NadamOptimizerState *>(h->opt.get())->usePooling;
    }
    return 0;
} catch (...) {
    note_exception();
    return -1;
}

void gmo_set_log_progress(uintptr_t opt, int on)
try {
    if (!opt) return;
    Handle *h = H(opt);
    if (h->kind == GMO_ADAGRAD) static_cast<AdaGradOptimizerState *>(h->opt.get())->logProgress = on != 0;
    if (h->kind == GMO_ADADELTA) static_cast<AdaDeltaOptimizerState *>(h->opt.get())->logProgress = on != 0;
} catch (...) {
    note_exception();
}

static AdamOptimizerState *adam_of(uintptr_t opt)
{
    Handle *h = H(opt);
    if (!h || h->kind != GMO_ADAM) return nullptr;
    return static_cast<AdamOptimizerState *>(h->opt.get());
}

int gmo_enable_mixed_precision(uintptr_t opt, float initial_scale, float growth_factor, float backoff_factor,
                               int growth_interval)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto *a = adam_of(opt);
    if (!a) return fail(Errorf("mixed precision is only available on the Adam optimizer"));
    Error e = a->EnableMixedPrecision(initial_scale, growth_factor, backoff_factor, growth_interval);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_enable_ping_pong(uintptr_t opt)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto *a = adam_of(opt);
    if (!a) return fail(Errorf("mixed precision is only available on the Adam optimizer"));
    Error e = a->EnablePingPong();
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_current_set(uintptr_t opt)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto *a = adam_of(opt);
    if (!a) return fail(Errorf("mixed precision is only available on the Adam optimizer"));
    (void)a->CurrentWeightBuffers();          // brings the host's view up to date after asynchronous steps
    ok();
    return a->PingPong() ? a->currentSet : 0;
} catch (...) {
    note_exception();
    return -1;
}

int gmo_step_amp(uintptr_t opt, const uintptr_t *gradient16_buffers, const uintptr_t *weight16_buffers, int n,
                 int *skipped)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto *a = adam_of(opt);
    if (!a) return fail(Errorf("mixed precision is only available on the Adam optimizer"));
    auto [sk, e] = a->StepAMP(pointers(gradient16_buffers, n), pointers(weight16_buffers, weight16_buffers ? n : 0));
    if (!e.empty()) return fail(e);
    if (skipped) *skipped = sk ? 1 : 0;
    return ok();
} catch (...) {
    note_exception();
    return -1;
}

int gmo_step_amp_async(uintptr_t opt, const uintptr_t *gradient16_buffers, const uintptr_t *weight16_buffers, int n)
try {
    auto *a = adam_of(opt);
    if (!a) return fail(Errorf("mixed precision is only available on the Adam optimizer"));
    Error e = a->StepAMPAsync(pointers(gradient16_buffers, n), pointers(weight16_buffers, weight16_buffers ? n : 0));
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_sync_amp(uintptr_t opt, uint64_t *skipped_steps)
try {
    auto *a = adam_of(opt);
    if (!a) return fail(Errorf("mixed precision is only available on the Adam optimizer"));
    Error e = a->SyncAMP(skipped_steps);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

float gmo_loss_scale(uintptr_t opt)
try {
    if (!opt) return std::nanf("");
    auto *a = adam_of(opt);
    return a ? a->LossScale : std::nanf("");
} catch (...) {
    note_exception();
    return NAN;
}

int gmo_growth_tracker(uintptr_t opt)
try {
    if (!opt) return fail(Errorf("object handle is nil"));
    auto *a = adam_of(opt);
    return a ? a->GrowthTracker : -1;
} catch (...) {
    note_exception();
    return -1;
}

// ---- optimizer/lbfgs.go ----
static LBFGSOptimizerState *L(uintptr_t h) { return reinterpret_cast<LBFGSOptimizerState *>(h); }

void gmo_lbfgs_default_config(int *history_size, float *line_search_tol, int *max_line_search, float *c1,
                              float *c2, float *initial_step)
try {
    const LBFGSConfig d = DefaultLBFGSConfig();
    if (history_size) *history_size = d.HistorySize;
    if (line_search_tol) *line_search_tol = d.LineSearchTol;
    if (max_line_search) *max_line_search = d.MaxLineSearch;
    if (c1) *c1 = d.C1;
    if (c2) *c2 = d.C2;
    if (initial_step) *initial_step = d.InitialStep;
} catch (...) {
    note_exception();
}

uintptr_t gmo_lbfgs_new(int history_size, float line_search_tol, int max_line_search, float c1, float c2,
                        float initial_step, const int *dims, const int *ndims, int num_weights,
                        uintptr_t memory_manager, uintptr_t device)
try {
    Shapes shapes;
    const int *d = dims;
    for (int k = 0; k < num_weights; k++) {
        shapes.emplace_back(d, d + ndims[k]);
        d += ndims[k];
    }
    auto [opt, err] = NewLBFGSOptimizer(LBFGSConfig{history_size, line_search_tol, max_line_search, c1, c2,
                                                    initial_step},
                                        shapes, MM(memory_manager), reinterpret_cast<Pointer>(device));
    if (!err.empty()) {
        fail(err);
        return 0;
    }
    ok();
    return reinterpret_cast<uintptr_t>(opt.release());
} catch (...) {
    note_exception();
    return 0;
}

void gmo_lbfgs_free(uintptr_t lbfgs) { delete L(lbfgs); }

int gmo_lbfgs_set_weight_buffers(uintptr_t lbfgs, const uintptr_t *buffers, int n)
try {
    if (!lbfgs) return fail(Errorf("object handle is nil"));
    Error e = L(lbfgs)->SetWeightBuffers(pointers(buffers, n));
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_lbfgs_step(uintptr_t lbfgs, const uintptr_t *gradient_buffers, int n, float current_loss)
try {
    if (!lbfgs) return fail(Errorf("object handle is nil"));
    Error e = L(lbfgs)->Step(pointers(gradient_buffers, n), current_loss);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

void gmo_lbfgs_set_command_pool(uintptr_t lbfgs, uintptr_t pool)
try {
    if (!lbfgs) return;
    L(lbfgs)->SetCommandPool(reinterpret_cast<Pointer>(pool));
} catch (...) {
    note_exception();
}

int gmo_lbfgs_uses_pooling(uintptr_t lbfgs)
try {
    if (!lbfgs) return fail(Errorf("object handle is nil"));
    return L(lbfgs)->usePooling ? 1 : 0;
} catch (...) {
    note_exception();
    return -1;
}

uint64_t gmo_lbfgs_get_step(uintptr_t lbfgs)
try {
    if (!lbfgs) {
        fail(Errorf("object handle is nil"));
        return 0;
    }
    return L(lbfgs)->GetStep();
} catch (...) {
    note_exception();
    return 0;
}


void gmo_lbfgs_get_stats(uintptr_t lbfgs, uint64_t *step, int *history_size, int *history_used, float *prev_loss)
try {
    if (!lbfgs) return;
    auto stats = L(lbfgs)->GetStats();
    if (step) *step = std::get<uint64_t>(stats.at("step"));
    if (history_size) *history_size = (int)std::get<uint64_t>(stats.at("history_size"));
    if (history_used) *history_used = (int)std::get<uint64_t>(stats.at("history_used"));
    if (prev_loss) *prev_loss = std::get<float>(stats.at("prev_loss"));
} catch (...) {
    note_exception();
}

void gmo_lbfgs_history(uintptr_t lbfgs, int *count, int *index, float *last_step_size)
try {
    if (!lbfgs) return;
    if (count) *count = L(lbfgs)->historyCount;
    if (index) *index = L(lbfgs)->historyIndex;
    if (last_step_size) *last_step_size = L(lbfgs)->lastStepSize;
} catch (...) {
    note_exception();
}

void gmo_lbfgs_cleanup(uintptr_t lbfgs)
try {
    if (!lbfgs) return;
    L(lbfgs)->Cleanup();
} catch (...) {
    note_exception();
}


int gmo_lbfgs_update_learning_rate(uintptr_t lbfgs, float lr)
try {
    if (!lbfgs) return fail(Errorf("object handle is nil"));
    Error e = L(lbfgs)->UpdateLearningRate(lr);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

void gmo_lbfgs_set_log_progress(uintptr_t lbfgs, int on)
try {
    if (!lbfgs) return;
    L(lbfgs)->logProgress = on != 0;
} catch (...) {
    note_exception();
}


int gmo_lbfgs_buffer_size(uintptr_t lbfgs, int index)
try {
    if (!lbfgs) return fail(Errorf("object handle is nil"));
    auto *l = L(lbfgs);
    return index >= 0 && (size_t)index < l->bufferSizes.size() ? l->bufferSizes[index] : -1;
} catch (...) {
    note_exception();
    return -1;
}

uintptr_t gmo_lbfgs_buffer(uintptr_t lbfgs, const char *which, int history, int index)
try {
    if (!lbfgs) { fail(Errorf("object handle is nil")); return 0; }
    auto *l = L(lbfgs);
    const std::string w = which ? which : "";
    const bool h_ok = history >= 0 && history < l->config.HistorySize;
    const bool i_ok = index >= 0 && (size_t)index < l->WeightBuffers.size();
    Pointer p = nullptr;
    if (w == "s" && h_ok && i_ok) p = l->sVectors[history][index];
    else if (w == "y" && h_ok && i_ok) p = l->yVectors[history][index];
    else if (w == "rho" && h_ok) p = l->rhoBuffers[history];
    else if (w == "alpha") p = l->alphaBuffer;
    else if (w == "old_gradient" && i_ok) p = l->oldGradients[index];
    else if (w == "search_dir" && i_ok) p = l->searchDir[index];
    else if (w == "weight" && i_ok) p = l->WeightBuffers[index];
    return reinterpret_cast<uintptr_t>(p);
} catch (...) {
    note_exception();
    return 0;
}

static memory::Tensor *T(uintptr_t h) { return reinterpret_cast<memory::Tensor *>(h); }

uintptr_t gmo_tensor_new(const int *shape, int ndims, int dtype, int device_type)
try {
    auto [t, err] = memory::Tensor::NewTensor(std::vector<int>(shape, shape + (ndims > 0 ? ndims : 0)),
                                              (memory::DataType)dtype, (memory::DeviceType)device_type);
    if (!err.empty()) {
        fail(err);
        return 0;
    }
    ok();
    return reinterpret_cast<uintptr_t>(t);
} catch (...) {
    note_exception();
    return 0;
}

uintptr_t gmo_tensor_retain(uintptr_t tensor)
try {
    if (!tensor) {
        fail(Errorf("object handle is nil"));
        return 0;
    }
    return reinterpret_cast<uintptr_t>(T(tensor)->Retain());
} catch (...) {
    note_exception();
    return 0;
}

void gmo_tensor_release(uintptr_t tensor)
try {
    if (tensor) T(tensor)->Release();
} catch (...) {
    note_exception();
}

void gmo_tensor_free(uintptr_t tensor) { delete T(tensor); }
uintptr_t gmo_tensor_buffer(uintptr_t tensor)
try {
    if (!tensor) {
        fail(Errorf("object handle is nil"));
        return 0;
    }
    return reinterpret_cast<uintptr_t>(T(tensor)->MetalBuffer());
} catch (...) {
    note_exception();
    return 0;
}

int gmo_tensor_size(uintptr_t tensor)
try {
    if (!tensor) return fail(Errorf("object handle is nil"));
    return T(tensor)->Size();
} catch (...) {
    note_exception();
    return -1;
}

int gmo_tensor_ref_count(uintptr_t tensor)
try {
    if (!tensor) return fail(Errorf("object handle is nil"));
    return T(tensor)->RefCount();
} catch (...) {
    note_exception();
    return -1;
}

int gmo_tensor_dtype(uintptr_t tensor)
try {
    if (!tensor) return fail(Errorf("object handle is nil"));
    return (int)T(tensor)->DType();
} catch (...) {
    note_exception();
    return -1;
}


uintptr_t gmo_tensor_convert_to(uintptr_t tensor, int dtype)
try {
    if (!tensor) { fail(Errorf("object handle is nil")); return 0; }
    auto [t, err] = T(tensor)->ConvertTo((memory::DataType)dtype);
    if (!err.empty()) {
        fail(err);
        return 0;
    }
    ok();
    return reinterpret_cast<uintptr_t>(t);
} catch (...) {
    note_exception();
    return 0;
}

int gmo_tensor_copy_float32_data(uintptr_t tensor, const float *data, int n)
try {
    if (!tensor) return fail(Errorf("object handle is nil"));
    Error e = T(tensor)->CopyFloat32Data(std::vector<float>(data, data + (n > 0 ? n : 0)));
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_tensor_to_float32_slice(uintptr_t tensor, float *out, int capacity)
try {
    if (!tensor) return fail(Errorf("object handle is nil"));
    auto [data, err] = T(tensor)->ToFloat32Slice();
    if (!err.empty()) return fail(err);
    if ((int)data.size() > capacity) return fail(Errorf("output holds %d elements, tensor has %d", capacity, (int)data.size()));
    std::memcpy(out, data.data(), data.size() * sizeof(float));
    ok();
    return (int)data.size();
} catch (...) {
    note_exception();
    return -1;
}

char *gmo_tensor_string(uintptr_t tensor)
try {
    if (!tensor) {
        fail(Errorf("object handle is nil"));
        return nullptr;
    }
    ok();
    const std::string text = T(tensor)->String();
    char *out = (char *)std::malloc(text.size() + 1);
    if (out) std::memcpy(out, text.c_str(), text.size() + 1);
    return out;
} catch (...) {
    note_exception();
    return nullptr;
}

int gmo_tensor_copy_from(uintptr_t dst, uintptr_t src)
try {
    if (!dst) return fail(Errorf("object handle is nil"));
    Error e = T(dst)->CopyFrom(T(src));
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_calculate_size(const int *shape, int ndims, int dtype)
try {
    return memory::calculateSize(std::vector<int>(shape, shape + (ndims > 0 ? ndims : 0)), (memory::DataType)dtype);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_execute_step_with_precomputed_gradients(uintptr_t opt, const uintptr_t *weight_tensors, int num_weights,
                                                const uintptr_t *gradient_tensors, int num_gradients)
try {
    std::vector<memory::Tensor *> w, g;     // a nil optimizer is the engine's own error case
    for (int k = 0; k < num_weights; k++) w.push_back(T(weight_tensors[k]));
    for (int k = 0; k < num_gradients; k++) g.push_back(T(gradient_tensors[k]));
    static const char *names[] = {"SGD", "Adam", "RMSProp", "AdaGrad", "AdaDelta", "Nadam"};
    Handle *h = H(opt);
    Error e = engine::ExecuteStepWithPrecomputedGradients(h ? h->opt.get() : nullptr, w, g, h ? names[h->kind] : "Adam");
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

struct SchedulerHandle {
    int kind;
    std::unique_ptr<training::LRScheduler> s;
    std::string name;
};

uintptr_t gmo_scheduler_new(int kind, int a, double b, double c, const char *mode)
try {
    auto *h = new SchedulerHandle{kind, nullptr, ""};
    switch (kind) {
    case 0: h->s = std::make_unique<training::StepLRScheduler>(a, b); break;
    case 1: h->s = std::make_unique<training::ExponentialLRScheduler>(b); break;
    case 2: h->s = std::make_unique<training::CosineAnnealingLRScheduler>(a, b); break;
    case 3: h->s = std::make_unique<training::ReduceLROnPlateauScheduler>(b, a, c, mode ? mode : ""); break;
    case 4: h->s = std::make_unique<training::NoOpScheduler>(); break;
    default: delete h; fail(Errorf("unknown scheduler kind %d", kind)); return 0;
    }
    h->name = h->s->GetName();
    return reinterpret_cast<uintptr_t>(h);
} catch (...) {
    note_exception();
    return 0;
}

void gmo_scheduler_free(uintptr_t scheduler) { delete reinterpret_cast<SchedulerHandle *>(scheduler); }

double gmo_scheduler_get_lr(uintptr_t scheduler, int epoch, int step, double base_lr)
try {
    if (!scheduler) return std::nan("");
    return reinterpret_cast<SchedulerHandle *>(scheduler)->s->GetLR(epoch, step, base_lr);
} catch (...) {
    note_exception();
    return NAN;
}

double gmo_scheduler_plateau_step(uintptr_t scheduler, double metric, double current_lr)
try {
    if (!scheduler) return std::nan("");
    auto *h = reinterpret_cast<SchedulerHandle *>(scheduler);
    if (h->kind != 3) return std::nan("");
    return static_cast<training::ReduceLROnPlateauScheduler *>(h->s.get())->Step(metric, current_lr);
} catch (...) {
    note_exception();
    return NAN;
}

const char *gmo_scheduler_name(uintptr_t scheduler)
try {
    if (!scheduler) {
        fail(Errorf("object handle is nil"));
        return "";
    }
    return reinterpret_cast<SchedulerHandle *>(scheduler)->name.c_str();
} catch (...) {
    note_exception();
    return nullptr;
}


double gmo_scheduler_apply(uintptr_t scheduler, uintptr_t opt, int epoch, int step, double base_lr)
try {
    if (!scheduler) return std::nan("");
    const double lr = gmo_scheduler_get_lr(scheduler, epoch, step, base_lr);
    if (opt) H(opt)->opt->UpdateLearningRate((float)lr);
    return lr;
} catch (...) {
    note_exception();
    return NAN;
}

float gmo_pow(float x, float y) { return optimizer::pow(x, y); }

int gmo_extract_buffer_index(const char *name) { return extractBufferIndex(name ? name : ""); }

float gmo_extract_float32_param(const char *parameters_json, const char *key, float default_value)
try {
    return extractFloat32Param(parametersFrom(parameters_json), key ? key : "", default_value);
} catch (...) {
    note_exception();
    return default_value;
}

int gmo_extract_bool_param(const char *parameters_json, const char *key, int default_value)
try {
    return extractBoolParam(parametersFrom(parameters_json), key ? key : "", default_value != 0) ? 1 : 0;
} catch (...) {
    note_exception();
    return default_value;
}

uint64_t gmo_extract_uint64_param(const char *parameters_json, const char *key, uint64_t default_value)
try {
    return extractUint64Param(parametersFrom(parameters_json), key ? key : "", default_value);
} catch (...) {
    note_exception();
    return default_value;
}

int gmo_validate_state_type(const char *optimizer_type, const char *state_type)
try {
    OptimizerState state;
    state.Type = state_type ? state_type : "";
    Error e = validateStateType(optimizer_type ? optimizer_type : "", &state);
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_restore_buffer_state(uintptr_t buffer, const float *data, int num_elements, int buffer_size,
                             const char *name)
try {
    std::vector<float> values;
    if (data && num_elements > 0) values.assign(data, data + num_elements);
    Error e = restoreBufferState(reinterpret_cast<Pointer>(buffer), values, buffer_size, name ? name : "");
    return e.empty() ? ok() : fail(e);
} catch (...) {
    note_exception();
    return -1;
}

int gmo_extract_buffer_state(uintptr_t buffer, int buffer_size, const char *name, const char *state_type,
                             float *data, int num_elements)
try {
    auto [tensor, err] = extractBufferState(reinterpret_cast<Pointer>(buffer), buffer_size, name ? name : "",
                                            state_type ? state_type : "");
    if (!err.empty()) return fail(err);
    ok();
    if (!tensor) return 0;
    if (data)
        for (int i = 0; i < num_elements && i < (int)tensor->Data.size(); i++) data[i] = tensor->Data[i];
    return 1;
} catch (...) {
    note_exception();
    return -1;
}

int gmo_calculate_tensor_size(const int *dims, int ndims)
try {
    return calculateTensorSize(std::vector<int>(dims, dims + (ndims > 0 ? ndims : 0)));
} catch (...) {
    note_exception();
    return -1;
}

}  // extern "C"
