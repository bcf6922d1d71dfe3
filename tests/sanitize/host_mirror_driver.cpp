// Drives the host-side mirror of the Go packages (go-metal_amd/host/*.cpp) through its C view
// (include/gometal_optimizer.h) on top of the CPU stand-in device (cpu_device.cpp).  Built with
// -fsanitize=address,undefined: the point is that none of these calls reads or writes out of
// bounds, leaks, or hits undefined behaviour; functional results are asserted where cheap.
#include "../../include/gometal_hip.h"
#include "../../include/gometal_optimizer.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

static int g_failures = 0;
#define CHECK(cond)                                                                     \
    do {                                                                                \
        if (!(cond)) {                                                                  \
            std::fprintf(stderr, "FAIL %s:%d %s  (last error: %s)\n", __FILE__, __LINE__, #cond, gmo_last_error()); \
            g_failures++;                                                               \
        }                                                                               \
    } while (0)

static std::string take(char *s)
{
    std::string out = s ? s : "";
    if (s) gmo_free_string(s);
    return out;
}

static const int kDims[] = {32, 3, 3, 3, 32, 300, 17, 1, 70001};
static const int kNdims[] = {4, 1, 2, 1, 1};
static const int kSizes[] = {864, 32, 5100, 1, 70001};
static const int kTensors = 5;

static std::vector<float> read_buffer(uintptr_t h, int n)
{
    std::vector<float> out((size_t)n);
    CHECK(copy_metal_buffer_to_float32_array(h, out.data(), n) == 0);
    return out;
}

static void optimizers(uintptr_t device, uintptr_t mm)
{
    const char *state_kinds[] = {"momentum", "variance", "squared_grad_avg", "gradient_avg", "squared_update_avg"};
    for (int kind = GMO_SGD; kind <= GMO_NADAM; kind++) {
        for (int variant = 0; variant < 2; variant++) {
            float cfg[6] = {0};
            gmo_default_config(kind, cfg);
            if (kind == GMO_SGD) cfg[1] = variant ? 0.9f : 0.0f;
            if (kind == GMO_RMSPROP && variant) {
                cfg[4] = 0.9f;
                cfg[5] = 1.0f;
            }
            uintptr_t opt = gmo_optimizer_new(kind, cfg, kDims, kNdims, kTensors, mm, device);
            CHECK(opt != 0);
            if (!opt) continue;
            gmo_set_log_progress(opt, 0);
            uintptr_t w[kTensors], g[kTensors];
            for (int i = 0; i < kTensors; i++) {
                w[i] = gmo_allocate_buffer(mm, kSizes[i] * 4);
                g[i] = gmo_allocate_buffer(mm, kSizes[i] * 4);
                CHECK(w[i] && g[i]);
                CHECK(zero_metal_buffer(device, w[i], kSizes[i] * 4) == 0);
                CHECK(zero_metal_buffer(device, g[i], kSizes[i] * 4) == 0);
            }
            CHECK(gmo_set_weight_buffers(opt, w, kTensors) == 0);
            CHECK(gmo_set_weight_buffers(opt, w, kTensors - 1) != 0);
            for (int step = 0; step < 3; step++) CHECK(gmo_step(opt, g, kTensors) == 0);
            CHECK(gmo_step(opt, g, kTensors - 1) != 0);
            CHECK(gmo_get_step_count(opt) == 3);
            // the stand-in bumps every written element once per step
            for (int i = 0; i < kTensors; i++) {
                const std::vector<float> got = read_buffer(w[i], kSizes[i]);
                bool all3 = true;
                for (float x : got) all3 = all3 && x == 3.0f;
                CHECK(all3);
            }
            gmo_update_learning_rate(opt, 0.5f);
            (void)gmo_get_field(opt, "LearningRate");
            (void)gmo_get_field(opt, "NoSuchField");
            for (const char *k : state_kinds)
                for (int i = -1; i <= kTensors; i++) (void)gmo_state_buffer(opt, k, i);

            // checkpoint round trip into a second object
            const std::string js = take(gmo_get_state_json(opt));
            CHECK(!js.empty());
            const std::string ck = take(gmo_get_checkpoint_json(opt));
            CHECK(!ck.empty());
            uintptr_t other = gmo_optimizer_new(kind, cfg, kDims, kNdims, kTensors, mm, device);
            CHECK(other != 0);
            if (other) {
                gmo_set_log_progress(other, 0);
                CHECK(gmo_load_state_json(other, js.c_str()) == 0);
                CHECK(gmo_get_step_count(other) == 3);
                CHECK(gmo_load_checkpoint_json(other, ck.c_str()) == 0);
                CHECK(take(gmo_get_state_json(other)) == js);
                // a document for another optimizer type, truncated documents, wrong lengths
                CHECK(gmo_load_state_json(other, "{\"type\":\"Nope\",\"parameters\":{},\"state_data\":[]}") != 0);
                for (size_t cut = 0; cut < js.size(); cut += js.size() / 97 + 1)
                    (void)gmo_load_state_json(other, js.substr(0, cut).c_str());
                gmo_cleanup(other);
                gmo_cleanup(other);           // idempotent
                gmo_optimizer_free(other);
            }
            gmo_cleanup(opt);
            gmo_optimizer_free(opt);
            for (int i = 0; i < kTensors; i++) {
                gmo_release_buffer(mm, w[i]);
                gmo_release_buffer(mm, g[i]);
            }
        }
    }
}

static void mixed_precision(uintptr_t device, uintptr_t mm)
{
    float cfg[6];
    gmo_default_config(GMO_ADAM, cfg);
    uintptr_t opt = gmo_optimizer_new(GMO_ADAM, cfg, kDims, kNdims, kTensors, mm, device);
    CHECK(opt != 0);
    uintptr_t w[kTensors], g16[kTensors], w16[kTensors];
    for (int i = 0; i < kTensors; i++) {
        w[i] = gmo_allocate_buffer(mm, kSizes[i] * 4);
        g16[i] = gmo_allocate_buffer(mm, kSizes[i] * 2);
        w16[i] = gmo_allocate_buffer(mm, kSizes[i] * 2);
        zero_metal_buffer(device, w[i], kSizes[i] * 4);
        zero_metal_buffer(device, g16[i], kSizes[i] * 2);
        zero_metal_buffer(device, w16[i], kSizes[i] * 2);
    }
    CHECK(gmo_set_weight_buffers(opt, w, kTensors) == 0);
    int skipped = -1;
    CHECK(gmo_step_amp(opt, g16, w16, kTensors, &skipped) != 0);            // not enabled yet
    CHECK(gmo_enable_mixed_precision(opt, 65536.0f, 2.0f, 0.5f, 2) == 0);
    for (int step = 0; step < 4; step++) {
        CHECK(gmo_step_amp(opt, g16, w16, kTensors, &skipped) == 0 && skipped == 0);
    }
    CHECK(gmo_loss_scale(opt) == 4 * 65536.0f && gmo_growth_tracker(opt) == 0);
    uint16_t inf = 0x7C00;
    CHECK(copy_buffer_to_buffer_sync(g16[4], g16[4], 0, 0, 2) == 0);
    std::vector<int> words((size_t)(kSizes[4] * 2 + 3) / 4, 0);
    std::memcpy(reinterpret_cast<char *>(words.data()) + 2 * (kSizes[4] - 1), &inf, 2);
    CHECK(copy_int32_array_to_metal_buffer(g16[4], words.data(), (int)words.size()) == 0);
    CHECK(gmo_step_amp(opt, g16, w16, kTensors, &skipped) == 0 && skipped == 1);
    CHECK(gmo_loss_scale(opt) == 2 * 65536.0f);
    CHECK(gmo_get_step_count(opt) == 4);
    CHECK(gmo_step_amp_async(opt, g16, w16, kTensors) == 0);
    uint64_t dropped = 0;
    CHECK(gmo_sync_amp(opt, &dropped) == 0);
    const std::string js = take(gmo_get_state_json(opt));
    CHECK(js.find("loss_scale") != std::string::npos);
    CHECK(gmo_load_state_json(opt, js.c_str()) == 0);

    // the one-pass step over ping-pong state: clean gradients again
    CHECK(zero_metal_buffer(device, g16[4], kSizes[4] * 2) == 0);
    CHECK(gmo_current_set(opt) == 0);
    CHECK(gmo_enable_ping_pong(opt) == 0 && gmo_enable_ping_pong(opt) == 0);
    const uint64_t before = gmo_get_step_count(opt);
    CHECK(gmo_step_amp(opt, g16, w16, kTensors, &skipped) == 0 && skipped == 0 && gmo_current_set(opt) == 1);
    CHECK(gmo_state_buffer(opt, "weight", 0) != w[0] && gmo_state_buffer(opt, "weight", 0) != 0);
    CHECK(gmo_step_amp_async(opt, g16, w16, kTensors) == 0);
    CHECK(gmo_current_set(opt) == 0 && gmo_state_buffer(opt, "weight", 0) == w[0]);
    CHECK(gmo_get_step_count(opt) == before + 2);
    CHECK(copy_int32_array_to_metal_buffer(g16[4], words.data(), (int)words.size()) == 0);      // the inf again
    CHECK(gmo_step_amp(opt, g16, w16, kTensors, &skipped) == 0 && skipped == 1 && gmo_current_set(opt) == 0);
    const std::string js2 = take(gmo_get_state_json(opt));
    CHECK(!js2.empty() && gmo_load_state_json(opt, js2.c_str()) == 0);
    CHECK(gmo_step(opt, w, kTensors) == 0);                      // an fp32 step on the current set
    gmo_cleanup(opt);
    gmo_optimizer_free(opt);
    for (int i = 0; i < kTensors; i++) {
        gmo_release_buffer(mm, w[i]);
        gmo_release_buffer(mm, g16[i]);
        gmo_release_buffer(mm, w16[i]);
    }
}

extern "C" int cpu_device_requested_phase(uintptr_t buffer);      // cpu_device.cpp

// The state buffers of large tensors are asked for at the phases memory_manager.hpp names (512 KiB, 1.5 MiB,
// 1 MiB for the first, second and third state), small ones and the callers' own buffers at none, and a
// released state buffer goes back to the pool of its phase: the next optimizer gets the same handles.
static void state_buffer_phases(uintptr_t device, uintptr_t mm)
{
    const int dims[] = {1100, 1024, 17};            // 1126400 floats = 4.5 MB (the 16 MiB tier), and a small tensor
    const int ndims[] = {2, 1};
    float cfg[6] = {0};
    gmo_default_config(GMO_RMSPROP, cfg);
    cfg[4] = 0.9f;                                   // momentum
    cfg[5] = 1.0f;                                   // centered
    uintptr_t first_handles[3] = {0, 0, 0};
    const char *kinds[3] = {"squared_grad_avg", "momentum", "gradient_avg"};
    const int want[3] = {512 << 10, 1536 << 10, 1 << 20};
    for (int round = 0; round < 2; round++) {
        uintptr_t opt = gmo_optimizer_new(GMO_RMSPROP, cfg, dims, ndims, 2, mm, device);
        CHECK(opt != 0);
        if (!opt) return;
        for (int k = 0; k < 3; k++) {
            const uintptr_t big = gmo_state_buffer(opt, kinds[k], 0), small = gmo_state_buffer(opt, kinds[k], 1);
            CHECK(big != 0 && small != 0);
            CHECK(cpu_device_requested_phase(big) == want[k]);
            CHECK(cpu_device_requested_phase(small) == -1);
            if (round == 0) first_handles[k] = big;
            else CHECK(big == first_handles[k]);     // taken back from the pool of the same phase
        }
        gmo_cleanup(opt);
        gmo_optimizer_free(opt);
    }
    const uintptr_t plain = gmo_allocate_buffer(mm, 1100 * 1024 * 4);
    CHECK(plain != 0 && cpu_device_requested_phase(plain) == -1);
    for (int k = 0; k < 3; k++) CHECK(plain != first_handles[k]);    // the plain pool is another pool
    gmo_release_buffer(mm, plain);
    CHECK(gm_allocate_buffer_phased(device, 1 << 21, 1, 100) == 0);          // not a multiple of 256
    CHECK(gm_allocate_buffer_phased(device, 1 << 21, 1, 2 << 20) == 0);      // not below the period
}

static void json_documents()
{
    // What encoding/json accepts and refuses, and nothing that strtod alone would let through.
    struct Doc {
        const char *text;
        bool ok;
    } docs[] = {
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":1,\"b\":-0.5e-3,\"c\":true,\"d\":\"x\",\"e\":null},\"state_data\":[]}", true},
        {"{\"type\":\"Adam\",\"parameters\":{},\"state_data\":[{\"name\":\"momentum_0\",\"shape\":[3],\"data\":[1,2.5,-3e2],\"state_type\":\"momentum\"}]}", true},
        {"{\"type\":\"Adam\",\"parameters\":{},\"state_data\":null}", true},
        {"{\"type\":\"Adam\",\"parameters\":{},\"state_data\":[{\"name\":\"m\",\"shape\":[null],\"data\":[null],\"state_type\":\"momentum\"}]}", true},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":nan},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":-inf},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":Infinity},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":0x10},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":+1},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":01},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":1.},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":.5},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":1e},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"a\":1e400},\"state_data\":[]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{},\"state_data\":[{\"name\":\"m\",\"shape\":[1],\"data\":[1e39],\"state_type\":\"momentum\"}]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{},\"state_data\":[{\"name\":\"m\",\"shape\":[1.5],\"data\":[1],\"state_type\":\"momentum\"}]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{},\"state_data\":[{\"name\":\"m\",\"shape\":[1e10],\"data\":[1],\"state_type\":\"momentum\"}]}", false},
        {"{\"type\":\"Adam\",\"parameters\":{\"step_count\":-5},\"state_data\":[]}", true},
        {"{\"type\":\"Adam\",\"parameters\":{\"step_count\":1e300},\"state_data\":[]}", true},
        {"", false}, {"{", false}, {"[]", false}, {"{\"type\":\"Adam\"} x", false}, {"{\"type\":\"A\\u00", false},
        {"{\"type\":\"A\\", false}, {"{\"parameters\":{\"k\":[1,[2,{\"z\":[]}]]}}", true},
    };
    for (const Doc &d : docs) {
        char *out = gmo_state_json_normalize(d.text);
        if ((out != nullptr) != d.ok) {
            std::fprintf(stderr, "FAIL json document %s: %s (%s)\n", d.text, out ? "accepted" : "refused", gmo_last_error());
            g_failures++;
        }
        if (out) gmo_free_string(out);
    }
    // out-of-range counts saturate instead of invoking undefined conversions
    CHECK(gmo_extract_uint64_param("{\"step_count\":-5}", "step_count", 7) == 0);
    CHECK(gmo_extract_uint64_param("{\"step_count\":1e300}", "step_count", 7) == UINT64_MAX);
    CHECK(gmo_extract_uint64_param("{\"step_count\":12}", "step_count", 7) == 12);
    CHECK(gmo_extract_uint64_param("{\"other\":12}", "step_count", 7) == 7);
    CHECK(gmo_extract_float32_param("{\"lr\":0.25}", "lr", 1.0f) == 0.25f);
    CHECK(gmo_extract_bool_param("{\"n\":true}", "n", 0) == 1);
    CHECK(gmo_validate_state_type("Adam", "SGD") != 0 && gmo_validate_state_type("Adam", "Adam") == 0);
    const char *names[] = {"momentum_0", "variance_12", "x", "", "momentum_", "momentum_-3", "momentum_99999999999999999999", "_7"};
    for (const char *n : names) (void)gmo_extract_buffer_index(n);
    const int dims[] = {3, 4, 5};
    CHECK(gmo_calculate_tensor_size(dims, 3) == 60);
}

static void non_finite_state_is_refused(uintptr_t device, uintptr_t mm)
{
    float cfg[6];
    gmo_default_config(GMO_ADAGRAD, cfg);
    const int dims[] = {4}, ndims[] = {1};
    uintptr_t opt = gmo_optimizer_new(GMO_ADAGRAD, cfg, dims, ndims, 1, mm, device);
    CHECK(opt != 0);
    gmo_set_log_progress(opt, 0);
    float bad[4] = {1.0f, INFINITY, 2.0f, 3.0f};
    CHECK(copy_float32_array_to_metal_buffer(gmo_state_buffer(opt, "squared_grad_avg", 0), bad, 4) == 0);
    char *js = gmo_get_state_json(opt);
    CHECK(js == nullptr && std::strstr(gmo_last_error(), "unsupported value: +Inf") != nullptr);
    if (js) gmo_free_string(js);
    bad[1] = NAN;
    CHECK(copy_float32_array_to_metal_buffer(gmo_state_buffer(opt, "squared_grad_avg", 0), bad, 4) == 0);
    js = gmo_get_checkpoint_json(opt);
    CHECK(js == nullptr && std::strstr(gmo_last_error(), "unsupported value: NaN") != nullptr);
    if (js) gmo_free_string(js);
    gmo_cleanup(opt);
    gmo_optimizer_free(opt);
}

static void pools_and_tensors(uintptr_t device, uintptr_t mm)
{
    const int sizes[] = {1, 1023, 1024, 1025, 4096, 70000, 1 << 20, (1 << 26) + 5};
    std::vector<uintptr_t> held;
    for (int round = 0; round < 3; round++) {
        for (int s : sizes) {
            uintptr_t b = gmo_allocate_buffer(mm, s);
            CHECK(b != 0);
            CHECK(zero_metal_buffer(device, b, s) == 0);
            held.push_back(b);
            int a = 0, al = 0, mx = 0;
            (void)gmo_pool_stats(mm, gmo_find_pool_size(mm, s), &a, &al, &mx);
        }
        for (uintptr_t b : held) gmo_release_buffer(mm, b);
        held.clear();
    }
    gmo_release_buffer(mm, 0);
    for (int odd : {0, -4}) {          // AllocateBuffer rounds any size up to the smallest tier (manager.go:172-180)
        uintptr_t b = gmo_allocate_buffer(mm, odd);
        if (b) gmo_release_buffer(mm, b);
    }
    for (int s : {0, 1, 1024, 1 << 20, 1 << 30}) (void)gmo_calculate_max_pool_size(s), (void)gmo_reference_max_pool_size(s);

    const int shape[] = {3, 5};
    uintptr_t t = gmo_tensor_new(shape, 2, 0, 1);
    CHECK(t != 0 && gmo_tensor_size(t) == 60 && gmo_tensor_ref_count(t) == 1);
    float data[15], back[15];
    for (int i = 0; i < 15; i++) data[i] = (float)i * 0.5f - 3.0f;
    CHECK(gmo_tensor_copy_float32_data(t, data, 15) == 0);
    CHECK(gmo_tensor_copy_float32_data(t, data, 14) != 0);
    CHECK(gmo_tensor_to_float32_slice(t, back, 15) == 15 && std::memcmp(data, back, sizeof data) == 0);
    CHECK(gmo_tensor_to_float32_slice(t, back, 3) < 0);
    uintptr_t h = gmo_tensor_convert_to(t, 2);
    CHECK(h != 0 && gmo_tensor_dtype(h) == 2 && gmo_tensor_size(h) == 30);
    uintptr_t f = gmo_tensor_convert_to(h, 0);
    CHECK(f != 0 && gmo_tensor_to_float32_slice(f, back, 15) == 15 && std::memcmp(data, back, sizeof data) == 0);
    CHECK(gmo_tensor_convert_to(t, 3) == 0);
    uintptr_t same = gmo_tensor_convert_to(t, 0);
    CHECK(same == t && gmo_tensor_ref_count(t) == 2);
    gmo_tensor_release(same);
    uintptr_t u = gmo_tensor_new(shape, 2, 0, 1);
    CHECK(gmo_tensor_copy_from(u, t) == 0 && gmo_tensor_copy_from(u, h) != 0);
    CHECK(!take(gmo_tensor_string(t)).empty());
    CHECK(gmo_tensor_retain(t) == t);
    gmo_tensor_release(t);
    for (uintptr_t x : {t, h, f, u}) {
        gmo_tensor_release(x);
        CHECK(gmo_tensor_retain(x) == 0);
        gmo_tensor_release(x);            // releasing a dead tensor is harmless
        gmo_tensor_free(x);
    }
    const int bad_shape[] = {3, -1};
    CHECK(gmo_tensor_new(bad_shape, 2, 0, 1) == 0);
    CHECK(gmo_calculate_size(shape, 2, 2) == 30 && gmo_calculate_size(shape, 2, 9) < 0);

    // engine call site: tensors -> handles -> SetWeightBuffers -> Step
    float cfg[6];
    gmo_default_config(GMO_ADAM, cfg);
    const int ndims[] = {2};
    uintptr_t opt = gmo_optimizer_new(GMO_ADAM, cfg, shape, ndims, 1, mm, device);
    uintptr_t wt = gmo_tensor_new(shape, 2, 0, 1), gt = gmo_tensor_new(shape, 2, 0, 1);
    CHECK(gmo_tensor_copy_float32_data(wt, data, 15) == 0 && gmo_tensor_copy_float32_data(gt, data, 15) == 0);
    CHECK(gmo_execute_step_with_precomputed_gradients(opt, &wt, 1, &gt, 1) == 0);
    uintptr_t nil = 0;
    CHECK(gmo_execute_step_with_precomputed_gradients(opt, &nil, 1, &gt, 1) != 0);
    CHECK(gmo_execute_step_with_precomputed_gradients(opt, &wt, 1, &gt, 0) != 0);
    gmo_cleanup(opt);
    gmo_optimizer_free(opt);
    for (uintptr_t x : {wt, gt}) {
        gmo_tensor_release(x);
        gmo_tensor_free(x);
    }
}

static void lbfgs(uintptr_t device, uintptr_t mm)
{
    int hs, mls;
    float tol, c1, c2, step;
    gmo_lbfgs_default_config(&hs, &tol, &mls, &c1, &c2, &step);
    uintptr_t o = gmo_lbfgs_new(4, tol, mls, c1, c2, step, kDims, kNdims, kTensors, mm, device);
    CHECK(o != 0);
    gmo_lbfgs_set_log_progress(o, 0);
    uintptr_t w[kTensors], g[kTensors];
    for (int i = 0; i < kTensors; i++) {
        w[i] = gmo_allocate_buffer(mm, kSizes[i] * 4);
        g[i] = gmo_allocate_buffer(mm, kSizes[i] * 4);
        zero_metal_buffer(device, w[i], kSizes[i] * 4);
        zero_metal_buffer(device, g[i], kSizes[i] * 4);
    }
    CHECK(gmo_lbfgs_step(o, g, kTensors, 1.0f) != 0);                // weights not set; counted all the same (lbfgs.go:251)
    CHECK(gmo_lbfgs_set_weight_buffers(o, w, kTensors) == 0);
    for (int s = 0; s < 7; s++) CHECK(gmo_lbfgs_step(o, g, kTensors, 1.0f / (float)(s + 1)) == 0);
    CHECK(gmo_lbfgs_get_step(o) == 8);
    uint64_t st;
    int a, b;
    float loss;
    gmo_lbfgs_get_stats(o, &st, &a, &b, &loss);
    gmo_lbfgs_history(o, &a, &b, &loss);
    CHECK(gmo_lbfgs_update_learning_rate(o, 0.1f) != 0);
    for (int i = -1; i <= kTensors; i++) (void)gmo_lbfgs_buffer_size(o, i);
    for (const char *which : {"s", "y", "rho", "alpha", "old_gradient", "search_dir", "weight", "nope"})
        for (int h = -1; h <= 4; h++)
            for (int i = -1; i <= kTensors; i++) (void)gmo_lbfgs_buffer(o, which, h, i);
    gmo_lbfgs_cleanup(o);
    gmo_lbfgs_cleanup(o);
    gmo_lbfgs_free(o);
    for (int i = 0; i < kTensors; i++) {
        gmo_release_buffer(mm, w[i]);
        gmo_release_buffer(mm, g[i]);
    }
}

static void schedulers()
{
    for (int kind = 0; kind <= 4; kind++) {
        uintptr_t s = gmo_scheduler_new(kind, kind == 3 ? 2 : 5, 0.5, 1e-4, kind == 3 ? "max" : nullptr);
        CHECK(s != 0);
        for (int e = 0; e < 12; e++) {
            const double lr = gmo_scheduler_get_lr(s, e, 0, 0.1);
            CHECK(std::isfinite(lr));
            (void)gmo_scheduler_plateau_step(s, 1.0 / (e + 1), lr);
        }
        CHECK(gmo_scheduler_name(s) != nullptr);
        (void)gmo_scheduler_apply(s, 0, 3, 0, 0.1);
        gmo_scheduler_free(s);
    }
    CHECK(gmo_scheduler_new(99, 0, 0, 0, nullptr) == 0);
}

int main()
{
    const uintptr_t device = create_metal_device();
    gmo_initialize_global_memory_manager(device);
    const uintptr_t mm = gmo_get_global_memory_manager();
    CHECK(mm != 0);
    json_documents();
    optimizers(device, mm);
    mixed_precision(device, mm);
    non_finite_state_is_refused(device, mm);
    pools_and_tensors(device, mm);
    state_buffer_phases(device, mm);
    lbfgs(device, mm);
    schedulers();
    uintptr_t own = gmo_memory_manager_new(device);
    CHECK(own != 0);
    uintptr_t b = gmo_allocate_buffer(own, 5000);
    gmo_release_buffer(own, b);
    gmo_memory_manager_free(own);
    std::printf("host_mirror_driver: %d failures\n", g_failures);
    return g_failures == 0 ? 0 : 1;
}
