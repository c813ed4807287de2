// The reference's own tests for the optimizer step (nabla-train/tests/optim.rs:47-138,
// nabla-train/tests/trainer.rs:171-203), replayed through the C++ mirror of its
// interface (include/nabla_optim.hpp) on the device: f64, 1x1 tensors, the same
// values and the same assertions.  Exit code 0 = all passed.  With a directory as its
// argument the checkpoint test writes there (and leaves the files for the caller).
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

#include "../../include/nabla_checkpoint.hpp"
#include "../../include/nabla_groups.hpp"

using namespace nabla::optim;

static int failures = 0;
#define EXPECT(cond)                                                                   \
    do {                                                                               \
        if (!(cond)) {                                                                 \
            std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);            \
            failures++;                                                                \
        }                                                                              \
    } while (0)

// mat![[v]] on the device
struct Mat {
    double *d = nullptr;
    uint64_t n;
    explicit Mat(std::vector<double> v) : n(v.size())
    {
        if (hipMalloc((void **)&d, n * sizeof(double)) != hipSuccess) std::abort();
        if (hipMemcpy(d, v.data(), n * sizeof(double), hipMemcpyHostToDevice) != hipSuccess) std::abort();
    }
    ~Mat() { (void)hipFree(d); }
    Tensor tensor() const { return Tensor{d, 1, n, NBO_DT_F64}; }
    double get(uint64_t i = 0) const
    {
        sync();
        double x;
        if (hipMemcpy(&x, d + i, sizeof(double), hipMemcpyDeviceToHost) != hipSuccess) std::abort();
        return x;
    }
};

static void sgd_step_updates_param()  // optim.rs:47-57
{
    Mat param({1.0}), grad({1.0});
    Sgd opt(0.1, {{1, 1}}, NBO_DT_F64);
    opt.step({param.tensor()}, {grad.tensor()});
    EXPECT(std::fabs(param.get() - 0.9) < 1e-10);
}

static void step_with_vars_pulls_params_and_grads()  // optim/core.rs:18-39 on the same values
{
    Mat param({1.0}), grad({1.0});
    struct Module {
        std::vector<Tensor> p;
        std::vector<Tensor> parameters_mut() { return p; }
    } module{{param.tensor()}};
    struct Var {
        Tensor g;
        bool has;
        const Tensor *grad() const { return has ? &g : nullptr; }
    };
    Sgd opt(0.1, {{1, 1}}, NBO_DT_F64);
    opt.step_with_vars(module, std::vector<Var>{{grad.tensor(), true}});
    EXPECT(std::fabs(param.get() - 0.9) < 1e-10);
    bool panicked = false;
    try {
        opt.step_with_vars(module, std::vector<Var>{{grad.tensor(), false}});
    } catch (const Panic &e) {
        panicked = std::string(e.what()).find("param_vars[0] has no gradient (call backward first)") != std::string::npos;
    }
    EXPECT(panicked);
    panicked = false;
    try {
        opt.step_with_vars(module, std::vector<Var>{});
    } catch (const Panic &e) {
        panicked = std::string(e.what()).find("param_vars length (0) doesn't match module parameters count (1)") !=
                   std::string::npos;
    }
    EXPECT(panicked);
    EXPECT(std::fabs(param.get() - 0.9) < 1e-10);
}

static void adam_step_updates_param()  // optim.rs:59-69
{
    Mat param({1.0}), grad({1.0});
    Adam opt(0.1, {{1, 1}}, NBO_DT_F64);
    opt.step({param.tensor()}, {grad.tensor()});
    EXPECT(param.get() < 1.0);
    EXPECT(std::fabs(param.get() - 0.9) < 1e-7);  // step 1 from m = v = 0 is sign-SGD
    EXPECT(opt.step_count() == 1);
}

static void adamw_step_updates_param()  // optim.rs:71-81
{
    Mat param({1.0}), grad({1.0});
    AdamW opt(0.1, {{1, 1}}, NBO_DT_F64);
    opt.step({param.tensor()}, {grad.tensor()});
    EXPECT(param.get() < 1.0);
    EXPECT(std::fabs(param.get() - 0.899) < 1e-7);  // default weight_decay 0.01
}

static void grad_scaler_unscale()  // optim.rs:120-128
{
    GradScaler scaler;
    Mat g({2.0});
    TensorList grads({g.tensor()});
    EXPECT(scaler.unscale_and_update(grads));
    EXPECT(g.get() < 2.0);
    EXPECT(g.get() == 2.0 / 65536.0);
    Mat loss({0.75}), scaled({0.0});  // scale_loss, core.rs:347-349
    TensorList l({loss.tensor()}), o({scaled.tensor()});
    scaler.scale_loss(l, o);
    EXPECT(scaled.get() == 0.75 * 65536.0);
}

static void grad_scaler_detects_inf()  // optim.rs:130-138
{
    GradScaler scaler;
    Mat g({std::numeric_limits<double>::infinity()});
    TensorList grads({g.tensor()});
    EXPECT(!scaler.unscale_and_update(grads));
    EXPECT(std::fabs(g.get()) < 1e-12);
    EXPECT(scaler.scale_factor() == 32768.0);
    EXPECT(scaler.state().consecutive_ok == 0);
}

static void clip_grad_norm_scales()  // trainer.rs:171-203
{
    Mat a({3.0}), b({4.0});
    TensorList grads({a.tensor(), b.tensor()});
    const double reported = clip_grad_norm(grads, 2.5);
    const double after = std::sqrt(a.get() * a.get() + b.get() * b.get());
    EXPECT(std::fabs(reported - 5.0) < 1e-10);
    EXPECT(std::fabs(after - 2.5) < 1e-10);
    EXPECT(clip_grad_norm(grads, 0.0) == 0.0);  // trainer.rs:501-503
}

static void weight_decay_exclusion()  // optim.rs:140-165
{
    Mat weight({2.0}), bias({3.0}), zero_w({0.0}), zero_b({0.0});
    const std::vector<std::pair<std::string, Tensor>> named = {{"weight", weight.tensor()}, {"bias", bias.tensor()}};
    const ParamGroupConfig bias_group =
        ParamGroupConfig::sgd("no_decay", ParamSelector::Any({{ParamMatch::Suffix, "bias"}}), 1.0, 0.0, 0.0);
    const ParamGroupConfig decay_group = ParamGroupConfig::sgd("decay", ParamSelector::All(), 1.0, 0.0, 0.1);
    GroupOptimizer opt = GroupOptimizer::from_named_params(named, {bias_group}, &decay_group, NBO_DT_F64);
    EXPECT(opt.groups() == 2 && opt.group_indices(0) == std::vector<size_t>{1} && opt.group_indices(1) == std::vector<size_t>{0});
    opt.step({weight.tensor(), bias.tensor()}, {zero_w.tensor(), zero_b.tensor()});
    EXPECT(std::fabs(weight.get() - 1.8) < 1e-10);
    EXPECT(std::fabs(bias.get() - 3.0) < 1e-10);
    // set_lr keeps the groups' proportions (groups.rs:302-312); the fused tail decides once for all
    opt.set_lr(0.5);
    opt.fused_step({weight.tensor(), bias.tensor()}, {zero_w.tensor(), zero_b.tensor()}, nullptr, 1.0);
    EXPECT(std::fabs(weight.get() - 1.8 * (1.0 - 0.5 * 0.1)) < 1e-12);
    EXPECT(std::fabs(bias.get() - 3.0) < 1e-10);
    bool refused = false;
    try {
        GroupOptimizer::from_named_params(named, {bias_group}, nullptr, NBO_DT_F64);
    } catch (const StateError &e) {
        refused = std::string(e.what()) == "nabla-train: group assignment incomplete";
    }
    EXPECT(refused);
}

static void lr_schedules()  // optim.rs:83-118
{
    const LrSchedule lin = LrSchedule::linear(0, 10);
    EXPECT(std::fabs(lr_at_step(lin, 1.0, 0) - 1.0) < 1e-10);
    EXPECT(lr_at_step(lin, 1.0, 10) <= 1e-10);
    const LrSchedule stp = LrSchedule::step(2, 0.1);
    EXPECT(std::fabs(lr_at_step(stp, 1.0, 0) - 1.0) < 1e-10);
    EXPECT(std::fabs(lr_at_step(stp, 1.0, 2) - 0.1) < 1e-10);
    EXPECT(std::fabs(lr_at_step(stp, 1.0, 4) - 0.01) < 1e-10);
    const LrSchedule one = LrSchedule::one_cycle(1.0, 10, 0.5);
    EXPECT(lr_at_step(one, 0.1, 3) > 0.1);
    const LrSchedule cosine = LrSchedule::cosine(10, 110, 0.1);  // closed forms: ramp, mid-point, end
    EXPECT(std::fabs(lr_at_step(cosine, 1.0, 5) - 0.5) < 1e-12);
    EXPECT(std::fabs(lr_at_step(cosine, 1.0, 60) - 0.55) < 1e-12);
    EXPECT(std::fabs(lr_at_step(cosine, 1.0, 110) - 0.1) < 1e-12);
}

static void nan_policy_skip_drops_step()  // trainer.rs tests :148-169
{
    Mat w({1.0}), buf({0.0}), nan_grad({std::numeric_limits<double>::quiet_NaN()}), good({1.0});
    Sgd opt(0.1, {{1, 1}}, NBO_DT_F64);
    TensorList params({w.tensor()}), accum({buf.tensor()}), bad({nan_grad.tensor()}), ok({good.tensor()});
    TrainerTail trainer(opt, params, accum);
    trainer.with_nan_policy(GradNanPolicy::Skip);
    EXPECT(!trainer.after_backward(bad));
    EXPECT(trainer.step() == 0 && w.get() == 1.0);
    EXPECT(trainer.after_backward(ok));  // and a finite gradient afterwards steps
    EXPECT(trainer.step() == 1 && std::fabs(w.get() - 0.9) < 1e-12);
    TrainerTail stopper(opt, params, accum);
    stopper.with_nan_policy(GradNanPolicy::Stop);
    bool raised = false;
    try {
        stopper.after_backward(bad);
    } catch (const TrainError &e) {
        raised = std::string(e.what()) == "non-finite gradient";
    }
    EXPECT(raised);
}

static void trainer_accumulates_then_clips_and_steps()  // trainer.rs:253-291 on hand-checked values
{
    Mat w({1.0}), buf({0.0}), g1({3.0}), g2({5.0});
    Sgd opt(0.5, {{1, 1}}, NBO_DT_F64);
    TensorList params({w.tensor()}), accum({buf.tensor()}), a({g1.tensor()}), b({g2.tensor()});
    TrainerTail trainer(opt, params, accum);
    trainer.with_grad_accum(2).with_grad_clip(4.0).with_schedule(LrSchedule::step(1, 0.5), 0.5);
    EXPECT(!trainer.after_backward(a));
    EXPECT(buf.get() == 3.0 && w.get() == 1.0);
    EXPECT(trainer.after_backward(b));  // buf = 8, clipped to 4, lr(step 0) = 0.5: w = 1 - 0.5 * 4
    EXPECT(std::fabs(w.get() + 1.0) < 1e-12 && buf.get() == 0.0 && trainer.step() == 1);
    EXPECT(!trainer.after_backward(a));
    EXPECT(trainer.after_backward(a));  // buf = 6 -> 4, lr(step 1) = 0.25: w = -1 - 0.25 * 4
    EXPECT(std::fabs(w.get() + 2.0) < 1e-12 && trainer.step() == 2);
}

static void backend_axpy_is_multiply_then_add()  // cpu/mod.rs:216-223
{
    Mat y({1.0, 0.1}), x({3.0, 0.3});
    TensorList ly({y.tensor()}), lx({x.tensor()});
    backend::axpy_inplace(ly, 0.1, lx);
    EXPECT(y.get(0) == 1.0 + 0.1 * 3.0);
    const double prod = 0.1 * 0.3;  // rounded product, then rounded sum
    EXPECT(y.get(1) == 0.1 + prod);
}

static std::string g_checkpoint_dir;

static void checkpoint_roundtrip_with_schedule()  // trainer.rs tests :249-304
{
    std::string dir = g_checkpoint_dir;
    if (dir.empty()) {
        char tmpl[] = "/tmp/nbo_ckpt_XXXXXX";
        const char *made = mkdtemp(tmpl);
        EXPECT(made != nullptr);
        dir = made ? made : "/tmp";
    }
    Mat w({1.5}), b({-0.5});
    TensorList module({w.tensor(), b.tensor()});
    const std::vector<std::string> names = {"w", "b"};
    Sgd opt(0.1, {{1, 1}, {1, 1}}, NBO_DT_F64);
    GradScaler scaler;
    const ScheduleState schedule{0.1, LrSchedule::step(1, 0.9)};
    TrainState state;
    state.epoch = 2, state.step = 3, state.grad_accum = 1, state.rng_state = 42;
    save_checkpoint(dir, module, names, opt, &scaler, &schedule, state);

    Mat w2({0.0}), b2({0.0});
    TensorList module2({w2.tensor(), b2.tensor()});
    Sgd opt2(0.7, {{1, 1}, {1, 1}}, NBO_DT_F64);
    GradScaler scaler2;
    scaler2.load_state(GradScalerState{1.0, 3.0, 0.25, 7, 5});
    TrainState state2;
    std::optional<ScheduleState> schedule2;
    load_checkpoint(dir, module2, names, opt2, &scaler2, schedule2, state2);
    EXPECT(state2.epoch == 2);
    EXPECT(state2.step == 3);
    EXPECT(state2.rng_state && *state2.rng_state == 42);
    EXPECT(schedule2.has_value());
    EXPECT(schedule2 && schedule2->base_lr == 0.1 && schedule2->schedule.kind == LrSchedule::Step &&
           schedule2->schedule.step_size == 1 && schedule2->schedule.gamma == 0.9);
    EXPECT(w2.get() == 1.5 && b2.get() == -0.5);
    EXPECT(opt2.lr() == 0.1 && scaler2.scale_factor() == 65536.0 && scaler2.state().growth_interval == 2000);
    // Rust's f64 Display, which meta.txt is written with
    EXPECT(rust_f64_str(0.1) == "0.1" && rust_f64_str(65536.0) == "65536" && rust_f64_str(1e-8) == "0.00000001");
    EXPECT(rust_f64_str(1e21) == "1000000000000000000000" && rust_f64_str(-2.5) == "-2.5" && rust_f64_str(0.0) == "0");
    // a checkpoint of another optimizer kind is refused with the reference's error
    Adam other(0.1, {{1, 1}, {1, 1}}, NBO_DT_F64);
    std::string what;
    try {
        load_checkpoint(dir, module2, names, other, nullptr, schedule2, state2);
    } catch (const CheckpointError &e) {
        what = e.what();
    }
    EXPECT(what.find("missing m0") != std::string::npos || what.find("optim kind mismatch") != std::string::npos);
}

// A bf16 tensor on the device, filled from floats (rounded to nearest even by the library's cast).
struct HalfVec {
    uint16_t *d = nullptr;
    uint64_t n;
    explicit HalfVec(uint64_t n_) : n(n_)
    {
        if (hipMalloc((void **)&d, n * sizeof(uint16_t)) != hipSuccess) std::abort();
        if (hipMemset(d, 0, n * sizeof(uint16_t)) != hipSuccess) std::abort();
    }
    ~HalfVec() { (void)hipFree(d); }
    Tensor tensor() const { return Tensor{d, 1, n, NBO_DT_BF16}; }
    void put(const std::vector<uint16_t> &bits)
    {
        if (hipMemcpy(d, bits.data(), n * sizeof(uint16_t), hipMemcpyHostToDevice) != hipSuccess) std::abort();
    }
    std::vector<uint16_t> get() const
    {
        sync();
        std::vector<uint16_t> v(n);
        if (hipMemcpy(v.data(), d, n * sizeof(uint16_t), hipMemcpyDeviceToHost) != hipSuccess) std::abort();
        return v;
    }
};

// Checkpoint of a mixed-precision optimizer (bf16 tensors over f32 master weights; the
// reference has no such optimizer, the file formats are checkpoint.rs:38-150's): the master
// weights travel as an f32 params.nbla, and training resumed from the files continues with the
// bits of the run that was never interrupted.
static void mixed_precision_checkpoint_resumes_bit_for_bit()
{
    std::string dir = g_checkpoint_dir;
    if (dir.empty()) {
        char tmpl[] = "/tmp/nbo_ckpt_XXXXXX";
        const char *made = mkdtemp(tmpl);
        EXPECT(made != nullptr);
        dir = made ? made : "/tmp";
    }
    dir += "/mixed";
    const uint64_t n0 = 8192 + 37, n1 = 300;
    const Shapes shapes = {{1, n0}, {1, n1}};
    const std::vector<std::string> names = {"layer.w", "layer.b"};
    auto fill = [](uint64_t n, uint32_t seed, uint16_t exp_bits) { // bf16 bit patterns of moderate size, both signs
        std::vector<uint16_t> v(n);
        uint32_t x = seed;
        for (auto &e : v) {
            x = x * 1664525u + 1013904223u;
            e = (uint16_t)(((x >> 16) & 0x807f) | exp_bits);
        }
        return v;
    };
    HalfVec p0(n0), p1(n1), g0(n0), g1(n1);
    p0.put(fill(n0, 1, 0x3c00)), p1.put(fill(n1, 2, 0x3c00));
    TensorList params({p0.tensor(), p1.tensor()}), grads({g0.tensor(), g1.tensor()});
    AdamW opt(2e-4, shapes, NBO_DT_F32, /*master=*/true);
    opt.beta2(0.95).weight_decay(0.1);
    opt.master_from_params(params);
    GradScaler scaler;
    auto step = [&](AdamW &o, GradScaler &sc, TensorList &p, uint32_t k) {
        g0.put(fill(n0, 100 + k, 0x4300)), g1.put(fill(n1, 200 + k, 0x4300)); // about 128..256: times 1/65536 after unscale
        o.fused_step(p, grads, &sc, 1.0);
    };
    for (uint32_t k = 0; k < 3; k++) step(opt, scaler, params, k);
    TrainState state;
    state.epoch = 0, state.step = 3, state.grad_accum = 1;
    save_checkpoint(dir, params, names, opt, &scaler, nullptr, state);

    HalfVec q0(n0), q1(n1);
    TensorList params2({q0.tensor(), q1.tensor()});
    AdamW opt2(1.0, shapes, NBO_DT_F32, /*master=*/true);
    GradScaler scaler2;
    TrainState state2;
    std::optional<ScheduleState> schedule2;
    load_checkpoint(dir, params2, names, opt2, &scaler2, schedule2, state2);
    EXPECT(state2.step == 3 && !schedule2.has_value());
    EXPECT(q0.get() == p0.get() && q1.get() == p1.get()); // narrowed from the restored master weights
    for (uint32_t k = 3; k < 5; k++) {
        step(opt, scaler, params, k);
        step(opt2, scaler2, params2, k);
    }
    EXPECT(q0.get() == p0.get() && q1.get() == p1.get());
    for (const char *key : {"w0", "m0", "v0", "w1", "m1", "v1"}) {
        const uint64_t n = key[1] == '0' ? n0 : n1;
        std::vector<float> a(n), b(n);
        opt.state_read(key, a.data(), n, false);
        opt2.state_read(key, b.data(), n, false);
        EXPECT(std::memcmp(a.data(), b.data(), n * sizeof(float)) == 0);
    }
    EXPECT(opt.last_step().step_count == 5 && opt2.last_step().step_count == 5);
    // a file key the module does not have is load_state_dict's error (module/core.rs:42, 286-290)
    std::string what;
    try {
        load_checkpoint(dir, params2, {"layer.w", "other.b"}, opt2, &scaler2, schedule2, state2);
    } catch (const std::exception &e) {
        what = e.what();
    }
    EXPECT(what.find("unknown parameter key: layer.b") != std::string::npos);
}

// The same for a GroupOptimizer whose groups keep master weights: params.nbla holds every group's
// f32 master weights in the module's order under the parameters' names, the restored groups'
// 16-bit tensors are narrowed from them, and training goes on with the uninterrupted run's bits.
static void group_mixed_precision_checkpoint_resumes_bit_for_bit()
{
    if (g_checkpoint_dir.empty()) return;
    const std::string dir = g_checkpoint_dir + "/groups_mixed";
    const uint64_t nw = 8192 + 37, nb = 300, nn = 64;
    const std::vector<std::string> names = {"layer.w", "layer.bias", "layer.norm"};
    auto fill = [](uint64_t n, uint32_t seed, uint16_t exp_bits) {
        std::vector<uint16_t> v(n);
        uint32_t x = seed;
        for (auto &e : v) {
            x = x * 1664525u + 1013904223u;
            e = (uint16_t)(((x >> 16) & 0x807f) | exp_bits);
        }
        return v;
    };
    HalfVec pw(nw), pb(nb), pn(nn), gw(nw), gb(nb), gn(nn);
    pw.put(fill(nw, 1, 0x3c00)), pb.put(fill(nb, 2, 0x3c00)), pn.put(fill(nn, 3, 0x3c00));
    auto make = [&](const std::vector<Tensor> &t) {
        return GroupOptimizer::adamw_with_decay_exclusions({{names[0], t[0]}, {names[1], t[1]}, {names[2], t[2]}}, 2e-4, 0.1,
                                                           {"bias", "norm"}, NBO_DT_F32, /*master=*/true);
    };
    const std::vector<Tensor> params = {pw.tensor(), pb.tensor(), pn.tensor()};
    const std::vector<Tensor> grads = {gw.tensor(), gb.tensor(), gn.tensor()};
    GroupOptimizer opt = make(params);
    EXPECT(opt.groups() == 2 && opt.keeps_master() && (opt.group_indices(0) == std::vector<size_t>{1, 2}));
    for (size_t g = 0; g < opt.groups(); g++) {
        std::vector<Tensor> mine;
        for (size_t i : opt.group_indices(g)) mine.push_back(params[i]);
        TensorList l(mine);
        opt.group_optimizer(g).master_from_params(l);
    }
    GradScaler scaler;
    auto step = [&](GroupOptimizer &o, GradScaler &sc, const std::vector<Tensor> &p, uint32_t k) {
        gw.put(fill(nw, 100 + k, 0x4300)), gb.put(fill(nb, 200 + k, 0x4300)), gn.put(fill(nn, 300 + k, 0x4300));
        o.fused_step(p, grads, &sc, 1.0);
    };
    for (uint32_t k = 0; k < 3; k++) step(opt, scaler, params, k);
    TensorList module(params);
    TrainState state;
    state.epoch = 0, state.step = 3, state.grad_accum = 1;
    save_checkpoint(dir, module, names, opt, &scaler, nullptr, state);

    HalfVec qw(nw), qb(nb), qn(nn);
    const std::vector<Tensor> params2 = {qw.tensor(), qb.tensor(), qn.tensor()};
    GroupOptimizer opt2 = make(params2);
    TensorList module2(params2);
    GradScaler scaler2;
    TrainState state2;
    std::optional<ScheduleState> schedule2;
    load_checkpoint(dir, module2, names, opt2, &scaler2, schedule2, state2);
    EXPECT(state2.step == 3 && !schedule2.has_value());
    EXPECT(qw.get() == pw.get() && qb.get() == pb.get() && qn.get() == pn.get()); // narrowed from the master weights
    for (uint32_t k = 3; k < 5; k++) {
        step(opt, scaler, params, k);
        step(opt2, scaler2, params2, k);
    }
    EXPECT(qw.get() == pw.get() && qb.get() == pb.get() && qn.get() == pn.get());
    for (size_t g = 0; g < opt.groups(); g++)
        for (const char *key : {"w0", "m0", "v0"}) {
            const uint64_t n = g == 0 ? nb : nw;
            std::vector<float> a(n), b(n);
            opt.group_optimizer(g).state_read(key, a.data(), n, false);
            opt2.group_optimizer(g).state_read(key, b.data(), n, false);
            EXPECT(std::memcmp(a.data(), b.data(), n * sizeof(float)) == 0);
        }
    EXPECT(opt.group_optimizer(1).last_step().step_count == 5 && opt2.group_optimizer(1).last_step().step_count == 5);
    // the file is checked as a whole before anything is written: a key the module does not have
    std::string what;
    try {
        load_checkpoint(dir, module2, {"layer.w", "layer.bias", "other.norm"}, opt2, &scaler2, schedule2, state2);
    } catch (const std::exception &e) {
        what = e.what();
    }
    EXPECT(what.find("unknown parameter key: layer.norm") != std::string::npos);
}

static void panics_and_errors()  // alg.rs:110-119, 531-545; tensor/ops.rs:638-646
{
    Mat p({1.0}), g({1.0}), g2({1.0, 2.0});
    AdamW opt(0.1, {{1, 1}}, NBO_DT_F64);
    std::string what;
    try {
        opt.step({p.tensor()}, {g.tensor(), g.tensor()});
    } catch (const Panic &e) {
        what = e.what();
    }
    EXPECT(what == "nabla-train: AdamW params/grads length mismatch");
    what.clear();
    try {
        opt.step({p.tensor(), p.tensor()}, {g.tensor(), g.tensor()});
    } catch (const Panic &e) {
        what = e.what();
    }
    EXPECT(what == "nabla-train: AdamW params count mismatch");
    what.clear();
    try {
        opt.step({p.tensor()}, {g2.tensor()});
    } catch (const Panic &e) {
        what = e.what();
    }
    EXPECT(what.find("shapes must match") != std::string::npos);
    what.clear();
    try {
        opt.load_meta(OptimMeta{OptimKind::Sgd, 0.1, 0, 0, 0, 0, 0, 0});
    } catch (const StateError &e) {
        what = e.what();
    }
    EXPECT(what == "optim kind mismatch");
    what.clear();
    double buf = 0;
    try {
        opt.state_read("m7", &buf, 1, false);
    } catch (const StateError &e) {
        what = e.what();
    }
    EXPECT(what == "m index out of range: 7");
    what.clear();
    try {
        opt.state_read("mx", &buf, 1, false);
    } catch (const StateError &e) {
        what = e.what();
    }
    EXPECT(what == "bad tensor key: mx");
    EXPECT(p.get() == 1.0);  // nothing ran
    // addresses are checked against what the HIP runtime knows before any kernel sees them
    double on_host = 0.0;
    what.clear();
    try {
        TensorList bad({Tensor{&on_host, 1, 1, NBO_DT_F64}});
    } catch (const RuntimeError &e) {
        what = e.what();
    }
    EXPECT(what.find("not memory the HIP runtime knows") != std::string::npos);
    what.clear();
    try {
        TensorList bad({Tensor{g2.d, 1, 3, NBO_DT_F64}});  // a 2-element allocation described as 3 elements
    } catch (const RuntimeError &e) {
        what = e.what();
    }
    EXPECT(what.find("do not fit the allocation") != std::string::npos);
    TensorList fits({Tensor{g2.d + 1, 1, 1, NBO_DT_F64}});  // an interior address that ends inside
}

static void decay_presets_and_known_norm_group_step()  // groups.rs:134-150, 244-261
{
    Mat e({1.0}), w({2.0}), b({3.0}), ln({4.0}), ge({0.0}), gw({3.0}), gb({4.0}), gl({0.0});
    const std::vector<std::pair<std::string, Tensor>> named = {
        {"embed.table", e.tensor()}, {"l0.weight", w.tensor()}, {"l0.bias", b.tensor()}, {"l0.ln", ln.tensor()}};
    GroupOptimizer opt = GroupOptimizer::adamw_with_decay_presets(
        named, 0.1, 0.5, {ParamExclusionPreset::Bias, ParamExclusionPreset::Norm, ParamExclusionPreset::Embedding},
        NBO_DT_F64);
    EXPECT(opt.groups() == 2 && (opt.group_indices(0) == std::vector<size_t>{0, 2, 3}) &&
           (opt.group_indices(1) == std::vector<size_t>{1}));
    // gradients (0, 3, 4, 0): norm 5, clipped to 2.5 -> (1.5, 2); first AdamW step moves by lr * sign(g)
    const std::vector<Tensor> params = {e.tensor(), w.tensor(), b.tensor(), ln.tensor()};
    const std::vector<Tensor> grads = {ge.tensor(), gw.tensor(), gb.tensor(), gl.tensor()};
    opt.fused_step_norm(params, grads, 25.0, 2.5);
    EXPECT(e.get() == 1.0 && ln.get() == 4.0);                    // no gradient, no decay
    EXPECT(std::fabs(b.get() - (3.0 - 0.1)) < 1e-6);              // no decay
    EXPECT(std::fabs(w.get() - (2.0 * (1.0 - 0.05) - 0.1)) < 1e-6);  // decayed by lr * wd
    const nbo_step_info info = opt.group_optimizer(0).last_step();
    EXPECT(info.norm == 5.0 && info.clipped == 1 && info.step_count == 1);
}

static void group_checkpoint_roundtrip()  // checkpoint.rs:38-105 with groups.rs:320-420 as the OptimState
{
    if (g_checkpoint_dir.empty()) return;
    const std::string dir = g_checkpoint_dir + "/groups";
    Mat w({2.0, -1.0}), b({3.0}), gw({0.5, 0.25}), gb({1.0});
    const std::vector<std::pair<std::string, Tensor>> named = {{"l.weight", w.tensor()}, {"l.bias", b.tensor()}};
    const std::vector<std::string> names = {"l.weight", "l.bias"};
    auto make = [&](const std::vector<std::pair<std::string, Tensor>> &n) {
        const ParamGroupConfig plain =
            ParamGroupConfig::sgd("plain", ParamSelector::Any({{ParamMatch::Suffix, "bias"}}), 0.5, 0.9, 0.0);
        const ParamGroupConfig decay = ParamGroupConfig::adamw("decay", ParamSelector::All(), 0.01, 0.1);
        return GroupOptimizer::from_named_params(n, {plain}, &decay, NBO_DT_F64);
    };
    GroupOptimizer opt = make(named);
    opt.step({w.tensor(), b.tensor()}, {gw.tensor(), gb.tensor()});
    opt.step({w.tensor(), b.tensor()}, {gw.tensor(), gb.tensor()});
    TensorList module({w.tensor(), b.tensor()});
    const ScheduleState sched{0.5, LrSchedule::cosine(1, 10, 0.0)};
    save_checkpoint(dir, module, names, opt, nullptr, &sched, TrainState{1, 2, 1, std::nullopt});

    Mat w2({0.0, 0.0}), b2({0.0});
    GroupOptimizer opt2 = make({{"l.weight", w2.tensor()}, {"l.bias", b2.tensor()}});
    TensorList module2({w2.tensor(), b2.tensor()});
    std::optional<ScheduleState> schedule2;
    TrainState state2;
    load_checkpoint(dir, module2, names, opt2, nullptr, schedule2, state2);
    EXPECT(w2.get(0) == w.get(0) && w2.get(1) == w.get(1) && b2.get() == b.get());
    EXPECT(state2.epoch == 1 && state2.step == 2 && !state2.rng_state && schedule2 && schedule2->base_lr == 0.5);
    EXPECT(opt2.group_optimizer(1).step_count() == 2 && opt2.group_optimizer(0).meta().momentum == 0.9);
    double m1[2] = {0, 0}, m2[2] = {0, 0}, v1 = 0, v2 = 0;
    opt.group_optimizer(1).state_read("m0", m1, 2, false), opt2.group_optimizer(1).state_read("m0", m2, 2, false);
    opt.group_optimizer(0).state_read("v0", &v1, 1, false), opt2.group_optimizer(0).state_read("v0", &v2, 1, false);
    EXPECT(m1[0] == m2[0] && m1[1] == m2[1] && m1[1] != 0.0 && v1 == v2 && v1 != 0.0);
    // one more step on both: the same parameters
    opt.step({w.tensor(), b.tensor()}, {gw.tensor(), gb.tensor()});
    opt2.step({w2.tensor(), b2.tensor()}, {gw.tensor(), gb.tensor()});
    EXPECT(w2.get(0) == w.get(0) && w2.get(1) == w.get(1) && b2.get() == b.get());
    // a checkpoint with another group layout is refused with the reference's error
    const ParamGroupConfig all = ParamGroupConfig::adamw("decay", ParamSelector::All(), 0.01, 0.1);
    GroupOptimizer one = GroupOptimizer::from_named_params({{"l.weight", w2.tensor()}, {"l.bias", b2.tensor()}}, {}, &all,
                                                           NBO_DT_F64);
    std::string what;
    try {
        load_checkpoint(dir, module2, names, one, nullptr, schedule2, state2);
    } catch (const CheckpointError &e) {
        what = e.what();
    }
    EXPECT(what.find("group index out of range: 1") != std::string::npos);
}

static void constructors_and_set_state()  // alg.rs:41-45, 90-105, 244-250, 374-378; core.rs:12-16
{
    Mat p({1.0, 2.0}), g({1.0, 1.0});
    const std::vector<Tensor> params = {p.tensor()}, grads = {g.tensor()};
    EXPECT(shapes_of(params) == (Shapes{{1, 2}}));
    AdamW opt(0.1, shapes_of(params), NBO_DT_F64);  // AdamW::from_params(0.1, &params)
    EXPECT((opt.state_names() == std::vector<std::string>{"m0", "v0"}));
    opt.step_slices(params, grads);
    EXPECT(opt.step_count() == 1);
    opt.set_state(41, 0.8, 0.9, 1e-6, 0.25, 0.5);
    const OptimMeta m = opt.meta();
    EXPECT(m.step_count == 41 && m.beta1 == 0.8 && m.beta2 == 0.9 && m.eps == 1e-6 && m.weight_decay == 0.25 &&
           m.lr == 0.5 && opt.lr() == 0.5);
    opt.step_slices(params, grads);
    EXPECT(opt.step_count() == 42);
    Adam adam(0.1, shapes_of(params), NBO_DT_F64);
    adam.set_state(7, 0.5, 0.75, 1e-3, 0.125);
    const OptimMeta a = adam.meta();
    EXPECT(a.step_count == 7 && a.beta1 == 0.5 && a.beta2 == 0.75 && a.eps == 1e-3 && a.lr == 0.125 &&
           a.weight_decay == 0.0);
    Sgd sgd(0.1, shapes_of(params), NBO_DT_F64);
    EXPECT((sgd.state_names() == std::vector<std::string>{"v0"}));
    sgd.set_state(0.5, 0.0, 0.5);  // p <- p - 0.5 * (g + 0.5 * p)
    const double before = p.get(1);
    sgd.step_slices(params, grads);
    EXPECT(p.get(1) == before - 0.5 * (1.0 + before * 0.5));
    const OptimMeta sm = sgd.meta();
    EXPECT(sm.lr == 0.5 && sm.momentum == 0.0 && sm.weight_decay == 0.5 && sm.step_count == 0);
}

// `--lr`: prints lr_at_step for a grid of schedules and steps as f64 bit patterns, for a
// bit-for-bit comparison with the CPU oracle (needs no device).
static int print_lr_grid()
{
    const LrSchedule scheds[] = {LrSchedule::cosine(10, 110, 1e-5), LrSchedule::cosine(0, 7, 0.0),
                                 LrSchedule::linear(5, 50),         LrSchedule::linear(0, 1),
                                 LrSchedule::one_cycle(1e-2, 100, 0.3), LrSchedule::one_cycle(0.5, 9, 0.0),
                                 LrSchedule::step(3, 0.7),          LrSchedule::step(0, 0.5),
                                 // the reference's usize arithmetic at its edges (core.rs:86-89, 121-123, 165-167):
                                 // total_steps below warmup_steps, pct_start above 1, a decay exponent past i32
                                 LrSchedule::cosine(10, 5, 0.1),    LrSchedule::one_cycle(1e-2, 10, 1.5),
                                 LrSchedule::linear(40, 12)};
    for (size_t k = 0; k < sizeof(scheds) / sizeof(scheds[0]); k++)
        for (uint64_t step = 0; step <= 120; step += (step < 12 ? 1 : 9)) {
            const double lr = lr_at_step(scheds[k], 3e-4, step);
            uint64_t bits;
            static_assert(sizeof(bits) == sizeof(lr), "f64 is 64 bits");
            std::memcpy(&bits, &lr, 8);
            std::printf("%zu %llu %016llx\n", k, (unsigned long long)step, (unsigned long long)bits);
        }
    return 0;
}

int main(int argc, char **argv)
{
    if (argc > 1 && std::string(argv[1]) == "--lr") return print_lr_grid();
    if (argc > 1) g_checkpoint_dir = argv[1];
    struct {
        const char *name;
        void (*fn)();
    } tests[] = {{"sgd_step_updates_param", sgd_step_updates_param},
                 {"step_with_vars_pulls_params_and_grads", step_with_vars_pulls_params_and_grads},
                 {"adam_step_updates_param", adam_step_updates_param},
                 {"adamw_step_updates_param", adamw_step_updates_param},
                 {"grad_scaler_unscale", grad_scaler_unscale},
                 {"grad_scaler_detects_inf", grad_scaler_detects_inf},
                 {"clip_grad_norm_scales", clip_grad_norm_scales},
                 {"group_optimizer_weight_decay_exclusion", weight_decay_exclusion},
                 {"lr_schedules", lr_schedules},
                 {"nan_policy_skip_drops_step", nan_policy_skip_drops_step},
                 {"trainer_accumulates_then_clips_and_steps", trainer_accumulates_then_clips_and_steps},
                 {"backend_axpy_is_multiply_then_add", backend_axpy_is_multiply_then_add},
                 {"checkpoint_roundtrip_with_schedule", checkpoint_roundtrip_with_schedule},
                 {"mixed_precision_checkpoint_resumes_bit_for_bit", mixed_precision_checkpoint_resumes_bit_for_bit},
                 {"group_mixed_precision_checkpoint_resumes_bit_for_bit",
                  group_mixed_precision_checkpoint_resumes_bit_for_bit},
                 {"panics_and_errors", panics_and_errors},
                 {"group_checkpoint_roundtrip", group_checkpoint_roundtrip},
                 {"constructors_and_set_state", constructors_and_set_state},
                 {"decay_presets_and_known_norm_group_step", decay_presets_and_known_norm_group_step}};
    try {
        check(nbo_init());
        for (auto &t : tests) {
            const int before = failures;
            t.fn();
            std::printf("%s %s\n", failures == before ? "ok    " : "FAILED", t.name);
        }
    } catch (const std::exception &e) {
        std::printf("unexpected exception: %s\n", e.what());
        return 2;
    }
    std::printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
