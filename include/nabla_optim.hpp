// nabla_optim.hpp -- C++ mirror of nabla-train's optimizer interface over the C ABI of
// nabla_optim.h.  Header-only; link libnabla_optim.so.
//
// The reference's host language is Rust; this is the same surface for a C++ host:
// the names, the argument meaning and the error behaviour of
// nabla-train/src/optim/{core,alg}.rs and nabla-train/src/trainer.rs:500-523.
//   trait Optimizer   (core.rs:9-44)    -> nabla::optim::Optimizer  {step, reset, set_lr}
//   Sgd / Adam / AdamW (alg.rs)         -> same names, same builder setters
//   trait OptimState  (core.rs:64-79)   -> kind, state_read / state_write, meta, load_meta
//   GradScaler        (core.rs:334-413) -> same methods
//   clip_grad_norm, zero_grad, scale_grad, has_non_finite, accumulate -> free functions
//   LrSchedule / lr_at_step (core.rs:81-173)        -> same names (host arithmetic, f64)
//   Trainer's loop body after backward (trainer.rs:216-291) -> TrainerTail, GradNanPolicy
//   Backend primitives (nabla-core backend/mod.rs:82-216, 275-279) -> namespace backend
// Where the reference panics (assert_eq! on list lengths, shape asserts) this throws
// nabla::optim::Panic with the reference's message; where it returns Err(String) this
// throws nabla::optim::StateError.
#ifndef NABLA_OPTIM_HPP
#define NABLA_OPTIM_HPP

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "nabla_optim.h"

namespace nabla {
namespace optim {

struct Panic : std::logic_error {
    using std::logic_error::logic_error;
};
struct StateError : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct RuntimeError : std::runtime_error {
    int status;
    RuntimeError(int s, const std::string &m) : std::runtime_error(m), status(s) {}
};

inline void check(int status)
{
    if (status == NBO_OK) return;
    const std::string msg = nbo_last_error();
    if (status == NBO_ERR_LEN_MISMATCH || status == NBO_ERR_COUNT_MISMATCH || status == NBO_ERR_SHAPE)
        throw Panic(msg);
    if (status == NBO_ERR_STATE_KEY || status == NBO_ERR_STATE_INDEX || status == NBO_ERR_KIND)
        throw StateError(msg);
    throw RuntimeError(status, msg);
}

// A dense row-major (rows x cols) matrix in device memory: what `&Tensor<T, B>` is to
// the reference's optimizers.
struct Tensor {
    void *data = nullptr;
    uint64_t rows = 0, cols = 0;
    nbo_dtype dtype = NBO_DT_F32;
    std::pair<uint64_t, uint64_t> shape() const { return {rows, cols}; }
};

// `&[&Tensor]`: described to the device once, reusable across steps.
class TensorList {
public:
    TensorList() = default;
    explicit TensorList(const std::vector<Tensor> &tensors) { assign(tensors); }
    TensorList(const TensorList &) = delete;
    TensorList &operator=(const TensorList &) = delete;
    TensorList(TensorList &&o) noexcept : h_(o.h_), n_(o.n_), tensors_(std::move(o.tensors_)) { o.h_ = nullptr; }
    ~TensorList() { reset(); }

    void assign(const std::vector<Tensor> &tensors)
    {
        reset();
        std::vector<uint64_t> rows, cols;
        std::vector<const void *> ptrs;
        const nbo_dtype dt = tensors.empty() ? NBO_DT_F32 : tensors[0].dtype;
        for (const Tensor &t : tensors) {
            if (t.dtype != dt) throw RuntimeError(NBO_ERR_DTYPE, "all tensors of a list share one dtype");
            rows.push_back(t.rows);
            cols.push_back(t.cols);
            ptrs.push_back(t.data);
        }
        n_ = tensors.size();
        check(nbo_list_create(n_, rows.data(), cols.data(), dt, ptrs.data(), &h_));
        tensors_ = tensors;
    }
    nbo_list *handle() const { return h_; }
    size_t size() const { return n_; }
    // what the list was made from
    const std::vector<Tensor> &tensors() const { return tensors_; }

private:
    void reset()
    {
        if (h_) nbo_list_destroy(h_);
        h_ = nullptr;
    }
    nbo_list *h_ = nullptr;
    size_t n_ = 0;
    std::vector<Tensor> tensors_;
};

enum class OptimKind { AdamW = NBO_KIND_ADAMW, Adam = NBO_KIND_ADAM, Sgd = NBO_KIND_SGD };

// optim/core.rs:53-62
struct OptimMeta {
    OptimKind kind;
    double lr, beta1, beta2, eps, weight_decay, momentum;
    uint64_t step_count;
};

// optim/core.rs:326-332; defaults of core.rs:336-344
struct GradScalerState {
    double scale = 65536.0, growth_factor = 2.0, backoff_factor = 0.5;
    uint64_t growth_interval = 2000, consecutive_ok = 0;
};

class GradScaler {
public:
    GradScaler() = default;
    GradScaler(const GradScaler &) = delete;
    GradScaler &operator=(const GradScaler &) = delete;
    ~GradScaler()
    {
        if (h_) nbo_scaler_destroy(h_);
    }
    // core.rs:351-388: true if every gradient was finite (they are now unscaled), false
    // otherwise (they are now zeros and the scale has been backed off).
    bool unscale_and_update(TensorList &grads)
    {
        int ok = 0;
        check(nbo_scaler_unscale_and_update(handle(), grads.handle(), &ok));
        return ok != 0;
    }
    double scale_factor() { return state().scale; }
    // core.rs:347-349: out = loss * T::from_f64(scale)
    void scale_loss(TensorList &loss, TensorList &out)
    {
        check(nbo_backend_apply(NBO_BACKEND_SCALE, out.handle(), loss.handle(), nullptr, scale_factor()));
    }
    GradScalerState state()
    {
        if (!h_) return init_;
        nbo_scaler_state s;
        check(nbo_scaler_state_get(h_, &s));
        return {s.scale, s.growth_factor, s.backoff_factor, s.growth_interval, s.consecutive_ok};
    }
    void load_state(const GradScalerState &st)
    {
        init_ = st;
        if (h_) {
            const nbo_scaler_state s = {st.scale, st.growth_factor, st.backoff_factor, st.growth_interval,
                                        st.consecutive_ok};
            check(nbo_scaler_load_state(h_, &s));
        }
    }
    nbo_scaler *handle()
    {
        if (!h_) {
            const nbo_scaler_state s = {init_.scale, init_.growth_factor, init_.backoff_factor,
                                        init_.growth_interval, init_.consecutive_ok};
            check(nbo_scaler_create(&s, &h_));
        }
        return h_;
    }

private:
    nbo_scaler *h_ = nullptr;
    GradScalerState init_;
};

// trait Optimizer + trait OptimState.  T is float or double (the arithmetic type);
// with `master` the caller's tensors may be bf16 or f16 while the state stays f32.
class Optimizer {
public:
    Optimizer(const Optimizer &) = delete;
    Optimizer &operator=(const Optimizer &) = delete;
    virtual ~Optimizer()
    {
        if (h_) nbo_optim_destroy(h_);
    }

    // optim/core.rs:10: panics (throws Panic) on length or shape mismatch
    void step(TensorList &params, TensorList &grads) { check(nbo_optim_step(handle(), params.handle(), grads.handle())); }
    void step(const std::vector<Tensor> &params, const std::vector<Tensor> &grads)
    {
        TensorList p(params), g(grads);
        step(p, g);
    }
    // optim/core.rs:12-16: the default forwards to step
    void step_slices(const std::vector<Tensor> &params, const std::vector<Tensor> &grads) { step(params, grads); }
    // optim/core.rs:18-39.  `module.parameters_mut()` yields a std::vector<Tensor>; each
    // variable's `grad()` yields a `const Tensor *`, null when backward has not run.
    template <typename Module, typename Var> void step_with_vars(Module &module, const std::vector<Var> &param_vars)
    {
        const std::vector<Tensor> params = module.parameters_mut();
        if (params.size() != param_vars.size())
            throw Panic("nabla-train: step_with_vars param_vars length (" +
                                                  std::to_string(param_vars.size()) +
                                                  ") doesn't match module parameters count (" +
                                                  std::to_string(params.size()) + ")");
        std::vector<Tensor> grads;
        for (size_t i = 0; i < param_vars.size(); i++) {
            const Tensor *g = param_vars[i].grad();
            if (!g)
                throw Panic("nabla-train: step_with_vars: param_vars[" + std::to_string(i) +
                                             "] has no gradient (call backward first)");
            grads.push_back(*g);
        }
        step(params, grads);
    }
    void reset() { check(nbo_optim_reset(handle())); }
    void set_lr(double lr)
    {
        meta_.lr = lr;
        if (h_) check(nbo_optim_set_lr(h_, lr));
    }
    double lr() const { return meta_.lr; }
    uint64_t step_count() { return meta().step_count; }

    // the Trainer tail (trainer.rs:230-291) in one asynchronous call
    void fused_step(TensorList &params, TensorList &grads, GradScaler *scaler, double max_norm,
                    bool zero_grads = false, bool skip_nonfinite = false, bool zero_on_skip = false)
    {
        check(nbo_fused_step(handle(), scaler ? scaler->handle() : nullptr, params.handle(), grads.handle(),
                             max_norm,
                             (zero_grads ? NBO_STEP_ZERO_GRADS : 0u) | (skip_nonfinite ? NBO_STEP_SKIP_NONFINITE : 0u) |
                                 (zero_on_skip ? NBO_STEP_ZERO_ON_SKIP : 0u)));
    }
    // clip + step (+ zeroing) over gradients whose sum of squares is already known
    void fused_step_norm(TensorList &params, TensorList &grads, double sumsq, double max_norm, bool zero_grads = false)
    {
        check(nbo_fused_step_norm(handle(), params.handle(), grads.handle(), max_norm, sumsq,
                                  zero_grads ? NBO_STEP_ZERO_GRADS : 0u));
    }
    nbo_step_info last_step()
    {
        nbo_step_info info;
        check(nbo_optim_last_step(handle(), &info));
        return info;
    }

    OptimKind kind() const { return (OptimKind)meta_.kind; }
    OptimMeta meta()
    {
        nbo_meta m = meta_;
        if (h_) check(nbo_optim_get_meta(h_, &m));
        else if (meta_.kind == NBO_KIND_SGD) m.beta1 = m.beta2 = m.eps = 0.0, m.step_count = 0;
        return {(OptimKind)m.kind, m.lr, m.beta1, m.beta2, m.eps, m.weight_decay, m.momentum, m.step_count};
    }
    // alg.rs:531-545: Err("optim kind mismatch") -> StateError
    void load_meta(const OptimMeta &m)
    {
        const nbo_meta c = {(int32_t)m.kind, 0, m.lr, m.beta1, m.beta2, m.eps, m.weight_decay, m.momentum,
                            m.step_count};
        check(nbo_optim_load_meta(handle(), &c));
        meta_.lr = m.lr;
    }
    // one state tensor ("m3", "v3", "w3"); buffers hold rows*cols elements of the state type
    void state_read(const std::string &name, void *buf, uint64_t n, bool on_device)
    {
        check(nbo_optim_state_read(handle(), name.c_str(), buf, n, on_device ? 1 : 0));
    }
    void state_write(const std::string &name, const void *buf, uint64_t n, bool on_device)
    {
        check(nbo_optim_state_write(handle(), name.c_str(), buf, n, on_device ? 1 : 0));
    }
    // optim.nbla of a checkpoint (checkpoint.rs:59-62, 92-95): state_tensors() through
    // save_tensors, load_tensors into load_state_tensors; errors as StateError / RuntimeError
    void save_state(const std::string &path) { check(nbo_optim_save_state(handle(), path.c_str())); }
    void load_state(const std::string &path) { check(nbo_optim_load_state(handle(), path.c_str())); }
    bool keeps_master() const { return master_; }
    // params.nbla of a mixed-precision optimizer: its f32 master weights under the parameters' names
    void save_master(const std::string &path, const std::vector<std::string> &names)
    {
        std::vector<const char *> raw;
        for (const std::string &n : names) raw.push_back(n.c_str());
        check(nbo_optim_save_master(handle(), path.c_str(), raw.data()));
    }
    void load_master(const std::string &path, const std::vector<std::string> &names)
    {
        std::vector<const char *> raw;
        for (const std::string &n : names) raw.push_back(n.c_str());
        check(nbo_optim_load_master(handle(), path.c_str(), raw.data()));
    }
    void master_from_params(TensorList &params_half) { check(nbo_optim_master_from_params(handle(), params_half.handle())); }
    void params_from_master(TensorList &params_half) { check(nbo_optim_params_from_master(handle(), params_half.handle())); }
    // names of state_tensors() in their order (alg.rs:476-485, 553-562, 623-629)
    std::vector<std::string> state_names() const
    {
        std::vector<std::string> out;
        if (meta_.kind != NBO_KIND_SGD)
            for (size_t i = 0; i < shapes_.size(); i++) out.push_back("m" + std::to_string(i));
        for (size_t i = 0; i < shapes_.size(); i++) out.push_back("v" + std::to_string(i));
        return out;
    }

    nbo_optim *handle()
    {
        if (!h_) {
            std::vector<uint64_t> rows, cols;
            for (const auto &s : shapes_) {
                rows.push_back(s.first);
                cols.push_back(s.second);
            }
            check(nbo_optim_create(&meta_, shapes_.size(), rows.data(), cols.data(), state_dtype_,
                                   master_ ? 1 : 0, &h_));
        }
        return h_;
    }

protected:
    Optimizer(nbo_kind kind, double lr, std::vector<std::pair<uint64_t, uint64_t>> shapes, nbo_dtype state_dtype,
              bool master)
        : shapes_(std::move(shapes)), state_dtype_(state_dtype), master_(master)
    {
        meta_ = nbo_meta{(int32_t)kind, 0, lr, 0.0, 0.0, 0.0, 0.0, 0.0, 0};
    }
    void builder_guard() const
    {
        if (h_) throw RuntimeError(NBO_ERR_ARG, "builder setters apply before the first use");
    }
    nbo_meta meta_;

private:
    std::vector<std::pair<uint64_t, uint64_t>> shapes_;
    nbo_dtype state_dtype_;
    bool master_;
    nbo_optim *h_ = nullptr;
};

using Shapes = std::vector<std::pair<uint64_t, uint64_t>>;

// `X::from_params(lr, params)` is `X(lr, shapes_of(params))` (alg.rs:41-45, 201-205, 332-336)
inline Shapes shapes_of(const std::vector<Tensor> &params)
{
    Shapes out;
    for (const Tensor &p : params) out.push_back(p.shape());
    return out;
}

// alg.rs:310-428
class Sgd : public Optimizer {
public:
    Sgd(double lr, Shapes shapes, nbo_dtype state_dtype = NBO_DT_F32, bool master = false)
        : Optimizer(NBO_KIND_SGD, lr, std::move(shapes), state_dtype, master)
    {
    }
    Sgd &momentum(double m) { builder_guard(); meta_.momentum = m; return *this; }
    Sgd &weight_decay(double wd) { builder_guard(); meta_.weight_decay = wd; return *this; }
    double momentum_value() const { return meta_.momentum; }
    double weight_decay_value() const { return meta_.weight_decay; }
    // alg.rs:374-378
    void set_state(double lr, double momentum, double weight_decay)
    {
        load_meta({OptimKind::Sgd, lr, 0.0, 0.0, 0.0, weight_decay, momentum, 0});
        meta_.momentum = momentum, meta_.weight_decay = weight_decay;
    }
};

// alg.rs:169-308
class Adam : public Optimizer {
public:
    Adam(double lr, Shapes shapes, nbo_dtype state_dtype = NBO_DT_F32, bool master = false)
        : Optimizer(NBO_KIND_ADAM, lr, std::move(shapes), state_dtype, master)
    {
        meta_.beta1 = 0.9, meta_.beta2 = 0.999, meta_.eps = 1e-8;
    }
    Adam &beta1(double b) { builder_guard(); meta_.beta1 = b; return *this; }
    Adam &beta2(double b) { builder_guard(); meta_.beta2 = b; return *this; }
    Adam &eps(double e) { builder_guard(); meta_.eps = e; return *this; }
    // alg.rs:244-250
    void set_state(uint64_t step_count, double beta1, double beta2, double eps, double lr)
    {
        load_meta({OptimKind::Adam, lr, beta1, beta2, eps, 0.0, 0.0, step_count});
        meta_.beta1 = beta1, meta_.beta2 = beta2, meta_.eps = eps;
    }
};

// alg.rs:7-167
class AdamW : public Optimizer {
public:
    AdamW(double lr, Shapes shapes, nbo_dtype state_dtype = NBO_DT_F32, bool master = false)
        : Optimizer(NBO_KIND_ADAMW, lr, std::move(shapes), state_dtype, master)
    {
        meta_.beta1 = 0.9, meta_.beta2 = 0.999, meta_.eps = 1e-8, meta_.weight_decay = 0.01;
    }
    AdamW &beta1(double b) { builder_guard(); meta_.beta1 = b; return *this; }
    AdamW &beta2(double b) { builder_guard(); meta_.beta2 = b; return *this; }
    AdamW &eps(double e) { builder_guard(); meta_.eps = e; return *this; }
    AdamW &weight_decay(double wd) { builder_guard(); meta_.weight_decay = wd; return *this; }
    // alg.rs:90-105
    void set_state(uint64_t step_count, double beta1, double beta2, double eps, double weight_decay, double lr)
    {
        load_meta({OptimKind::AdamW, lr, beta1, beta2, eps, weight_decay, 0.0, step_count});
        meta_.beta1 = beta1, meta_.beta2 = beta2, meta_.eps = eps, meta_.weight_decay = weight_decay;
    }
};

// nabla-train/src/trainer.rs:500-523; returns the pre-clip norm
inline double clip_grad_norm(TensorList &grads, double max_norm)
{
    double norm = 0.0;
    check(nbo_clip_grad_norm(grads.handle(), max_norm, &norm));
    return norm;
}
// nabla-ml/src/autograd/ops.rs:1668-1680
inline void zero_grad(TensorList &grads) { check(nbo_zero_grad(grads.handle())); }
inline void scale_grad(TensorList &grads, double factor) { check(nbo_scale_grad(grads.handle(), factor)); }
inline void sync() { check(nbo_sync()); }
// Trainer::has_non_finite, trainer.rs:387-400
inline bool has_non_finite(TensorList &grads)
{
    int found = 0;
    check(nbo_has_non_finite(grads.handle(), &found));
    return found != 0;
}
// buf[i] = &buf[i] + g, trainer.rs:262-266
inline void accumulate(TensorList &accum, TensorList &grads, bool zero_grads = false)
{
    check(nbo_accumulate(accum.handle(), grads.handle(), zero_grads ? 1 : 0));
}
// One micro-batch of the accumulating Trainer in a single pass (trainer.rs:230-267): finite
// scan + loss-scale update, buf[i] = &buf[i] + g / scale, and the new buffer's sum of squares.
// Returns false on a non-finite gradient (the buffer then holds garbage, the Trainer discards it).
// sumsq may be null: only the last micro-batch of an accumulation needs the sum of squares, and a
// pass without it has nothing to reduce but one bit (one small launch fewer).
inline bool unscale_accumulate(TensorList &accum, TensorList &grads, GradScaler *scaler, double *sumsq,
                               bool check_finite = false, bool write_grads = false)
{
    int ok = 0;
    check(nbo_unscale_accumulate(scaler ? scaler->handle() : nullptr, accum.handle(), grads.handle(),
                                 (check_finite ? NBO_ACC_CHECK_FINITE : 0u) | (write_grads ? NBO_ACC_WRITE_GRADS : 0u),
                                 &ok, sumsq));
    return ok != 0;
}

// params.nbla of a checkpoint: save_tensors / load_tensors + load_state_dict
// (nabla-ml/src/module/core.rs:66-120, 281-304) over a list of device tensors
inline void save_tensors(const std::string &path, TensorList &list, const std::vector<std::string> &names)
{
    std::vector<const char *> c;
    for (const std::string &n : names) c.push_back(n.c_str());
    check(nbo_nbla_save_list(path.c_str(), list.handle(), c.data()));
}
inline void load_state_dict(const std::string &path, TensorList &list, const std::vector<std::string> &names)
{
    std::vector<const char *> c;
    for (const std::string &n : names) c.push_back(n.c_str());
    check(nbo_nbla_load_list(path.c_str(), list.handle(), c.data()));
}

// ---- LrSchedule (optim/core.rs:81-173): host arithmetic in f64 -------------------------
struct LrSchedule {
    enum Kind { Cosine, Linear, OneCycle, Step } kind;
    uint64_t warmup_steps = 0, total_steps = 0, step_size = 0;
    double min_lr = 0.0, max_lr = 0.0, pct_start = 0.0, gamma = 0.0;
    static LrSchedule cosine(uint64_t warmup, uint64_t total, double min_lr)
    {
        LrSchedule s{Cosine};
        s.warmup_steps = warmup, s.total_steps = total, s.min_lr = min_lr;
        return s;
    }
    static LrSchedule linear(uint64_t warmup, uint64_t total)
    {
        LrSchedule s{Linear};
        s.warmup_steps = warmup, s.total_steps = total;
        return s;
    }
    static LrSchedule one_cycle(double max_lr, uint64_t total, double pct_start)
    {
        LrSchedule s{OneCycle};
        s.max_lr = max_lr, s.total_steps = total, s.pct_start = pct_start;
        return s;
    }
    static LrSchedule step(uint64_t step_size, double gamma)
    {
        LrSchedule s{Step};
        s.step_size = step_size, s.gamma = gamma;
        return s;
    }
};

namespace detail {
// f64::powi as compiler-rt's __powidf2: square-and-multiply from the low bit
inline double powi(double a, int n)
{
    const bool recip = n < 0;
    unsigned b = recip ? 0u - (unsigned)n : (unsigned)n;
    double r = 1.0;
    for (;;) {
        if (b & 1u) r *= a;
        b >>= 1;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0 / r : r;
}
inline double warmup_lr(double base_lr, uint64_t step, uint64_t warmup)
{
    return base_lr * (double)step / (double)(warmup > 1 ? warmup : 1);
}
inline double decay_progress(uint64_t step, uint64_t start, uint64_t total)
{
    const uint64_t d = total - start; // usize subtraction, as the reference writes it
    return (double)(step - start) / (double)(d > 1 ? d : 1);
}
inline double cosine_decay(double high, double low, double progress)
{
    return low + 0.5 * (high - low) * (1.0 + std::cos(3.14159265358979323846264338327950288 * progress));
}
} // namespace detail

inline double lr_at_step(const LrSchedule &s, double base_lr, uint64_t step)
{
    using namespace detail;
    switch (s.kind) {
    case LrSchedule::Cosine:
        if (step < s.warmup_steps) return warmup_lr(base_lr, step, s.warmup_steps);
        return cosine_decay(base_lr, s.min_lr, decay_progress(step, s.warmup_steps, s.total_steps));
    case LrSchedule::Linear: {
        if (step < s.warmup_steps) return warmup_lr(base_lr, step, s.warmup_steps);
        const double p = 1.0 - decay_progress(step, s.warmup_steps, s.total_steps);
        return base_lr * (p > 0.0 ? p : 0.0);
    }
    case LrSchedule::OneCycle: {
        // Rust's `as usize`: truncation toward zero, saturating at both ends, NaN -> 0
        const double upf = (double)s.total_steps * s.pct_start;
        const uint64_t up = !(upf > 0.0) ? 0 : upf >= 18446744073709551616.0 ? UINT64_MAX : (uint64_t)upf;
        if (step < up) return base_lr + (s.max_lr - base_lr) * (double)step / (double)(up > 1 ? up : 1);
        return cosine_decay(s.max_lr, base_lr, decay_progress(step, up, s.total_steps));
    }
    default: {
        const uint64_t sz = s.step_size > 1 ? s.step_size : 1;
        return base_lr * powi(s.gamma, (int32_t)(uint32_t)(step / sz)); // `k as i32`: the low 32 bits
    }
    }
}

// ---- Backend primitives on tensor lists (nbo_backend_apply / nbo_backend_cast) ----------
namespace backend {
inline void apply(nbo_backend_op op, TensorList &out, TensorList *a, TensorList *b, double s)
{
    check(nbo_backend_apply(op, out.handle(), a ? a->handle() : nullptr, b ? b->handle() : nullptr, s));
}
inline void scale(TensorList &a, double s, TensorList &out) { apply(NBO_BACKEND_SCALE, out, &a, nullptr, s); }
inline void axpy_inplace(TensorList &y, double alpha, TensorList &x) { apply(NBO_BACKEND_AXPY, y, &x, nullptr, alpha); }
inline void add(TensorList &a, TensorList &b, TensorList &out) { apply(NBO_BACKEND_ADD, out, &a, &b, 0.0); }
inline void emul(TensorList &a, TensorList &b, TensorList &out) { apply(NBO_BACKEND_EMUL, out, &a, &b, 0.0); }
inline void ediv(TensorList &a, TensorList &b, TensorList &out) { apply(NBO_BACKEND_EDIV, out, &a, &b, 0.0); }
inline void powf(TensorList &a, double p, TensorList &out) { apply(NBO_BACKEND_POWF, out, &a, nullptr, p); }
inline void map_add(TensorList &a, double c, TensorList &out) { apply(NBO_BACKEND_ADD_SCALAR, out, &a, nullptr, c); }
inline void zeros(TensorList &out) { apply(NBO_BACKEND_ZEROS, out, nullptr, nullptr, 0.0); }
inline void clone_storage(TensorList &a, TensorList &out) { apply(NBO_BACKEND_CLONE, out, &a, nullptr, 0.0); }
inline void cast(TensorList &src, TensorList &dst) { check(nbo_backend_cast(dst.handle(), src.handle())); }
} // namespace backend

// ---- the Trainer's loop body after backward (trainer.rs:216-291) --------------------------
enum class GradNanPolicy { Skip, Stop }; // trainer.rs:403-406
struct TrainError : std::runtime_error { // TrainError::EvalError
    using std::runtime_error::runtime_error;
};

// Per micro-batch: scaler -> nan policy -> accumulate -> (every grad_accum-th) schedule,
// clip, step, zero.  `accum` is caller-provided zero-filled storage shaped like the
// gradients (the reference allocates it; this library allocates nothing per step).
// Without accumulation and with at most one of scaler / nan policy the whole sequence is
// one fused step whose skip is decided on the device (the decision is read back only
// because step(), which the schedule is a function of, must not advance on a skipped step);
// otherwise the decisions are the reference's synchronous ones: scan, unscale and
// accumulation are one pass over the gradients, which also yields the buffer's sum of
// squares, and clip + step + zero over the accumulation buffer are one fused step.
// The reference unscales the gradients in place on the way; here they are only read.
class TrainerTail {
public:
    TrainerTail(Optimizer &optimizer, TensorList &params, TensorList &accum)
        : opt_(optimizer), params_(params), accum_(accum)
    {
    }
    TrainerTail &with_schedule(const LrSchedule &s, double base_lr) { schedule_ = s, base_lr_ = base_lr, has_schedule_ = true; return *this; }
    TrainerTail &with_grad_scaler(GradScaler &s) { scaler_ = &s; return *this; }
    TrainerTail &with_grad_accum(uint64_t steps) { grad_accum_ = steps > 1 ? steps : 1; return *this; }
    TrainerTail &with_nan_policy(GradNanPolicy p) { policy_ = p, has_policy_ = true; return *this; }
    TrainerTail &with_grad_clip(double max_norm) { grad_clip_ = max_norm > 0.0 ? max_norm : 0.0; return *this; }
    uint64_t step() const { return step_; }
    double loss_scale() { return scaler_ ? scaler_->scale_factor() : 1.0; } // trainer.rs:218-221

    // returns true if the optimizer stepped
    bool after_backward(TensorList &grads)
    {
        if (grad_accum_ == 1 && !(scaler_ && has_policy_)) return fused(grads);
        if (accum_count_ == 0 && dirty_) { // a dropped accumulation starts again from zeros (:253-260)
            zero_grad(accum_);
            dirty_ = false;
        }
        double sumsq = -1.0;
        if (scaler_ && has_policy_) {
            // both decisions, in the reference's order: a micro-batch whose unscaled gradients
            // overflow is the nan policy's, not the scaler's
            if (!scaler_->unscale_and_update(grads)) return drop(); // :230-237
            if (has_non_finite(grads)) {                            // :239-251
                if (policy_ == GradNanPolicy::Skip) return drop();
                throw TrainError("non-finite gradient");
            }
            accumulate(accum_, grads); // :262-266
            dirty_ = true;
        } else {
            dirty_ = true; // a non-finite micro-batch leaves garbage in the buffer
            const bool last = accum_count_ + 1 >= grad_accum_; // the clip needs the sum of squares then
            if (!unscale_accumulate(accum_, grads, scaler_, last ? &sumsq : nullptr, has_policy_)) {
                drop();
                if (!scaler_ && policy_ == GradNanPolicy::Stop) throw TrainError("non-finite gradient");
                return false;
            }
        }
        accum_count_ += 1;
        if (accum_count_ < grad_accum_) return false;
        if (has_schedule_) opt_.set_lr(lr_at_step(schedule_, base_lr_, step_)); // :270-273
        if (sumsq < 0.0) opt_.fused_step(params_, accum_, nullptr, grad_clip_, /*zero_grads=*/true); // :274-290
        else opt_.fused_step_norm(params_, accum_, sumsq, grad_clip_, /*zero_grads=*/true);
        accum_count_ = 0;
        dirty_ = false;
        step_ += 1;
        return true;
    }

private:
    bool fused(TensorList &grads)
    {
        if (has_schedule_) opt_.set_lr(lr_at_step(schedule_, base_lr_, step_)); // harmless if the step is skipped
        opt_.fused_step(params_, grads, scaler_, grad_clip_, false, has_policy_);
        if ((scaler_ || has_policy_) && opt_.last_step().found_inf) {
            if (!scaler_ && policy_ == GradNanPolicy::Stop) throw TrainError("non-finite gradient");
            return false;
        }
        step_ += 1;
        return true;
    }
    bool drop()
    {
        accum_count_ = 0; // accum_grads = None: the buffer is cleared before its next use
        return false;
    }
    Optimizer &opt_;
    TensorList &params_;
    TensorList &accum_;
    GradScaler *scaler_ = nullptr;
    LrSchedule schedule_{LrSchedule::Linear};
    double base_lr_ = 0.0, grad_clip_ = 0.0;
    bool has_schedule_ = false, has_policy_ = false, dirty_ = false;
    GradNanPolicy policy_ = GradNanPolicy::Skip;
    uint64_t grad_accum_ = 1, accum_count_ = 0, step_ = 0;
};

} // namespace optim
} // namespace nabla

#endif
