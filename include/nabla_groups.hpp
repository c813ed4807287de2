// nabla_groups.hpp -- C++ mirror of nabla-train's parameter groups
// (nabla-train/src/optim/groups.rs:11-313) over the C ABI of nabla_optim.h.  Header-only.
//
// Name patterns select which per-group Sgd / Adam / AdamW a parameter belongs to (first
// matching group wins, then the default group).  Where the reference clones parameters
// into per-group vectors and back every step (groups.rs:281-292), each group here simply
// holds the list of its own tensors.
#ifndef NABLA_GROUPS_HPP
#define NABLA_GROUPS_HPP

#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "nabla_optim.hpp"

namespace nabla {
namespace optim {

// groups.rs:11-17
struct ParamMatch {
    enum Kind { Equals, Prefix, Suffix, Contains } kind;
    std::string text;
    bool matches(const std::string &name) const
    {
        switch (kind) {
        case Equals: return name == text;
        case Prefix: return name.compare(0, text.size(), text) == 0 && name.size() >= text.size();
        case Suffix:
            return name.size() >= text.size() && name.compare(name.size() - text.size(), text.size(), text) == 0;
        default: return name.find(text) != std::string::npos;
        }
    }
};

// groups.rs:19-38
struct ParamSelector {
    bool all = true;
    std::vector<ParamMatch> any;
    static ParamSelector All() { return {}; }
    static ParamSelector Any(std::vector<ParamMatch> m)
    {
        ParamSelector s;
        s.all = false;
        s.any = std::move(m);
        return s;
    }
    bool matches(const std::string &name) const
    {
        if (all) return true;
        for (const ParamMatch &m : any)
            if (m.matches(name)) return true;
        return false;
    }
};

// groups.rs:40-132
struct ParamGroupConfig {
    std::string name;
    ParamSelector selector;
    OptimKind kind;
    double lr, weight_decay = 0.0, momentum = 0.0, beta1 = 0.9, beta2 = 0.999, eps = 1e-8;
    static ParamGroupConfig adamw(std::string name, ParamSelector sel, double lr, double weight_decay)
    {
        ParamGroupConfig c{std::move(name), std::move(sel), OptimKind::AdamW, lr};
        c.weight_decay = weight_decay;
        return c;
    }
    static ParamGroupConfig adam(std::string name, ParamSelector sel, double lr)
    {
        return ParamGroupConfig{std::move(name), std::move(sel), OptimKind::Adam, lr};
    }
    static ParamGroupConfig sgd(std::string name, ParamSelector sel, double lr, double momentum, double weight_decay)
    {
        ParamGroupConfig c{std::move(name), std::move(sel), OptimKind::Sgd, lr};
        c.momentum = momentum, c.weight_decay = weight_decay, c.beta1 = c.beta2 = c.eps = 0.0;
        return c;
    }
};

// groups.rs:134-150
enum class ParamExclusionPreset { Bias, Norm, Embedding };
inline std::vector<std::string> preset_patterns(ParamExclusionPreset p)
{
    switch (p) {
    case ParamExclusionPreset::Bias: return {"bias"};
    case ParamExclusionPreset::Norm: return {"norm", "bn", "ln"};
    default: return {"embed", "embedding"};
    }
}

class GroupOptimizer {
public:
    // groups.rs:168-226; throws StateError("nabla-train: group assignment incomplete")
    static GroupOptimizer from_named_params(const std::vector<std::pair<std::string, Tensor>> &named,
                                            const std::vector<ParamGroupConfig> &groups,
                                            const ParamGroupConfig *default_group,
                                            nbo_dtype state_dtype = NBO_DT_F32, bool master = false)
    {
        std::vector<std::pair<ParamGroupConfig, std::vector<size_t>>> buckets;
        for (const ParamGroupConfig &g : groups) buckets.push_back({g, {}});
        std::vector<size_t> default_idx;
        for (size_t i = 0; i < named.size(); i++) {
            bool placed = false;
            for (auto &b : buckets)
                if (b.first.selector.matches(named[i].first)) {
                    b.second.push_back(i);
                    placed = true;
                    break;
                }
            if (!placed) {
                if (!default_group) throw StateError("nabla-train: group assignment incomplete");
                default_idx.push_back(i);
            }
        }
        if (default_group) buckets.push_back({*default_group, default_idx});
        GroupOptimizer out;
        out.param_count_ = named.size();
        for (auto &b : buckets) {
            if (b.second.empty()) continue;
            Shapes shapes;
            for (size_t i : b.second) shapes.push_back(named[i].second.shape());
            out.groups_.push_back(Entry{b.second, b.first.name, b.first.lr, make(b.first, shapes, state_dtype, master),
                                        nullptr, nullptr, {}, {}});
        }
        out.base_lr_ = out.groups_.empty() ? 1.0 : out.groups_.front().base_lr;
        return out;
    }

    // groups.rs:228-242
    static GroupOptimizer adamw_with_decay_exclusions(const std::vector<std::pair<std::string, Tensor>> &named,
                                                      double lr, double weight_decay,
                                                      const std::vector<std::string> &exclude,
                                                      nbo_dtype state_dtype = NBO_DT_F32, bool master = false)
    {
        std::vector<ParamMatch> m;
        for (const std::string &s : exclude) {
            m.push_back({ParamMatch::Suffix, s});
            m.push_back({ParamMatch::Contains, s});
        }
        const ParamGroupConfig no_decay = ParamGroupConfig::adamw("no_decay", ParamSelector::Any(m), lr, 0.0);
        const ParamGroupConfig decay = ParamGroupConfig::adamw("decay", ParamSelector::All(), lr, weight_decay);
        return from_named_params(named, {no_decay}, &decay, state_dtype, master);
    }

    // groups.rs:244-261
    static GroupOptimizer adamw_with_decay_presets(const std::vector<std::pair<std::string, Tensor>> &named, double lr,
                                                   double weight_decay,
                                                   const std::vector<ParamExclusionPreset> &presets,
                                                   nbo_dtype state_dtype = NBO_DT_F32, bool master = false)
    {
        std::vector<std::string> patterns;
        for (ParamExclusionPreset p : presets)
            for (const std::string &s : preset_patterns(p)) patterns.push_back(s);
        return adamw_with_decay_exclusions(named, lr, weight_decay, patterns, state_dtype, master);
    }

    size_t groups() const { return groups_.size(); }
    const std::vector<size_t> &group_indices(size_t g) const { return groups_[g].indices; }
    Optimizer &group_optimizer(size_t g) { return *groups_[g].optimizer; }
    const std::string &group_name(size_t g) const { return groups_[g].name; }
    // groups.rs:416-418: after the groups' metas were loaded, the base lr is the first group's
    void refresh_base_lr()
    {
        if (!groups_.empty()) base_lr_ = groups_.front().optimizer->meta().lr;
    }

    // trait Optimizer, groups.rs:268-313
    void step(const std::vector<Tensor> &params, const std::vector<Tensor> &grads)
    {
        bind(params, grads);
        for (Entry &g : groups_) g.optimizer->step(*g.params, *g.grads);
    }
    // the Trainer tail with one unscale / found-inf / clip decision over all gradients
    void fused_step(const std::vector<Tensor> &params, const std::vector<Tensor> &grads, GradScaler *scaler,
                    double max_norm, bool zero_grads = false, bool zero_on_skip = false)
    {
        bind(params, grads);
        if (!all_grads_ || all_key_ != key_of(grads)) {
            all_grads_.reset(new TensorList(grads));
            all_key_ = key_of(grads);
        }
        std::vector<nbo_optim *> opts;
        std::vector<nbo_list *> pl, gl;
        for (Entry &g : groups_) {
            opts.push_back(g.optimizer->handle());
            pl.push_back(g.params->handle());
            gl.push_back(g.grads->handle());
        }
        check(nbo_fused_step_groups(groups_.size(), opts.data(), pl.data(), gl.data(),
                                    scaler ? scaler->handle() : nullptr, all_grads_->handle(), max_norm,
                                    (zero_grads ? NBO_STEP_ZERO_GRADS : 0u) | (zero_on_skip ? NBO_STEP_ZERO_ON_SKIP : 0u)));
    }
    // the same over gradients whose sum of squares is already known (nbo_unscale_accumulate)
    void fused_step_norm(const std::vector<Tensor> &params, const std::vector<Tensor> &grads, double sumsq,
                         double max_norm, bool zero_grads = false)
    {
        bind(params, grads);
        std::vector<nbo_optim *> opts;
        std::vector<nbo_list *> pl, gl;
        for (Entry &g : groups_) {
            opts.push_back(g.optimizer->handle());
            pl.push_back(g.params->handle());
            gl.push_back(g.grads->handle());
        }
        check(nbo_fused_step_groups_norm(groups_.size(), opts.data(), pl.data(), gl.data(), max_norm, sumsq,
                                         zero_grads ? NBO_STEP_ZERO_GRADS : 0u));
    }
    // optim.nbla of a checkpoint with the keys of groups.rs:320-350 ("g{gi}.m{i}", "g{gi}.v{i}")
    void save_state(const std::string &path) { check(nbo_optim_save_state_groups(groups_.size(), handles().data(), path.c_str())); }
    void load_state(const std::string &path) { check(nbo_optim_load_state_groups(groups_.size(), handles().data(), path.c_str())); }
    // params.nbla of a checkpoint (checkpoint.rs:54-58, 88-90) for the module whose parameters
    // these groups hold: a group that keeps master weights writes (receives) those under the
    // parameters' names -- the 16-bit tensors are derived from them and are narrowed from them
    // again after loading -- the other groups their tensors as they are.
    bool keeps_master() const
    {
        for (const Entry &g : groups_)
            if (g.optimizer->keeps_master()) return true;
        return false;
    }
    void save_params(const std::string &path, const std::vector<Tensor> &params, const std::vector<std::string> &names)
    {
        params_file(nbo_optim_save_params_groups, path, params, names);
    }
    void load_params(const std::string &path, const std::vector<Tensor> &params, const std::vector<std::string> &names)
    {
        params_file(nbo_optim_load_params_groups, path, params, names);
        for (Entry &g : groups_)
            if (g.optimizer->keeps_master()) g.optimizer->params_from_master(*g.params);
    }
    void reset()
    {
        for (Entry &g : groups_) g.optimizer->reset();
    }
    // groups.rs:302-312: every group's lr follows its own base in the same proportion
    void set_lr(double lr)
    {
        for (Entry &g : groups_) g.optimizer->set_lr(base_lr_ <= 0.0 ? lr : g.base_lr * (lr / base_lr_));
    }

private:
    struct Entry {
        std::vector<size_t> indices;
        std::string name;
        double base_lr;
        std::shared_ptr<Optimizer> optimizer;
        std::shared_ptr<TensorList> params, grads;
        std::vector<uint64_t> pkey, gkey;
    };
    static std::shared_ptr<Optimizer> make(const ParamGroupConfig &c, const Shapes &shapes, nbo_dtype dt, bool master)
    {
        if (c.kind == OptimKind::AdamW) {
            auto o = std::make_shared<AdamW>(c.lr, shapes, dt, master);
            o->beta1(c.beta1).beta2(c.beta2).eps(c.eps).weight_decay(c.weight_decay);
            return o;
        }
        if (c.kind == OptimKind::Adam) {
            auto o = std::make_shared<Adam>(c.lr, shapes, dt, master);
            o->beta1(c.beta1).beta2(c.beta2).eps(c.eps);
            return o;
        }
        auto o = std::make_shared<Sgd>(c.lr, shapes, dt, master);
        o->momentum(c.momentum).weight_decay(c.weight_decay);
        return o;
    }
    std::vector<nbo_optim *> handles()
    {
        std::vector<nbo_optim *> h;
        for (Entry &g : groups_) h.push_back(g.optimizer->handle());
        return h;
    }
    // what a list was built from: address, shape and element type of every tensor
    static std::vector<uint64_t> key_of(const std::vector<Tensor> &t)
    {
        std::vector<uint64_t> k;
        for (const Tensor &x : t) {
            k.push_back((uint64_t)(uintptr_t)x.data);
            k.push_back(x.rows);
            k.push_back(x.cols);
            k.push_back((uint64_t)x.dtype);
        }
        return k;
    }
    void bind_params(const std::vector<Tensor> &params)
    {
        if (params.size() != param_count_) throw Panic("nabla-train: GroupOptimizer param count mismatch");
        for (Entry &g : groups_) {
            std::vector<Tensor> p;
            for (size_t i : g.indices) p.push_back(params[i]);
            if (!g.params || g.pkey != key_of(p)) g.params.reset(new TensorList(p)), g.pkey = key_of(p);
        }
    }
    void bind(const std::vector<Tensor> &params, const std::vector<Tensor> &grads)
    {
        if (params.size() != grads.size()) throw Panic("nabla-train: GroupOptimizer params/grads length mismatch");
        bind_params(params);
        for (Entry &g : groups_) {
            std::vector<Tensor> q;
            for (size_t i : g.indices) q.push_back(grads[i]);
            if (!g.grads || g.gkey != key_of(q)) g.grads.reset(new TensorList(q)), g.gkey = key_of(q);
        }
    }
    template <typename Call>
    void params_file(Call call, const std::string &path, const std::vector<Tensor> &params,
                     const std::vector<std::string> &names)
    {
        if (names.size() != params.size()) throw Panic("nabla-train: GroupOptimizer param count mismatch");
        bind_params(params);
        std::vector<uint32_t> group_of(params.size()), index_in(params.size());
        std::vector<nbo_list *> lists;
        for (size_t g = 0; g < groups_.size(); g++) {
            lists.push_back(groups_[g].params->handle());
            for (size_t k = 0; k < groups_[g].indices.size(); k++)
                group_of[groups_[g].indices[k]] = (uint32_t)g, index_in[groups_[g].indices[k]] = (uint32_t)k;
        }
        std::vector<const char *> raw;
        for (const std::string &n : names) raw.push_back(n.c_str());
        check(call(groups_.size(), handles().data(), lists.data(), params.size(), group_of.data(), index_in.data(),
                   raw.data(), path.c_str()));
    }
    std::vector<Entry> groups_;
    size_t param_count_ = 0;
    double base_lr_ = 1.0;
    std::shared_ptr<TensorList> all_grads_;
    std::vector<uint64_t> all_key_;
};

} // namespace optim
} // namespace nabla

#endif
