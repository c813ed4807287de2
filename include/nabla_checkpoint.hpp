// nabla_checkpoint.hpp -- C++ mirror of nabla-train's checkpoints
// (nabla-train/src/checkpoint.rs:34-231) over the C ABI of nabla_optim.h.  Header-only.
//
// A checkpoint directory holds params.nbla and optim.nbla (tensor files, written and
// read by the library straight from device memory: nbo_nbla_*_list, nbo_optim_*_state)
// and meta.txt (key=value lines: version, epoch, step, grad_accum, rng.state, the
// optimizer's meta pairs of optim/core.rs:263-324, the schedule's pairs of
// core.rs:175-252, the scaler's state).  Floats are written the way Rust's Display prints
// an f64: the shortest digits that round-trip, never in scientific notation.
#ifndef NABLA_CHECKPOINT_HPP
#define NABLA_CHECKPOINT_HPP

#include <charconv>
#include <fstream>
#include <limits>
#include <map>
#include <optional>
#include <sstream>
#include <string>
#include <type_traits>
#include <sys/stat.h>
#include <utility>
#include <vector>

#include "nabla_groups.hpp"

namespace nabla {
namespace optim {

// checkpoint.rs:14-20: Io / State / Optim / Parse
struct CheckpointError : std::runtime_error {
    std::string kind;
    CheckpointError(std::string k, const std::string &m) : std::runtime_error(k + ": " + m), kind(std::move(k)) {}
};

// trainer.rs TrainState
struct TrainState {
    uint64_t epoch = 0, step = 0, grad_accum = 1;
    std::optional<uint64_t> rng_state;
};

// optim/core.rs:118-122
struct ScheduleState {
    double base_lr;
    LrSchedule schedule;
};

using Pairs = std::vector<std::pair<std::string, std::string>>;
using MetaMap = std::map<std::string, std::string>;

// Rust's `f64::to_string()`
inline std::string rust_f64_str(double x)
{
    if (x != x) return "NaN";
    if (x == std::numeric_limits<double>::infinity()) return "inf";
    if (x == -std::numeric_limits<double>::infinity()) return "-inf";
    char buf[400];
    const auto r = std::to_chars(buf, buf + sizeof(buf), x, std::chars_format::fixed);
    return std::string(buf, r.ptr);
}

namespace detail {
inline const std::string &get(const MetaMap &m, const std::string &key)
{
    const auto it = m.find(key);
    if (it == m.end()) throw StateError("missing " + key);
    return it->second;
}
// what Rust's str::parse::<f64> accepts, as far as these files need it: an optional
// sign, then a decimal or scientific number, "inf", "infinity" or "nan"; nothing around it
inline double parse_f64(const MetaMap &m, const std::string &key)
{
    const std::string &v = get(m, key);
    const char *p = v.c_str(), *end = p + v.size();
    if (p != end && *p == '+') p++;
    double out = 0.0;
    const auto r = std::from_chars(p, end, out);
    if (p == end || r.ec != std::errc() || r.ptr != end) throw StateError("bad " + key + ": " + v);
    return out;
}
inline uint64_t parse_usize(const MetaMap &m, const std::string &key)
{
    const std::string &v = get(m, key);
    const char *p = v.c_str(), *end = p + v.size();
    if (p != end && *p == '+') p++;
    uint64_t out = 0;
    const auto r = std::from_chars(p, end, out);
    if (p == end || r.ec != std::errc() || r.ptr != end) throw StateError("bad " + key + ": " + v);
    return out;
}
inline const char *kind_str(OptimKind k)
{
    return k == OptimKind::AdamW ? "adamw" : k == OptimKind::Adam ? "adam" : "sgd";
}
} // namespace detail

// optim/core.rs:263-277
inline Pairs optim_meta_pairs(const OptimMeta &m)
{
    return {{"optim.kind", detail::kind_str(m.kind)},
            {"optim.lr", rust_f64_str(m.lr)},
            {"optim.beta1", rust_f64_str(m.beta1)},
            {"optim.beta2", rust_f64_str(m.beta2)},
            {"optim.eps", rust_f64_str(m.eps)},
            {"optim.weight_decay", rust_f64_str(m.weight_decay)},
            {"optim.momentum", rust_f64_str(m.momentum)},
            {"optim.step_count", std::to_string(m.step_count)}};
}

// optim/core.rs:279-308
inline OptimMeta parse_optim_meta(const MetaMap &m)
{
    const std::string &kind = detail::get(m, "optim.kind");
    OptimKind k;
    if (kind == "adamw") k = OptimKind::AdamW;
    else if (kind == "adam") k = OptimKind::Adam;
    else if (kind == "sgd") k = OptimKind::Sgd;
    else throw StateError("bad optim.kind: " + kind);
    return {k,
            detail::parse_f64(m, "optim.lr"),
            detail::parse_f64(m, "optim.beta1"),
            detail::parse_f64(m, "optim.beta2"),
            detail::parse_f64(m, "optim.eps"),
            detail::parse_f64(m, "optim.weight_decay"),
            detail::parse_f64(m, "optim.momentum"),
            detail::parse_usize(m, "optim.step_count")};
}

// optim/core.rs:175-216
inline Pairs schedule_pairs(const ScheduleState &st)
{
    const LrSchedule &s = st.schedule;
    Pairs out = {{"schedule.enabled", "1"}, {"schedule.base_lr", rust_f64_str(st.base_lr)}};
    switch (s.kind) {
    case LrSchedule::Cosine:
        out.insert(out.end(), {{"schedule.kind", "cosine"},
                               {"schedule.warmup_steps", std::to_string(s.warmup_steps)},
                               {"schedule.total_steps", std::to_string(s.total_steps)},
                               {"schedule.min_lr", rust_f64_str(s.min_lr)}});
        break;
    case LrSchedule::Linear:
        out.insert(out.end(), {{"schedule.kind", "linear"},
                               {"schedule.warmup_steps", std::to_string(s.warmup_steps)},
                               {"schedule.total_steps", std::to_string(s.total_steps)}});
        break;
    case LrSchedule::OneCycle:
        out.insert(out.end(), {{"schedule.kind", "onecycle"},
                               {"schedule.max_lr", rust_f64_str(s.max_lr)},
                               {"schedule.total_steps", std::to_string(s.total_steps)},
                               {"schedule.pct_start", rust_f64_str(s.pct_start)}});
        break;
    default:
        out.insert(out.end(), {{"schedule.kind", "step"},
                               {"schedule.step_size", std::to_string(s.step_size)},
                               {"schedule.gamma", rust_f64_str(s.gamma)}});
    }
    return out;
}

// optim/core.rs:218-252
inline std::optional<ScheduleState> parse_schedule_state(const MetaMap &m)
{
    const auto en = m.find("schedule.enabled");
    if (en == m.end() || en->second != "1") return std::nullopt;
    const double base_lr = detail::parse_f64(m, "schedule.base_lr");
    const std::string &kind = detail::get(m, "schedule.kind");
    if (kind == "cosine")
        return ScheduleState{base_lr, LrSchedule::cosine(detail::parse_usize(m, "schedule.warmup_steps"),
                                                         detail::parse_usize(m, "schedule.total_steps"),
                                                         detail::parse_f64(m, "schedule.min_lr"))};
    if (kind == "linear")
        return ScheduleState{base_lr, LrSchedule::linear(detail::parse_usize(m, "schedule.warmup_steps"),
                                                         detail::parse_usize(m, "schedule.total_steps"))};
    if (kind == "onecycle")
        return ScheduleState{base_lr, LrSchedule::one_cycle(detail::parse_f64(m, "schedule.max_lr"),
                                                            detail::parse_usize(m, "schedule.total_steps"),
                                                            detail::parse_f64(m, "schedule.pct_start"))};
    if (kind == "step")
        return ScheduleState{base_lr, LrSchedule::step(detail::parse_usize(m, "schedule.step_size"),
                                                       detail::parse_f64(m, "schedule.gamma"))};
    throw StateError("bad schedule.kind: " + kind);
}

// OptimState::meta_pairs / load_meta_pairs: the defaults (core.rs:71-78) for Sgd / Adam /
// AdamW, GroupOptimizer's own (groups.rs:368-420)
inline Pairs meta_pairs_of(Optimizer &o) { return optim_meta_pairs(o.meta()); }
inline void load_meta_pairs_into(Optimizer &o, const MetaMap &m) { o.load_meta(parse_optim_meta(m)); }
inline Pairs meta_pairs_of(GroupOptimizer &o)
{
    Pairs out = {{"optim.group.count", std::to_string(o.groups())}};
    for (size_t gi = 0; gi < o.groups(); gi++) {
        const std::string p = "optim.group." + std::to_string(gi) + ".";
        out.push_back({p + "name", o.group_name(gi)});
        for (const auto &kv : optim_meta_pairs(o.group_optimizer(gi).meta()))
            out.push_back({p + kv.first.substr(6), kv.second}); // "optim.lr" -> "optim.group.{gi}.lr"
    }
    return out;
}
inline void load_meta_pairs_into(GroupOptimizer &o, const MetaMap &m)
{
    if (detail::parse_usize(m, "optim.group.count") != o.groups()) throw StateError("optim.group.count mismatch");
    for (size_t gi = 0; gi < o.groups(); gi++) {
        const std::string p = "optim.group." + std::to_string(gi) + ".";
        if (detail::get(m, p + "name") != o.group_name(gi))
            throw StateError("optim.group." + std::to_string(gi) + ".name mismatch");
        const std::string &kind = detail::get(m, p + "kind");
        OptimKind k;
        if (kind == "adamw") k = OptimKind::AdamW;
        else if (kind == "adam") k = OptimKind::Adam;
        else if (kind == "sgd") k = OptimKind::Sgd;
        else throw StateError("bad optim.kind: " + kind);
        o.group_optimizer(gi).load_meta({k, detail::parse_f64(m, p + "lr"), detail::parse_f64(m, p + "beta1"),
                                         detail::parse_f64(m, p + "beta2"), detail::parse_f64(m, p + "eps"),
                                         detail::parse_f64(m, p + "weight_decay"), detail::parse_f64(m, p + "momentum"),
                                         detail::parse_usize(m, p + "step_count")});
    }
    o.refresh_base_lr();
}

// checkpoint.rs:107-150
template <typename Opt>
void write_meta(const std::string &path, Opt &optimizer, GradScaler *scaler, const ScheduleState *schedule,
                const TrainState &state)
{
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    if (!f) throw CheckpointError("Io", path + ": cannot create");
    f << "version=1\n"
      << "epoch=" << state.epoch << "\n"
      << "step=" << state.step << "\n"
      << "grad_accum=" << state.grad_accum << "\n";
    if (state.rng_state) f << "rng.state=" << *state.rng_state << "\n";
    for (const auto &kv : meta_pairs_of(optimizer)) f << kv.first << "=" << kv.second << "\n";
    if (schedule)
        for (const auto &kv : schedule_pairs(*schedule)) f << kv.first << "=" << kv.second << "\n";
    if (scaler) {
        const GradScalerState st = scaler->state();
        f << "scaler.enabled=1\n"
          << "scaler.scale=" << rust_f64_str(st.scale) << "\n"
          << "scaler.growth_factor=" << rust_f64_str(st.growth_factor) << "\n"
          << "scaler.backoff_factor=" << rust_f64_str(st.backoff_factor) << "\n"
          << "scaler.growth_interval=" << st.growth_interval << "\n"
          << "scaler.consecutive_ok=" << st.consecutive_ok << "\n";
    } else {
        f << "scaler.enabled=0\n";
    }
    if (!f.flush()) throw CheckpointError("Io", path + ": write failed");
}

struct MetaContents {
    std::optional<GradScalerState> scaler;
    TrainState state;
    std::optional<ScheduleState> schedule;
};

// checkpoint.rs:152-212; the optimizer's hyper-parameters and step_count are loaded into it
template <typename Opt> MetaContents read_meta(const std::string &path, Opt &optimizer)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) throw CheckpointError("Io", path + ": cannot open");
    MetaMap m;
    std::string line;
    while (std::getline(f, line)) {
        if (!line.empty() && line.back() == '\r') line.pop_back(); // str::lines drops "\r\n" too
        if (line.find_first_not_of(" \t") == std::string::npos) continue;
        const size_t eq = line.find('=');
        if (eq == std::string::npos) throw CheckpointError("Parse", line);
        m[line.substr(0, eq)] = line.substr(eq + 1);
    }
    auto parse = [&](auto fn, const std::string &key) {
        try {
            return fn(m, key);
        } catch (const StateError &e) {
            throw CheckpointError("Parse", e.what());
        }
    };
    MetaContents out;
    out.state.epoch = parse(detail::parse_usize, "epoch");
    out.state.step = parse(detail::parse_usize, "step");
    out.state.grad_accum = parse(detail::parse_usize, "grad_accum");
    try {
        load_meta_pairs_into(optimizer, m);
    } catch (const StateError &e) {
        throw CheckpointError("Optim", e.what());
    }
    bool scaler_enabled = false;
    try {
        scaler_enabled = detail::parse_usize(m, "scaler.enabled") == 1;
    } catch (const StateError &) {
    }
    if (scaler_enabled)
        out.scaler = GradScalerState{parse(detail::parse_f64, "scaler.scale"),
                                     parse(detail::parse_f64, "scaler.growth_factor"),
                                     parse(detail::parse_f64, "scaler.backoff_factor"),
                                     parse(detail::parse_usize, "scaler.growth_interval"),
                                     parse(detail::parse_usize, "scaler.consecutive_ok")};
    try {
        out.state.rng_state = detail::parse_usize(m, "rng.state");
    } catch (const StateError &) {
    }
    try {
        out.schedule = parse_schedule_state(m);
    } catch (const StateError &e) {
        throw CheckpointError("Optim", e.what());
    }
    return out;
}

namespace detail {
// an optimizer that reads and writes the module's params.nbla itself (GroupOptimizer: its groups
// may hold master weights for some of the parameters)
template <typename Opt, typename = void> struct has_params_file : std::false_type {};
template <typename Opt>
struct has_params_file<Opt, std::void_t<decltype(std::declval<Opt &>().save_params(
                                std::declval<const std::string &>(), std::declval<const std::vector<Tensor> &>(),
                                std::declval<const std::vector<std::string> &>()))>> : std::true_type {};

template <typename F> void tensor_file(const char *kind, F &&call)
{
    try {
        call();
    } catch (const StateError &e) {
        throw CheckpointError(kind, e.what());
    } catch (const Panic &e) {
        throw CheckpointError("State", e.what());
    } catch (const RuntimeError &e) {
        throw CheckpointError(e.status == NBO_ERR_IO ? "Io" : "State", e.what());
    }
}
} // namespace detail

// checkpoint.rs:38-69.  `params` / `names` are the module's state_dict.  A mixed-precision
// optimizer's checkpoint keeps its f32 master weights as the parameters, under the parameters'
// names: the 16-bit tensors are derived from them and could not restore them.
template <typename Opt>
void save_checkpoint(const std::string &dir, TensorList &params, const std::vector<std::string> &names, Opt &optimizer,
                     GradScaler *scaler, const ScheduleState *schedule, const TrainState &state)
{
    ::mkdir(dir.c_str(), 0777); // fs::create_dir_all for the last component; an existing directory is fine
    bool from_master = false;
    if constexpr (std::is_base_of_v<Optimizer, Opt>) {
        if (optimizer.keeps_master()) {
            detail::tensor_file("State", [&] { optimizer.save_master(dir + "/params.nbla", names); });
            from_master = true;
        }
    } else if constexpr (detail::has_params_file<Opt>::value) {
        if (optimizer.keeps_master()) {
            detail::tensor_file("State", [&] { optimizer.save_params(dir + "/params.nbla", params.tensors(), names); });
            from_master = true;
        }
    }
    if (!from_master) detail::tensor_file("State", [&] { save_tensors(dir + "/params.nbla", params, names); });
    detail::tensor_file("Optim", [&] { optimizer.save_state(dir + "/optim.nbla"); });
    write_meta(dir + "/meta.txt", optimizer, scaler, schedule, state);
}

// checkpoint.rs:71-105: parameters into `params` (load_state_dict), moments and meta into
// `optimizer`, the scaler's state into `scaler` if both are there.
template <typename Opt>
void load_checkpoint(const std::string &dir, TensorList &params, const std::vector<std::string> &names, Opt &optimizer,
                     GradScaler *scaler, std::optional<ScheduleState> &schedule, TrainState &state)
{
    bool into_master = false;
    if constexpr (std::is_base_of_v<Optimizer, Opt>) {
        if (optimizer.keeps_master()) { // master weights into the optimizer, the 16-bit `params` narrowed from them
            detail::tensor_file("State", [&] {
                optimizer.load_master(dir + "/params.nbla", names);
                optimizer.params_from_master(params);
            });
            into_master = true;
        }
    } else if constexpr (detail::has_params_file<Opt>::value) {
        if (optimizer.keeps_master()) { // each group's master weights, then its 16-bit tensors narrowed from them
            detail::tensor_file("State", [&] { optimizer.load_params(dir + "/params.nbla", params.tensors(), names); });
            into_master = true;
        }
    }
    if (!into_master) detail::tensor_file("State", [&] { load_state_dict(dir + "/params.nbla", params, names); });
    detail::tensor_file("Optim", [&] { optimizer.load_state(dir + "/optim.nbla"); });
    MetaContents meta = read_meta(dir + "/meta.txt", optimizer);
    if (scaler && meta.scaler) scaler->load_state(*meta.scaler);
    state = meta.state;
    schedule = meta.schedule;
}

} // namespace optim
} // namespace nabla

#endif
