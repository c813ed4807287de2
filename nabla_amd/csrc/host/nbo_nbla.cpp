// NBLA tensor files -- the bulk part of nabla-train's checkpoints (params.nbla,
// optim.nbla; nabla-train/src/checkpoint.rs:34-105) in the format of
// nabla-ml/src/module/core.rs:21,66-120: "NBLA", u32 count, then per tensor u32 name
// length, UTF-8 name, u32 rows, u32 cols and rows*cols f64 values, all little-endian.
// Values are f64 whatever the element type (T::to_f64 on save, T::from_f64 on load), so
// f32 and bf16 state round-trips exactly.  Device memory is streamed through a bounded
// host buffer; nothing here needs the whole tensor on the host.
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <memory>

#include "nbo_host.hpp"

using namespace nbo;

namespace {

constexpr size_t kChunkElems = (size_t)1 << 20; // elements per streaming step

struct FileCloser {
    void operator()(std::FILE *f) const
    {
        if (f) std::fclose(f);
    }
};
using FilePtr = std::unique_ptr<std::FILE, FileCloser>;

FilePtr open_file(const char *path, const char *mode)
{
    if (!path) fail(NBO_ERR_ARG, "null path");
    FilePtr f(std::fopen(path, mode));
    if (!f) fail(NBO_ERR_IO, std::string(path) + ": " + std::strerror(errno));
    return f;
}

void write_all(std::FILE *f, const void *p, size_t n)
{
    if (n && std::fwrite(p, 1, n, f) != n) fail(NBO_ERR_IO, std::string("write failed: ") + std::strerror(errno));
}

void read_exact(std::FILE *f, void *p, size_t n)
{
    if (n && std::fread(p, 1, n, f) != n) fail(NBO_ERR_IO, "failed to fill whole buffer"); // io::ErrorKind::UnexpectedEof
}

void write_u32(std::FILE *f, uint32_t v)
{
    const unsigned char b[4] = {(unsigned char)v, (unsigned char)(v >> 8), (unsigned char)(v >> 16),
                                (unsigned char)(v >> 24)};
    write_all(f, b, 4);
}

uint32_t read_u32(std::FILE *f)
{
    unsigned char b[4];
    read_exact(f, b, 4);
    return (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24);
}

size_t dtype_bytes(int dtype) { return dtype == NBO_DT_F64 ? 8 : is_half(dtype) ? 2 : 4; }

// half::bf16::from_f32 / f32::from(bf16) on the host (common/scalar/mod.rs:338-344)
uint16_t bf16_from_f32(float v)
{
    uint32_t x;
    std::memcpy(&x, &v, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    return (uint16_t)((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

float bf16_to_f32(uint16_t h)
{
    const uint32_t x = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// half::f16::from_f32 / f32::from(f16) on the host: IEEE binary16, round to nearest even,
// subnormals kept, overflow to infinity, NaN payloads truncated with the quiet bit set.
uint16_t f16_from_f32(float v)
{
    uint32_t x;
    std::memcpy(&x, &v, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, ax = x & 0x7FFFFFFFu;
    if (ax > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x03FFu));
    if (ax >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); // 65536 and above, infinity
    if (ax >= 0x38800000u) {                                  // normal in binary16 (2^-14 and above)
        const uint32_t r = ax - 0x38000000u;                  // exponent rebiased from 127 to 15
        return (uint16_t)(sign | ((r + 0x0FFFu + ((r >> 13) & 1u)) >> 13)); // a carry into exponent 31 is infinity
    }
    if (ax <= 0x33000000u) return (uint16_t)sign; // up to 2^-25 (the tie to zero included)
    const uint32_t man = (ax & 0x007FFFFFu) | 0x00800000u, shift = 126u - (ax >> 23); // 14..24
    const uint32_t rem = man & ((1u << shift) - 1u), half_way = 1u << (shift - 1u);
    uint32_t q = man >> shift; // multiples of 2^-24
    if (rem > half_way || (rem == half_way && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

float f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x03FFu;
    uint32_t x;
    if (e == 0) {
        const float sub = (float)m * 5.9604644775390625e-08f; // m * 2^-24, exact
        std::memcpy(&x, &sub, 4);
        x |= sign;
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112u) << 23) | (m << 13);
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// T::to_f64 over `n` raw elements
void widen(int dtype, const void *raw, double *out, size_t n)
{
    if (dtype == NBO_DT_F64) std::memcpy(out, raw, n * 8);
    else if (dtype == NBO_DT_F32)
        for (size_t i = 0; i < n; i++) out[i] = (double)((const float *)raw)[i];
    else if (dtype == NBO_DT_F16)
        for (size_t i = 0; i < n; i++) out[i] = (double)f16_to_f32(((const uint16_t *)raw)[i]);
    else
        for (size_t i = 0; i < n; i++) out[i] = (double)bf16_to_f32(((const uint16_t *)raw)[i]);
}

// T::from_f64 over `n` values (f32: one rounding; bf16 / f16: through f32, scalar/mod.rs:338-340)
void narrow(int dtype, const double *in, void *raw, size_t n)
{
    if (dtype == NBO_DT_F64) std::memcpy(raw, in, n * 8);
    else if (dtype == NBO_DT_F32)
        for (size_t i = 0; i < n; i++) ((float *)raw)[i] = (float)in[i];
    else if (dtype == NBO_DT_F16)
        for (size_t i = 0; i < n; i++) ((uint16_t *)raw)[i] = f16_from_f32((float)in[i]);
    else
        for (size_t i = 0; i < n; i++) ((uint16_t *)raw)[i] = bf16_from_f32((float)in[i]);
}

struct Buffers {
    std::vector<unsigned char> raw;
    std::vector<double> f64;
    Buffers() : raw(kChunkElems * 8), f64(kChunkElems) {}
};

void write_header(std::FILE *f, const std::string &name, uint64_t rows, uint64_t cols)
{
    if (rows > 0xFFFFFFFFull || cols > 0xFFFFFFFFull || name.size() > 0xFFFFFFFFull)
        fail(NBO_ERR_TOO_LARGE, "tensor '" + name + "' does not fit the file format's 32-bit fields");
    write_u32(f, (uint32_t)name.size());
    write_all(f, name.data(), name.size());
    write_u32(f, (uint32_t)rows);
    write_u32(f, (uint32_t)cols);
}

// device elements -> f64 little-endian values in the file
void stream_out(std::FILE *f, const void *dev, int dtype, uint64_t n, Buffers &b)
{
    Runtime &rt = Runtime::get();
    const size_t eb = dtype_bytes(dtype);
    for (uint64_t done = 0; done < n;) {
        const size_t k = (size_t)std::min<uint64_t>(kChunkElems, n - done);
        rt.read_back(b.raw.data(), (const char *)dev + done * eb, k * eb);
        widen(dtype, b.raw.data(), b.f64.data(), k);
        write_all(f, b.f64.data(), k * 8); // the build targets little-endian hosts only
        done += k;
    }
}

// f64 values in the file -> device elements
void stream_in(std::FILE *f, void *dev, int dtype, uint64_t n, Buffers &b)
{
    Runtime &rt = Runtime::get();
    const size_t eb = dtype_bytes(dtype);
    for (uint64_t done = 0; done < n;) {
        const size_t k = (size_t)std::min<uint64_t>(kChunkElems, n - done);
        read_exact(f, b.f64.data(), k * 8);
        narrow(dtype, b.f64.data(), b.raw.data(), k);
        rt.upload((char *)dev + done * eb, b.raw.data(), k * eb);
        done += k;
    }
}

struct Entry {
    std::string name;
    uint64_t rows, cols;
    long data_offset;
};

// Reads the file's table of contents, skipping over the values.  Lengths come from the
// file, so each is checked against what is left of it before anything is sized by it; a
// file that ends early is the reference's read_exact error.
std::vector<Entry> read_index(std::FILE *f)
{
    if (std::fseek(f, 0, SEEK_END) != 0) fail(NBO_ERR_IO, "seek failed");
    const long file_size = std::ftell(f);
    if (file_size < 0 || std::fseek(f, 0, SEEK_SET) != 0) fail(NBO_ERR_IO, "seek failed");
    const auto left = [&]() -> uint64_t {
        const long pos = std::ftell(f);
        if (pos < 0) fail(NBO_ERR_IO, "seek failed");
        return pos < file_size ? (uint64_t)(file_size - pos) : 0;
    };
    char magic[4];
    read_exact(f, magic, 4);
    if (std::memcmp(magic, "NBLA", 4) != 0) fail(NBO_ERR_IO, "not a nabla tensor file");
    const uint32_t count = read_u32(f);
    std::vector<Entry> out;
    for (uint32_t i = 0; i < count; i++) {
        Entry e;
        const uint32_t name_len = read_u32(f);
        if (name_len > left()) fail(NBO_ERR_IO, "failed to fill whole buffer");
        e.name.resize(name_len);
        read_exact(f, e.name.empty() ? nullptr : &e.name[0], name_len);
        e.rows = read_u32(f);
        e.cols = read_u32(f);
        e.data_offset = std::ftell(f);
        if (e.data_offset < 0) fail(NBO_ERR_IO, "seek failed");
        const uint64_t elems = e.rows * e.cols; // both below 2^32
        if (elems > left() / 8) fail(NBO_ERR_IO, "failed to fill whole buffer");
        if (std::fseek(f, (long)(elems * 8), SEEK_CUR) != 0) fail(NBO_ERR_IO, "seek failed");
        out.push_back(std::move(e));
    }
    return out;
}

void seek_to(std::FILE *f, long off)
{
    if (std::fseek(f, off, SEEK_SET) != 0) fail(NBO_ERR_IO, "seek failed");
}

} // namespace

namespace nbo {

void nbla_save_list(const char *path, const nbo_list *list, const char *const *names)
{
    const uint64_t nt = list->layout.nt();
    if (nt && !names) fail(NBO_ERR_ARG, "null name array");
    if (nt > 0xFFFFFFFFull) fail(NBO_ERR_TOO_LARGE, "too many tensors for the file format");
    Runtime::get().sync(); // everything enqueued so far is part of what gets saved
    FilePtr f = open_file(path, "wb");
    Buffers b;
    write_all(f.get(), "NBLA", 4);
    write_u32(f.get(), (uint32_t)nt);
    for (uint64_t t = 0; t < nt; t++) {
        if (!names[t]) fail(NBO_ERR_ARG, "null tensor name");
        write_header(f.get(), names[t], list->layout.rows[t], list->layout.cols[t]);
        stream_out(f.get(), (const void *)(uintptr_t)list->ptrs[t], list->dtype, list->layout.n[t], b);
    }
    if (std::fflush(f.get()) != 0) fail(NBO_ERR_IO, std::string("write failed: ") + std::strerror(errno));
}

// Module::load_state_dict (nabla-ml/src/module/core.rs:281-304) over load_tensors: every
// tensor of the file must name a tensor of the list and have its shape.
void nbla_load_list(const char *path, nbo_list *list, const char *const *names)
{
    const uint64_t nt = list->layout.nt();
    if (nt && !names) fail(NBO_ERR_ARG, "null name array");
    FilePtr f = open_file(path, "rb");
    const std::vector<Entry> index = read_index(f.get());
    std::vector<uint64_t> target(index.size());
    for (size_t k = 0; k < index.size(); k++) {
        uint64_t t = 0;
        while (t < nt && index[k].name != names[t]) t++;
        if (t == nt) fail(NBO_ERR_STATE_KEY, "unknown parameter key: " + index[k].name);
        if (index[k].rows != list->layout.rows[t] || index[k].cols != list->layout.cols[t])
            fail(NBO_ERR_SHAPE, "shape mismatch for '" + index[k].name + "': expected (" +
                                    std::to_string(list->layout.rows[t]) + ", " +
                                    std::to_string(list->layout.cols[t]) + "), got (" +
                                    std::to_string(index[k].rows) + ", " + std::to_string(index[k].cols) + ")");
        target[k] = t;
    }
    Buffers b;
    for (size_t k = 0; k < index.size(); k++) {
        seek_to(f.get(), index[k].data_offset);
        stream_in(f.get(), (void *)(uintptr_t)list->ptrs[target[k]], list->dtype, list->layout.n[target[k]], b);
    }
}

namespace {

// One optimizer's state tensors in state_tensors() order -- m0.., then v0.. (Sgd: v0.. =
// velocity) -- each name behind `prefix` (alg.rs:476-485, 553-562, 623-629).
void write_optim_entries(std::FILE *f, const nbo_optim *opt, const std::string &prefix, Buffers &b)
{
    const uint64_t nt = opt->layout.nt();
    const bool adam_like = opt->meta.kind != NBO_KIND_SGD;
    const size_t eb = opt->elem_bytes();
    for (int which = 0; which < (adam_like ? 2 : 1); which++) {
        const char letter = adam_like && which == 0 ? 'm' : 'v';
        const uint32_t part = which == 0 ? 0u : opt->arena.part_v;
        for (uint64_t t = 0; t < nt; t++) {
            write_header(f, prefix + letter + std::to_string(t), opt->layout.rows[t], opt->layout.cols[t]);
            const char *dev = (const char *)opt->arena.part[part] + (size_t)opt->layout.soff[t] * eb;
            stream_out(f, dev, opt->state_dtype, opt->layout.n[t], b);
        }
    }
}

uint64_t optim_entry_count(const nbo_optim *opt)
{
    return opt->layout.nt() * (opt->meta.kind != NBO_KIND_SGD ? 2u : 1u);
}

// Where in the file each state tensor of one optimizer is.
struct LoadPlan {
    std::vector<long> m_at, v_at;
};

// OptimState::load_state_tensors (alg.rs:487-516, 564-593, 631-648) up to the point where it
// would start writing: other prefixes are ignored, every expected tensor must be present.
// `names[k]` is entry k's key as this optimizer sees it (a group prefix already taken off).
LoadPlan plan_optim_load(const nbo_optim *opt, const std::vector<const Entry *> &entries,
                         const std::vector<std::string> &names)
{
    const uint64_t nt = opt->layout.nt();
    const bool adam_like = opt->meta.kind != NBO_KIND_SGD;
    LoadPlan plan;
    plan.m_at.assign(nt, -1);
    plan.v_at.assign(nt, -1);
    for (size_t k = 0; k < entries.size(); k++) {
        const Entry &e = *entries[k];
        const std::string &name = names[k];
        const char c = name.empty() ? '\0' : name[0];
        if (!(c == 'v' || (c == 'm' && adam_like))) continue;
        // what Rust's str::parse::<usize> accepts: an optional '+', then decimal digits
        const char *p = name.c_str() + 1;
        if (*p == '+') p++;
        if (*p == '\0') fail(NBO_ERR_STATE_KEY, "bad tensor key: " + name);
        uint64_t idx = 0;
        for (; *p; p++) {
            if (*p < '0' || *p > '9' || idx > (UINT64_MAX - (uint64_t)(*p - '0')) / 10)
                fail(NBO_ERR_STATE_KEY, "bad tensor key: " + name);
            idx = idx * 10 + (uint64_t)(*p - '0');
        }
        if (idx >= nt) fail(NBO_ERR_STATE_INDEX, std::string(1, c) + " index out of range: " + std::to_string(idx));
        if (e.rows * e.cols != opt->layout.n[idx])
            fail(NBO_ERR_SHAPE, "state tensor " + name + " has " + std::to_string(opt->layout.n[idx]) +
                                    " elements, file has " + std::to_string(e.rows * e.cols));
        (c == 'm' ? plan.m_at : plan.v_at)[idx] = e.data_offset; // a later duplicate wins, as in the reference
    }
    if (adam_like)
        for (uint64_t t = 0; t < nt; t++)
            if (plan.m_at[t] < 0) fail(NBO_ERR_STATE_KEY, "missing m" + std::to_string(t));
    for (uint64_t t = 0; t < nt; t++)
        if (plan.v_at[t] < 0) fail(NBO_ERR_STATE_KEY, "missing v" + std::to_string(t));
    return plan;
}

void apply_optim_load(std::FILE *f, nbo_optim *opt, const LoadPlan &plan, Buffers &b)
{
    const uint64_t nt = opt->layout.nt();
    const bool adam_like = opt->meta.kind != NBO_KIND_SGD;
    const size_t eb = opt->elem_bytes();
    for (int which = 0; which < (adam_like ? 2 : 1); which++) {
        const std::vector<long> &at = adam_like && which == 0 ? plan.m_at : plan.v_at;
        const uint32_t part = which == 0 ? 0u : opt->arena.part_v;
        for (uint64_t t = 0; t < nt; t++) {
            seek_to(f, at[t]);
            char *dev = (char *)opt->arena.part[part] + (size_t)opt->layout.soff[t] * eb;
            stream_in(f, dev, opt->state_dtype, opt->layout.n[t], b);
        }
    }
}

} // namespace

// optim.nbla of a checkpoint: OptimState::state_tensors written by save_tensors
// (checkpoint.rs:59-62).
void optim_save_state(const nbo_optim *opt, const char *path)
{
    Runtime::get().sync();
    FilePtr f = open_file(path, "wb");
    Buffers b;
    write_all(f.get(), "NBLA", 4);
    write_u32(f.get(), (uint32_t)optim_entry_count(opt));
    write_optim_entries(f.get(), opt, "", b);
    if (std::fflush(f.get()) != 0) fail(NBO_ERR_IO, std::string("write failed: ") + std::strerror(errno));
}

// load_tensors into OptimState::load_state_tensors (checkpoint.rs:92-95); nothing is written
// unless the whole file checks out.
void optim_load_state(nbo_optim *opt, const char *path)
{
    FilePtr f = open_file(path, "rb");
    const std::vector<Entry> index = read_index(f.get());
    std::vector<const Entry *> entries;
    std::vector<std::string> names;
    for (const Entry &e : index) entries.push_back(&e), names.push_back(e.name);
    const LoadPlan plan = plan_optim_load(opt, entries, names);
    Buffers b;
    apply_optim_load(f.get(), opt, plan, b);
}

// params.nbla of a mixed-precision optimizer: the reference has no such optimizer, but what its
// checkpoint holds as parameters (checkpoint.rs:54-58: the module's state_dict through
// save_tensors) is here the f32 master weights -- the 16-bit parameters are derived from them.
void optim_save_master(const nbo_optim *opt, const char *path, const char *const *names)
{
    const uint64_t nt = opt->layout.nt();
    if (!opt->keep_master) fail(NBO_ERR_DTYPE, "optimizer was created without master weights");
    if (!opt->master_valid) fail(NBO_ERR_NO_MASTER, "master weights not set");
    if (nt && !names) fail(NBO_ERR_ARG, "null name array");
    if (nt > 0xFFFFFFFFull) fail(NBO_ERR_TOO_LARGE, "too many tensors for the file format");
    Runtime::get().sync();
    FilePtr f = open_file(path, "wb");
    Buffers b;
    write_all(f.get(), "NBLA", 4);
    write_u32(f.get(), (uint32_t)nt);
    for (uint64_t t = 0; t < nt; t++) {
        if (!names[t]) fail(NBO_ERR_ARG, "null tensor name");
        write_header(f.get(), names[t], opt->layout.rows[t], opt->layout.cols[t]);
        const char *dev = (const char *)opt->arena.part[opt->arena.part_w] + (size_t)opt->layout.soff[t] * 4;
        stream_out(f.get(), dev, NBO_DT_F32, opt->layout.n[t], b);
    }
    if (std::fflush(f.get()) != 0) fail(NBO_ERR_IO, std::string("write failed: ") + std::strerror(errno));
}

// load_tensors + Module::load_state_dict (module/core.rs:281-304) into the master weights: the
// same checks as nbla_load_list, and every master tensor must be in the file -- a master weight
// that kept its old value would silently diverge from its 16-bit parameter.
void optim_load_master(nbo_optim *opt, const char *path, const char *const *names)
{
    const uint64_t nt = opt->layout.nt();
    if (!opt->keep_master) fail(NBO_ERR_DTYPE, "optimizer was created without master weights");
    if (nt && !names) fail(NBO_ERR_ARG, "null name array");
    FilePtr f = open_file(path, "rb");
    const std::vector<Entry> index = read_index(f.get());
    std::vector<long> at(nt, -1);
    for (const Entry &e : index) {
        uint64_t t = 0;
        while (t < nt && e.name != names[t]) t++;
        if (t == nt) fail(NBO_ERR_STATE_KEY, "unknown parameter key: " + e.name);
        if (e.rows != opt->layout.rows[t] || e.cols != opt->layout.cols[t])
            fail(NBO_ERR_SHAPE, "shape mismatch for '" + e.name + "': expected (" + std::to_string(opt->layout.rows[t]) +
                                    ", " + std::to_string(opt->layout.cols[t]) + "), got (" + std::to_string(e.rows) +
                                    ", " + std::to_string(e.cols) + ")");
        at[t] = e.data_offset;
    }
    for (uint64_t t = 0; t < nt; t++)
        if (at[t] < 0) fail(NBO_ERR_STATE_KEY, std::string("missing parameter key: ") + names[t]);
    Buffers b;
    for (uint64_t t = 0; t < nt; t++) {
        seek_to(f.get(), at[t]);
        char *dev = (char *)opt->arena.part[opt->arena.part_w] + (size_t)opt->layout.soff[t] * 4;
        stream_in(f.get(), dev, NBO_DT_F32, opt->layout.n[t], b);
    }
    opt->master_valid = true;
}

// params.nbla of a GroupOptimizer (checkpoint.rs:54-58 over the module's state_dict): the module's
// parameter i is tensor index_in_group[i] of group group_of[i]; what is written under names[i] is
// that group's f32 master weight if the group keeps master weights, else the caller's tensor itself.
namespace {
struct GroupSlot { // where parameter i lives
    int dtype;
    uint64_t rows, cols, n;
    void *dev;
    bool master;
};

std::vector<GroupSlot> group_slots(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                   uint64_t n_params, const uint32_t *group_of, const uint32_t *index_in_group,
                                   bool saving)
{
    if (n_params && (!group_of || !index_in_group)) fail(NBO_ERR_ARG, "null index array");
    std::vector<GroupSlot> out(n_params);
    std::vector<std::vector<char>> seen(n_groups);
    for (uint64_t g = 0; g < n_groups; g++) {
        if (!opts[g] || !params[g]) fail(NBO_ERR_ARG, "null optimizer or list");
        if (params[g]->layout.nt() != opts[g]->layout.nt()) fail(NBO_ERR_COUNT_MISMATCH, "params count mismatch");
        seen[g].assign(opts[g]->layout.nt(), 0);
    }
    for (uint64_t i = 0; i < n_params; i++) {
        const uint32_t g = group_of[i], k = index_in_group[i];
        if (g >= n_groups || k >= opts[g]->layout.nt() || seen[g][k])
            fail(NBO_ERR_ARG, "parameter " + std::to_string(i) + ": not a tensor of its group, or named twice");
        seen[g][k] = 1;
        const nbo_optim *o = opts[g];
        GroupSlot &s = out[i];
        s.master = o->keep_master;
        s.rows = o->layout.rows[k], s.cols = o->layout.cols[k], s.n = o->layout.n[k];
        if (params[g]->layout.rows[k] != s.rows || params[g]->layout.cols[k] != s.cols)
            fail(NBO_ERR_SHAPE, "shapes must match (group " + std::to_string(g) + ", tensor " + std::to_string(k) + ")");
        if (s.master) {
            if (saving && !o->master_valid) fail(NBO_ERR_NO_MASTER, "master weights not set");
            s.dtype = NBO_DT_F32;
            s.dev = (char *)o->arena.part[o->arena.part_w] + (size_t)o->layout.soff[k] * 4;
        } else {
            s.dtype = params[g]->dtype;
            s.dev = (void *)(uintptr_t)params[g]->ptrs[k];
        }
    }
    for (uint64_t g = 0; g < n_groups; g++)
        for (char c : seen[g])
            if (!c) fail(NBO_ERR_COUNT_MISMATCH, "nabla-train: GroupOptimizer param count mismatch");
    return out;
}
} // namespace

void optim_save_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params, uint64_t n_params,
                              const uint32_t *group_of, const uint32_t *index_in_group, const char *const *names,
                              const char *path)
{
    if (n_params && !names) fail(NBO_ERR_ARG, "null name array");
    if (n_params > 0xFFFFFFFFull) fail(NBO_ERR_TOO_LARGE, "too many tensors for the file format");
    const std::vector<GroupSlot> slots = group_slots(n_groups, opts, params, n_params, group_of, index_in_group, true);
    Runtime::get().sync();
    FilePtr f = open_file(path, "wb");
    Buffers b;
    write_all(f.get(), "NBLA", 4);
    write_u32(f.get(), (uint32_t)n_params);
    for (uint64_t i = 0; i < n_params; i++) {
        if (!names[i]) fail(NBO_ERR_ARG, "null tensor name");
        write_header(f.get(), names[i], slots[i].rows, slots[i].cols);
        stream_out(f.get(), slots[i].dev, slots[i].dtype, slots[i].n, b);
    }
    if (std::fflush(f.get()) != 0) fail(NBO_ERR_IO, std::string("write failed: ") + std::strerror(errno));
}

// load_tensors + Module::load_state_dict (module/core.rs:281-304) for a GroupOptimizer's module:
// every tensor of the file must name a parameter and have its shape, and every parameter whose
// group keeps master weights must be in the file (a master weight that kept its old value would
// silently diverge from its 16-bit parameter).  Nothing is written unless the whole file checks
// out.  Afterwards those groups' master weights count as set; the caller derives the 16-bit
// parameters from them (nbo_optim_params_from_master per group).
void optim_load_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params, uint64_t n_params,
                              const uint32_t *group_of, const uint32_t *index_in_group, const char *const *names,
                              const char *path)
{
    if (n_params && !names) fail(NBO_ERR_ARG, "null name array");
    const std::vector<GroupSlot> slots = group_slots(n_groups, opts, params, n_params, group_of, index_in_group, false);
    FilePtr f = open_file(path, "rb");
    const std::vector<Entry> index = read_index(f.get());
    std::vector<long> at(n_params, -1);
    for (const Entry &e : index) {
        uint64_t i = 0;
        while (i < n_params && e.name != names[i]) i++;
        if (i == n_params) fail(NBO_ERR_STATE_KEY, "unknown parameter key: " + e.name);
        if (e.rows != slots[i].rows || e.cols != slots[i].cols)
            fail(NBO_ERR_SHAPE, "shape mismatch for '" + e.name + "': expected (" + std::to_string(slots[i].rows) + ", " +
                                    std::to_string(slots[i].cols) + "), got (" + std::to_string(e.rows) + ", " +
                                    std::to_string(e.cols) + ")");
        at[i] = e.data_offset;
    }
    for (uint64_t i = 0; i < n_params; i++)
        if (at[i] < 0 && slots[i].master) fail(NBO_ERR_STATE_KEY, std::string("missing parameter key: ") + names[i]);
    Buffers b;
    for (uint64_t i = 0; i < n_params; i++) {
        if (at[i] < 0) continue;
        seek_to(f.get(), at[i]);
        stream_in(f.get(), slots[i].dev, slots[i].dtype, slots[i].n, b);
    }
    for (uint64_t g = 0; g < n_groups; g++)
        if (opts[g]->keep_master) opts[g]->master_valid = true;
}

// GroupOptimizer's OptimState (groups.rs:320-373): every group's tensors behind "g{gi}.".
void optim_save_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path)
{
    uint64_t total = 0;
    for (uint64_t g = 0; g < n_groups; g++) total += optim_entry_count(opts[g]);
    if (total > 0xFFFFFFFFull) fail(NBO_ERR_TOO_LARGE, "too many tensors for the file format");
    Runtime::get().sync();
    FilePtr f = open_file(path, "wb");
    Buffers b;
    write_all(f.get(), "NBLA", 4);
    write_u32(f.get(), (uint32_t)total);
    for (uint64_t g = 0; g < n_groups; g++)
        write_optim_entries(f.get(), opts[g], "g" + std::to_string(g) + ".", b);
    if (std::fflush(f.get()) != 0) fail(NBO_ERR_IO, std::string("write failed: ") + std::strerror(errno));
}

void optim_load_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path)
{
    FilePtr f = open_file(path, "rb");
    const std::vector<Entry> index = read_index(f.get());
    std::vector<std::vector<const Entry *>> entries(n_groups);
    std::vector<std::vector<std::string>> names(n_groups);
    for (const Entry &e : index) { // groups.rs:339-361: "g{gi}.{key}", every tensor of the file
        const size_t dot = e.name.find('.');
        if (dot == std::string::npos || e.name[0] != 'g') fail(NBO_ERR_STATE_KEY, "bad group tensor key: " + e.name);
        const std::string idx = e.name.substr(1, dot - 1);
        const char *p = idx.c_str();
        if (*p == '+') p++;
        if (*p == '\0') fail(NBO_ERR_STATE_KEY, "bad group index: " + idx);
        uint64_t gi = 0;
        for (; *p; p++) {
            if (*p < '0' || *p > '9' || gi > (UINT64_MAX - (uint64_t)(*p - '0')) / 10)
                fail(NBO_ERR_STATE_KEY, "bad group index: " + idx);
            gi = gi * 10 + (uint64_t)(*p - '0');
        }
        if (gi >= n_groups) fail(NBO_ERR_STATE_INDEX, "group index out of range: " + std::to_string(gi));
        entries[gi].push_back(&e);
        names[gi].push_back(e.name.substr(dot + 1));
    }
    std::vector<LoadPlan> plans;
    for (uint64_t g = 0; g < n_groups; g++) plans.push_back(plan_optim_load(opts[g], entries[g], names[g]));
    Buffers b;
    for (uint64_t g = 0; g < n_groups; g++) apply_optim_load(f.get(), opts[g], plans[g], b);
}

} // namespace nbo
