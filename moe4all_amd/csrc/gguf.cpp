// GGUF weight source behind include/infr_gguf.h: maps the file(s), walks header -> metadata ->
// tensor directory once, and afterwards only hands out pointers into the mappings.
//
// Behaviour follows the reference loader (crates/infr-gguf/src/lib.rs): versions 2 and 3, the
// `general.alignment` rules (:786-807), at most 4 dimensions (:46-54), whole-block element counts
// (:855-872), duplicate names refused (:673-691), shard sets stitched by `split.*` keys and the
// `<base>-NNNNN-of-MMMMM.gguf` naming (:502-598, crates/infr-core/src/gguf_split.rs).  All numbers
// read from a file are treated as hostile input.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <stdexcept>
#include <string>
#include <string_view>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "../../include/infr_gguf.h"

namespace {

thread_local std::string g_err;

infr_status fail(infr_status st, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return st;
}

// No exception crosses the C ABI: the entry points are function-try-blocks whose handler lands here.
infr_status guard_fail(const char* what) noexcept {
    try {
        try {
            throw;
        } catch (const std::bad_alloc&) {
            return fail(INFR_ERR_BACKEND, "%s: out of host memory", what);
        } catch (const std::exception& e) {
            return fail(INFR_ERR_BACKEND, "%s: %s", what, e.what());
        } catch (...) {
            return fail(INFR_ERR_BACKEND, "%s: unknown exception", what);
        }
    } catch (...) {
        return INFR_ERR_BACKEND;
    }
}

constexpr uint32_t kMagic = 0x46554747u;       // "GGUF"
constexpr uint64_t kDefaultAlign = 32;
constexpr uint64_t kMaxAlign = 16ull << 20;
constexpr uint32_t kMaxDims = 4;
constexpr int kMaxArrayDepth = 64;
constexpr size_t kMaxShardDigits = 5;

// infr_dtype ordinals from 15 on under the loader's own names; I2S is known to the loader only
// (crates/infr-core/src/tensor.rs:25-50)
enum : int32_t {
    DT_IQ1S = 15, DT_IQ1M, DT_IQ2XXS, DT_IQ2XS, DT_IQ2S, DT_IQ3XXS, DT_IQ3S, DT_IQ4NL, DT_IQ4XS,
    DT_TQ1_0, DT_TQ2_0, DT_I2S, DT_Q2_0, DT_MXFP4, DT_NVFP4
};

// ggml_type -> dtype ordinal (lib.rs:326-366); -1: not a type this engine knows
int32_t dtype_of_ggml(uint32_t t) {
    switch (t) {
        case 0: return INFR_F32;   case 1: return INFR_F16;   case 2: return INFR_Q4_0;  case 3: return INFR_Q4_1;
        case 6: return INFR_Q5_0;  case 7: return INFR_Q5_1;  case 8: return INFR_Q8_0;  case 10: return INFR_Q2K;
        case 11: return INFR_Q3K;  case 12: return INFR_Q4K;  case 13: return INFR_Q5K;  case 14: return INFR_Q6K;
        case 16: return DT_IQ2XXS; case 17: return DT_IQ2XS;  case 18: return DT_IQ3XXS; case 19: return DT_IQ1S;
        case 20: return DT_IQ4NL;  case 21: return DT_IQ3S;   case 22: return DT_IQ2S;   case 23: return DT_IQ4XS;
        case 26: return INFR_I32;  case 29: return DT_IQ1M;   case 30: return INFR_BF16; case 34: return DT_TQ1_0;
        case 35: return DT_TQ2_0;  case 36: return DT_I2S;    case 39: return DT_MXFP4;  case 40: return DT_NVFP4;
        case 42: return DT_Q2_0;
        default: return -1;
    }
}

// (elements, bytes) of one block, the ggml type_traits sizes (decode_spec.rs:455-504)
bool block_layout(int32_t dt, uint32_t* be, uint32_t* bb) {
    struct L { int32_t dt; uint32_t e, b; };
    static const L table[] = {
        {INFR_F32, 1, 4},   {INFR_F16, 1, 2},   {INFR_BF16, 1, 2},  {INFR_I32, 1, 4},    {INFR_U32, 1, 4},
        {INFR_Q4_0, 32, 18}, {INFR_Q4_1, 32, 20}, {INFR_Q5_0, 32, 22}, {INFR_Q5_1, 32, 24}, {INFR_Q8_0, 32, 34},
        {INFR_Q2K, 256, 84}, {INFR_Q3K, 256, 110}, {INFR_Q4K, 256, 144}, {INFR_Q5K, 256, 176}, {INFR_Q6K, 256, 210},
        {DT_IQ1S, 256, 50},  {DT_IQ1M, 256, 56},  {DT_IQ2XXS, 256, 66}, {DT_IQ2XS, 256, 74}, {DT_IQ2S, 256, 82},
        {DT_IQ3XXS, 256, 98}, {DT_IQ3S, 256, 110}, {DT_IQ4NL, 32, 18},  {DT_IQ4XS, 256, 136}, {DT_TQ1_0, 256, 54},
        {DT_TQ2_0, 256, 66}, {DT_Q2_0, 64, 18},   {DT_MXFP4, 32, 17},   {DT_NVFP4, 64, 36},
    };
    for (const L& l : table)
        if (l.dt == dt) { *be = l.e; *bb = l.b; return true; }
    return false;
}

struct Cursor {
    const uint8_t* base;
    size_t len, pos = 0;
    bool has(uint64_t n) const { return n <= len - pos; }
    template <class T>
    bool get(T* v) {
        if (!has(sizeof(T))) return false;
        memcpy(v, base + pos, sizeof(T));   // the file is little-endian, so is every host this runs on
        pos += sizeof(T);
        return true;
    }
    bool str(std::string_view* s) {
        uint64_t n;
        if (!get(&n) || !has(n)) return false;
        *s = std::string_view(reinterpret_cast<const char*>(base + pos), (size_t)n);
        pos += (size_t)n;
        return true;
    }
};

struct Meta {
    enum Kind : uint8_t { U64, I64, F64, BOOL, STR, ARR } kind;
    uint64_t u = 0;      // U64 value, BOOL, ARR length
    int64_t i = 0;
    double f = 0;
    std::string_view s;  // STR, into the mapping
};

struct Tensor {
    std::string name;
    int32_t dtype;
    uint32_t ggml_type, rank;
    uint64_t shape[4];
    uint64_t numel, offset, nbytes;   // offset: in the set's concatenated address space once assembled
};

struct Shard {
    std::string path;
    void* map = nullptr;
    size_t len = 0;
    uint64_t file_base = 0, data_start = 0;
    std::unordered_map<std::string, Meta> meta;
    std::vector<Tensor> tensors;
    Shard() = default;
    Shard(const Shard&) = delete;
    Shard& operator=(const Shard&) = delete;
    Shard(Shard&& o) noexcept { *this = std::move(o); }
    Shard& operator=(Shard&& o) noexcept {
        if (this != &o) {
            release();
            path = std::move(o.path); map = o.map; len = o.len; file_base = o.file_base; data_start = o.data_start;
            meta = std::move(o.meta); tensors = std::move(o.tensors);
            o.map = nullptr; o.len = 0;
        }
        return *this;
    }
    ~Shard() { release(); }
    void release() {
        if (map && len) munmap(map, len);
        map = nullptr;
    }
};

// One metadata value; arrays are walked (every element bounds-checked) but only their length is kept.
bool read_value(Cursor& c, uint32_t type, int depth, Meta* out, std::string* why) {
    auto eof = [&]() { *why = "unexpected end of file inside the metadata at offset " + std::to_string(c.pos); return false; };
    switch (type) {
        case 0: { uint8_t v; if (!c.get(&v)) return eof(); out->kind = Meta::U64; out->u = v; return true; }
        case 1: { int8_t v; if (!c.get(&v)) return eof(); out->kind = Meta::I64; out->i = v; return true; }
        case 2: { uint16_t v; if (!c.get(&v)) return eof(); out->kind = Meta::U64; out->u = v; return true; }
        case 3: { int16_t v; if (!c.get(&v)) return eof(); out->kind = Meta::I64; out->i = v; return true; }
        case 4: { uint32_t v; if (!c.get(&v)) return eof(); out->kind = Meta::U64; out->u = v; return true; }
        case 5: { int32_t v; if (!c.get(&v)) return eof(); out->kind = Meta::I64; out->i = v; return true; }
        case 6: { float v; if (!c.get(&v)) return eof(); out->kind = Meta::F64; out->f = v; return true; }
        case 7: { uint8_t v; if (!c.get(&v)) return eof(); out->kind = Meta::BOOL; out->u = v != 0; return true; }
        case 8: { if (!c.str(&out->s)) return eof(); out->kind = Meta::STR; return true; }
        case 9: {
            if (depth >= kMaxArrayDepth) {
                *why = "metadata arrays nest deeper than " + std::to_string(kMaxArrayDepth) + " levels at offset " + std::to_string(c.pos);
                return false;
            }
            uint32_t et;
            uint64_t n;
            if (!c.get(&et) || !c.get(&n)) return eof();
            static const int fixed[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};
            if (et < 13 && fixed[et]) {   // fixed-width elements: one bounds check for the lot
                if (n > (c.len - c.pos) / (uint64_t)fixed[et]) return eof();
                c.pos += (size_t)(n * (uint64_t)fixed[et]);
            } else {
                Meta scratch;
                for (uint64_t k = 0; k < n; k++)
                    if (!read_value(c, et, depth + 1, &scratch, why)) return false;
            }
            out->kind = Meta::ARR;
            out->u = n;
            return true;
        }
        case 10: { uint64_t v; if (!c.get(&v)) return eof(); out->kind = Meta::U64; out->u = v; return true; }
        case 11: { int64_t v; if (!c.get(&v)) return eof(); out->kind = Meta::I64; out->i = v; return true; }
        case 12: { double v; if (!c.get(&v)) return eof(); out->kind = Meta::F64; out->f = v; return true; }
        default: *why = "unknown metadata value type " + std::to_string(type); return false;
    }
}

bool meta_u64(const std::unordered_map<std::string, Meta>& m, const char* key, uint64_t* out) {
    auto it = m.find(key);
    if (it == m.end()) return false;
    if (it->second.kind == Meta::U64) { *out = it->second.u; return true; }
    if (it->second.kind == Meta::I64 && it->second.i >= 0) { *out = (uint64_t)it->second.i; return true; }
    return false;
}

// Maps and parses one file; tensor offsets stay relative to the file's own data region.
bool parse_file(const std::string& path, Shard* sh, std::string* why, bool* io_error) {
    *io_error = true;
    int fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) { *why = path + ": " + strerror(errno); return false; }
    struct stat st;
    if (fstat(fd, &st) != 0) { *why = path + ": " + strerror(errno); close(fd); return false; }
    sh->path = path;
    sh->len = (size_t)st.st_size;
    if (sh->len) {
        void* p = mmap(nullptr, sh->len, PROT_READ, MAP_PRIVATE, fd, 0);
        if (p == MAP_FAILED) { *why = path + ": mmap: " + strerror(errno); close(fd); sh->len = 0; return false; }
        sh->map = p;
        (void)madvise(p, sh->len, MADV_WILLNEED);   // a hint; the load does not depend on it
    }
    close(fd);
    *io_error = false;
    Cursor c{static_cast<const uint8_t*>(sh->map), sh->len};
    uint32_t magic = 0, version = 0;
    uint64_t n_tensors = 0, n_kv = 0;
    if (!c.get(&magic) || magic != kMagic) {
        char b[96];
        snprintf(b, sizeof b, "not a GGUF file (magic 0x%08X, expected 0x%08X)", magic, kMagic);
        *why = b;
        return false;
    }
    if (!c.get(&version) || (version != 2 && version != 3)) {
        *why = "unsupported GGUF version " + std::to_string(version) + " (supported: 2, 3)";
        return false;
    }
    if (!c.get(&n_tensors) || !c.get(&n_kv)) { *why = "unexpected end of file in the header"; return false; }
    for (uint64_t k = 0; k < n_kv; k++) {
        std::string_view key;
        uint32_t type;
        if (!c.str(&key) || !c.get(&type)) { *why = "unexpected end of file inside the metadata at offset " + std::to_string(c.pos); return false; }
        Meta v;
        if (!read_value(c, type, 0, &v, why)) return false;
        sh->meta[std::string(key)] = v;   // a repeated key keeps its last value, like the reference's map insert
    }
    uint64_t align = kDefaultAlign;
    {
        auto it = sh->meta.find("general.alignment");
        if (it != sh->meta.end() && !meta_u64(sh->meta, "general.alignment", &align)) align = 0;
    }
    if (align == 0 || (align & (align - 1)) != 0) {
        *why = "invalid general.alignment " + std::to_string(align) + " (must be a positive power of two)";
        return false;
    }
    if (align > kMaxAlign) {
        *why = "invalid general.alignment " + std::to_string(align) + " (exceeds the " + std::to_string(kMaxAlign) + "-byte cap)";
        return false;
    }
    for (uint64_t k = 0; k < n_tensors; k++) {
        Tensor t{};
        std::string_view name;
        if (!c.str(&name) || !c.get(&t.rank)) { *why = "unexpected end of file inside the tensor directory"; return false; }
        t.name = std::string(name);
        if (t.rank > kMaxDims) {
            *why = "tensor '" + t.name + "' declares " + std::to_string(t.rank) + " dimensions (max " + std::to_string(kMaxDims) + ")";
            return false;
        }
        t.numel = 1;
        bool overflow = false;
        for (uint32_t d = 0; d < t.rank; d++) {
            if (!c.get(&t.shape[d])) { *why = "unexpected end of file inside the tensor directory"; return false; }
            overflow |= __builtin_mul_overflow(t.numel, t.shape[d], &t.numel);
        }
        if (!c.get(&t.ggml_type) || !c.get(&t.offset)) { *why = "unexpected end of file inside the tensor directory"; return false; }
        if (overflow) { *why = "tensor '" + t.name + "': element count overflows 64 bits"; return false; }
        sh->tensors.push_back(std::move(t));
    }
    sh->data_start = (c.pos + align - 1) / align * align;
    for (Tensor& t : sh->tensors) {
        t.dtype = dtype_of_ggml(t.ggml_type);
        if (t.dtype < 0) { *why = "tensor '" + t.name + "': unsupported ggml type " + std::to_string(t.ggml_type); return false; }
        if (t.dtype == DT_I2S) {
            if (t.numel % 4) { *why = "tensor '" + t.name + "' has " + std::to_string(t.numel) + " elements, not a multiple of 4 (i2_s packs 4 codes per byte)"; return false; }
            t.nbytes = t.numel / 4 + 4;
            continue;
        }
        uint32_t be = 1, bb = 1;
        block_layout(t.dtype, &be, &bb);
        if (t.numel % be) {
            *why = "tensor '" + t.name + "' has " + std::to_string(t.numel) + " elements, not a whole number of blocks (" +
                   std::to_string(be) + " elements per block)";
            return false;
        }
        if (__builtin_mul_overflow(t.numel / be, (uint64_t)bb, &t.nbytes)) {
            *why = "tensor '" + t.name + "': byte size overflows 64 bits";
            return false;
        }
    }
    return true;
}

struct ShardName { std::string base; uint32_t index, total; size_t width; };

// "<base>-NNNNN-of-MMMMM.gguf" (crates/infr-core/src/gguf_split.rs: parse_shard)
bool parse_shard_name(const std::string& fname, ShardName* out) {
    if (fname.size() < 5) return false;
    std::string ext = fname.substr(fname.size() - 5);
    for (char& ch : ext) ch = (char)tolower((unsigned char)ch);
    if (ext != ".gguf") return false;
    const std::string stem = fname.substr(0, fname.size() - 5);
    const size_t of = stem.rfind("-of-");
    if (of == std::string::npos) return false;
    const std::string total = stem.substr(of + 4), left = stem.substr(0, of);
    const size_t dash = left.rfind('-');
    if (dash == std::string::npos) return false;
    const std::string idx = left.substr(dash + 1);
    auto digits = [](const std::string& s) {
        if (s.empty()) return false;
        for (char ch : s) if (ch < '0' || ch > '9') return false;
        return true;
    };
    if (!digits(total) || !digits(idx) || total.size() != idx.size() || total.size() > kMaxShardDigits) return false;
    out->base = left.substr(0, dash);
    out->index = (uint32_t)strtoul(idx.c_str(), nullptr, 10);
    out->total = (uint32_t)strtoul(total.c_str(), nullptr, 10);
    out->width = total.size();
    return true;
}

}  // namespace

struct infr_gguf {
    std::vector<Shard> shards;
    std::vector<Tensor> tensors;                      // all shards, in order
    std::unordered_map<std::string, size_t> by_name;
    const std::unordered_map<std::string, Meta>& meta() const { return shards[0].meta; }
};

namespace {

bool check_position(const Shard& sh, size_t index0, uint64_t count, std::string* why) {
    uint64_t no = 0, declared = 0;
    if (!meta_u64(sh.meta, "split.no", &no)) {
        *why = sh.path + " is named as shard " + std::to_string(index0 + 1) + " of " + std::to_string(count) +
               " but carries no split.no";
        return false;
    }
    if (no != index0) {
        *why = sh.path + " is named as shard " + std::to_string(index0 + 1) + " of " + std::to_string(count) +
               " but declares split.no = " + std::to_string(no);
        return false;
    }
    if (!meta_u64(sh.meta, "split.count", &declared)) {
        *why = sh.path + " is named as shard " + std::to_string(index0 + 1) + " but carries no split.count";
        return false;
    }
    if (declared != count) {
        *why = sh.path + " declares split.count = " + std::to_string(declared) + " but the rest of the set declares " +
               std::to_string(count);
        return false;
    }
    return true;
}

const Meta* find_meta(const infr_gguf* g, const char* key, Meta::Kind kind, const char* kind_name) {
    if (!g || !key) { fail(INFR_ERR_INVALID, "gguf: null handle or key"); return nullptr; }
    auto it = g->meta().find(key);
    if (it == g->meta().end()) { fail(INFR_ERR_INVALID, "gguf: no metadata key '%s'", key); return nullptr; }
    if (it->second.kind != kind) { fail(INFR_ERR_INVALID, "gguf: metadata key '%s' is not %s", key, kind_name); return nullptr; }
    return &it->second;
}

void fill(const Tensor& t, infr_gguf_tensor* out) {
    out->name = t.name.c_str();
    out->dtype = t.dtype;
    out->ggml_type = t.ggml_type;
    out->rank = t.rank;
    for (int d = 0; d < 4; d++) out->shape[d] = d < (int)t.rank ? t.shape[d] : 1;
    out->numel = t.numel;
    out->offset = t.offset;
    out->nbytes = t.nbytes;
}

}  // namespace

extern "C" const char* infr_gguf_last_error(void) { return g_err.c_str(); }

extern "C" infr_status infr_gguf_open(const char* path, infr_gguf** out) try {
    if (!path || !out) return fail(INFR_ERR_INVALID, "gguf open: null argument");
    *out = nullptr;
    std::string why;
    std::vector<Shard> parts(1);
    bool io = false;
    if (!parse_file(path, &parts[0], &why, &io)) return fail(io ? INFR_ERR_IO : INFR_ERR_LOADER, "GGUF: %s", why.c_str());
    uint64_t count = 0, expect_tensors = 0;
    bool split = meta_u64(parts[0].meta, "split.count", &count) && count > 1;
    if (split) {
        const std::string p(path);
        const size_t slash = p.rfind('/');
        const std::string dir = slash == std::string::npos ? std::string(".") : p.substr(0, slash);
        const std::string fname = slash == std::string::npos ? p : p.substr(slash + 1);
        ShardName sn;
        if (!parse_shard_name(fname, &sn))
            return fail(INFR_ERR_LOADER, "GGUF: %s declares split.count = %llu, but its name is not a <base>-NNNNN-of-MMMMM.gguf "
                        "shard name, so the rest of the set cannot be found", fname.c_str(), (unsigned long long)count);
        if (sn.total != count)
            return fail(INFR_ERR_LOADER, "GGUF: %s is named as one of %u shards but declares split.count = %llu", fname.c_str(),
                        sn.total, (unsigned long long)count);
        if (sn.index < 1 || sn.index > count)
            return fail(INFR_ERR_LOADER, "GGUF: %s is numbered %u of %llu, outside the set its own name describes", fname.c_str(),
                        sn.index, (unsigned long long)count);
        const size_t opened_at = sn.index - 1;
        if (!check_position(parts[0], opened_at, count, &why)) return fail(INFR_ERR_LOADER, "GGUF: %s", why.c_str());
        std::vector<Shard> all((size_t)count);
        for (size_t i = 0; i < (size_t)count; i++) {
            if (i == opened_at) { all[i] = std::move(parts[0]); continue; }
            char num[48];
            snprintf(num, sizeof num, "-%0*u-of-%0*u.gguf", (int)sn.width, (unsigned)(i + 1), (int)sn.width, sn.total);
            const std::string sp = dir + "/" + sn.base + num;
            if (!parse_file(sp, &all[i], &why, &io))
                return fail(io ? INFR_ERR_IO : INFR_ERR_LOADER, "GGUF: shard %zu of %llu (%s): %s", i + 1, (unsigned long long)count, sp.c_str(), why.c_str());
            if (!check_position(all[i], i, count, &why)) return fail(INFR_ERR_LOADER, "GGUF: %s", why.c_str());
        }
        parts = std::move(all);
        if (!meta_u64(parts[0].meta, "split.tensors.count", &expect_tensors))
            return fail(INFR_ERR_LOADER, "GGUF: %s declares split.count = %llu but carries no split.tensors.count",
                        parts[0].path.c_str(), (unsigned long long)count);
    }
    auto g = new infr_gguf();
    uint64_t file_base = 0;
    for (Shard& sh : parts) {
        sh.file_base = file_base;
        for (Tensor& t : sh.tensors) {
            uint64_t off;
            if (__builtin_add_overflow(t.offset, sh.data_start, &off) || __builtin_add_overflow(off, file_base, &off)) {
                delete g;
                return fail(INFR_ERR_LOADER, "GGUF: tensor '%s' offset overflows 64 bits", t.name.c_str());
            }
            t.offset = off;
            g->tensors.push_back(t);
        }
        sh.tensors.clear();
        file_base += sh.len;
    }
    g->shards = std::move(parts);
    for (size_t i = 0; i < g->tensors.size(); i++) {
        if (!g->by_name.emplace(g->tensors[i].name, i).second) {
            std::string n = g->tensors[i].name;
            delete g;
            return fail(INFR_ERR_LOADER, "GGUF: duplicate tensor name '%s'", n.c_str());
        }
    }
    if (split && g->tensors.size() != expect_tensors) {
        size_t have = g->tensors.size(), ns = g->shards.size();
        delete g;
        return fail(INFR_ERR_LOADER, "GGUF: the %zu shards hold %zu tensors between them but the model declares "
                    "split.tensors.count = %llu", ns, have, (unsigned long long)expect_tensors);
    }
    *out = g;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_open"); }

extern "C" void infr_gguf_close(infr_gguf* g) { delete g; }

extern "C" uint64_t infr_gguf_tensor_count(const infr_gguf* g) { return g ? g->tensors.size() : 0; }
extern "C" uint32_t infr_gguf_shard_count(const infr_gguf* g) { return g ? (uint32_t)g->shards.size() : 0; }

extern "C" infr_status infr_gguf_tensor_at(const infr_gguf* g, uint64_t index, infr_gguf_tensor* out) try {
    if (!g || !out) return fail(INFR_ERR_INVALID, "gguf: null argument");
    if (index >= g->tensors.size()) return fail(INFR_ERR_INVALID, "gguf: tensor index %llu out of range", (unsigned long long)index);
    fill(g->tensors[(size_t)index], out);
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_tensor_at"); }

extern "C" infr_status infr_gguf_tensor_find(const infr_gguf* g, const char* name, infr_gguf_tensor* out) try {
    if (!g || !name || !out) return fail(INFR_ERR_INVALID, "gguf: null argument");
    auto it = g->by_name.find(name);
    if (it == g->by_name.end()) return fail(INFR_ERR_LOADER, "tensor not found: '%s'", name);
    fill(g->tensors[it->second], out);
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_tensor_find"); }

extern "C" infr_status infr_gguf_tensor_bytes(const infr_gguf* g, const char* name, const void** data, uint64_t* nbytes) try {
    if (!g || !name || !data) return fail(INFR_ERR_INVALID, "gguf: null argument");
    auto it = g->by_name.find(name);
    if (it == g->by_name.end()) return fail(INFR_ERR_LOADER, "tensor not found: '%s'", name);
    const Tensor& t = g->tensors[it->second];
    // the shard holding an offset is the last one that starts at or before it
    size_t si = 0;
    while (si + 1 < g->shards.size() && g->shards[si + 1].file_base <= t.offset) si++;
    const Shard& sh = g->shards[si];
    const uint64_t off = t.offset - sh.file_base;
    uint64_t end;
    if (__builtin_add_overflow(off, t.nbytes, &end) || end > sh.len)
        return fail(INFR_ERR_LOADER, "tensor '%s' byte range %llu..+%llu exceeds the %zu bytes of %s", name,
                    (unsigned long long)off, (unsigned long long)t.nbytes, sh.len, sh.path.c_str());
    *data = static_cast<const uint8_t*>(sh.map) + off;
    if (nbytes) *nbytes = t.nbytes;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_tensor_bytes"); }

extern "C" infr_status infr_gguf_meta_u64(const infr_gguf* g, const char* key, uint64_t* out) try {
    if (!g || !key || !out) return fail(INFR_ERR_INVALID, "gguf: null argument");
    if (!meta_u64(g->meta(), key, out)) return fail(INFR_ERR_INVALID, "gguf: no unsigned metadata value '%s'", key);
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_meta_u64"); }
extern "C" infr_status infr_gguf_meta_i64(const infr_gguf* g, const char* key, int64_t* out) try {
    if (!g || !key || !out) return fail(INFR_ERR_INVALID, "gguf: null argument");
    auto it = g->meta().find(key);
    if (it != g->meta().end() && it->second.kind == Meta::I64) { *out = it->second.i; return INFR_OK; }
    if (it != g->meta().end() && it->second.kind == Meta::U64 && it->second.u <= (uint64_t)INT64_MAX) { *out = (int64_t)it->second.u; return INFR_OK; }
    return fail(INFR_ERR_INVALID, "gguf: no integer metadata value '%s'", key);
} catch (...) { return guard_fail("infr_gguf_meta_i64"); }
extern "C" infr_status infr_gguf_meta_f64(const infr_gguf* g, const char* key, double* out) try {
    const Meta* m = find_meta(g, key, Meta::F64, "a float");
    if (!m || !out) return INFR_ERR_INVALID;
    *out = m->f;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_meta_f64"); }
extern "C" infr_status infr_gguf_meta_bool(const infr_gguf* g, const char* key, int32_t* out) try {
    const Meta* m = find_meta(g, key, Meta::BOOL, "a bool");
    if (!m || !out) return INFR_ERR_INVALID;
    *out = (int32_t)m->u;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_meta_bool"); }
extern "C" infr_status infr_gguf_meta_str(const infr_gguf* g, const char* key, const char** data, uint64_t* len) try {
    const Meta* m = find_meta(g, key, Meta::STR, "a string");
    if (!m || !data || !len) return INFR_ERR_INVALID;
    *data = m->s.data();
    *len = m->s.size();
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_meta_str"); }
extern "C" infr_status infr_gguf_meta_array_len(const infr_gguf* g, const char* key, uint64_t* out) try {
    const Meta* m = find_meta(g, key, Meta::ARR, "an array");
    if (!m || !out) return INFR_ERR_INVALID;
    *out = m->u;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_meta_array_len"); }

extern "C" infr_status infr_gguf_block_layout(int32_t dtype, uint32_t* block_elems, uint32_t* block_bytes) try {
    uint32_t e, b;
    if (!block_layout(dtype, &e, &b)) return fail(INFR_ERR_UNSUPPORTED, "gguf: dtype %d has no block layout", dtype);
    if (block_elems) *block_elems = e;
    if (block_bytes) *block_bytes = b;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_block_layout"); }

extern "C" infr_status infr_gguf_bind_weight(const infr_gguf* g, const char* name, infr_hip_backend* be,
                                             infr_hip_buffer** out, int32_t* dtype, uint64_t* numel) try {
    if (!out) return fail(INFR_ERR_INVALID, "gguf bind: null argument");
    *out = nullptr;
    infr_gguf_tensor t;
    if (infr_status st = infr_gguf_tensor_find(g, name, &t)) return st;
    const void* data = nullptr;
    if (infr_status st = infr_gguf_tensor_bytes(g, name, &data, nullptr)) return st;
    infr_hip_buffer* buf = nullptr;
    infr_status st = infr_hip_alloc_uninit(be, (size_t)t.nbytes, INFR_USAGE_WEIGHTS, &buf);
    if (st == INFR_OK) st = infr_hip_upload(be, buf, data, (size_t)t.nbytes);
    if (st != INFR_OK) {
        g_err = std::string("gguf bind '") + name + "': " + infr_hip_last_error();
        if (buf) infr_hip_buffer_free(buf);
        return st;
    }
    *out = buf;
    if (dtype) *dtype = t.dtype;
    if (numel) *numel = t.numel;
    return INFR_OK;
} catch (...) { return guard_fail("infr_gguf_bind_weight"); }
