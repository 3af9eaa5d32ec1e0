// GGUF model-file reader: header, metadata, tensor directory, `gguf-split` shard sets, and the
// weight upload into backend buffers. Host code only.
//
// Behaviour follows the reference reader (crates/infr-gguf/src/lib.rs:156-1008) and its shard-name
// helper (crates/infr-core/src/gguf_split.rs:44-88): the same files open, the same files are
// refused, and a refusal names the same tensor / key / shard. The structure is this library's own:
// one cursor over a read-only mapping, a flat value arena, and a name index built once at open.
#include "../../include/infr_gguf.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

struct infr_gguf_value {
    int kind = INFR_GGUF_U64;
    union {
        uint64_t u;
        int64_t i;
        double f;
        bool b;
    };
    std::string s;
    std::vector<infr_gguf_value> arr;
    infr_gguf_value() : u(0) {}
};

namespace {

constexpr uint32_t kMagic = 0x46554747u;  // "GGUF" little-endian (lib.rs:32)
constexpr uint64_t kDefaultAlignment = 32;        // lib.rs:33
constexpr uint64_t kMaxAlignment = 16ull << 20;   // lib.rs:44
constexpr uint32_t kMaxDims = 4;                  // lib.rs:53
constexpr size_t kMaxMetaDepth = 64;              // lib.rs:67
constexpr int kI2S = 36;
const char* const kSplitNo = "split.no";
const char* const kSplitCount = "split.count";
const char* const kSplitTensors = "split.tensors.count";

thread_local std::string g_last_error;

struct Failure {
    int status;
    std::string msg;
};

[[noreturn]] void fail(int status, std::string msg) { throw Failure{status, std::move(msg)}; }
[[noreturn]] void loader(std::string msg) { fail(INFR_HIP_ERR_LOADER, std::move(msg)); }

std::string u64s(uint64_t v) { return std::to_string(v); }

// Rust's str::from_utf8 acceptance: shortest-form sequences only, no surrogates, <= U+10FFFF.
bool valid_utf8(const uint8_t* p, size_t n) {
    size_t i = 0;
    while (i < n) {
        const uint8_t c = p[i];
        if (c < 0x80) { ++i; continue; }
        size_t need;
        uint8_t lo = 0x80, hi = 0xBF;
        if (c >= 0xC2 && c <= 0xDF) need = 1;
        else if (c == 0xE0) { need = 2; lo = 0xA0; }
        else if (c >= 0xE1 && c <= 0xEC) need = 2;
        else if (c == 0xED) { need = 2; hi = 0x9F; }
        else if (c >= 0xEE && c <= 0xEF) need = 2;
        else if (c == 0xF0) { need = 3; lo = 0x90; }
        else if (c >= 0xF1 && c <= 0xF3) need = 3;
        else if (c == 0xF4) { need = 3; hi = 0x8F; }
        else return false;
        if (n - i <= need) return false;
        if (p[i + 1] < lo || p[i + 1] > hi) return false;
        for (size_t k = 2; k <= need; ++k)
            if ((p[i + k] & 0xC0) != 0x80) return false;
        i += need + 1;
    }
    return true;
}

// ── block geometry of every ggml type the reader accepts ────────────────────────────────────
struct TypeRow { int id, elems, bytes; const char* name; };
constexpr TypeRow kTypes[] = {
    {0, 1, 4, "F32"},        {1, 1, 2, "F16"},        {2, 32, 18, "Q4_0"},     {3, 32, 20, "Q4_1"},
    {6, 32, 22, "Q5_0"},     {7, 32, 24, "Q5_1"},     {8, 32, 34, "Q8_0"},     {10, 256, 84, "Q2K"},
    {11, 256, 110, "Q3K"},   {12, 256, 144, "Q4K"},   {13, 256, 176, "Q5K"},   {14, 256, 210, "Q6K"},
    {16, 256, 66, "Iq2Xxs"}, {17, 256, 74, "Iq2Xs"},  {18, 256, 98, "Iq3Xxs"}, {19, 256, 50, "Iq1S"},
    {20, 32, 18, "Iq4Nl"},   {21, 256, 110, "Iq3S"},  {22, 256, 82, "Iq2S"},   {23, 256, 136, "Iq4Xs"},
    {26, 1, 4, "I32"},       {29, 256, 56, "Iq1M"},   {30, 1, 2, "Bf16"},      {34, 256, 54, "Tq1_0"},
    {35, 256, 66, "Tq2_0"},  {36, 4, 1, "I2S"},       {39, 32, 17, "Mxfp4"},   {40, 64, 36, "Nvfp4"},
    {42, 64, 18, "Q2_0"},
};

const TypeRow* type_row(int id) {
    for (const TypeRow& r : kTypes)
        if (r.id == id) return &r;
    return nullptr;
}

// checked_tensor_nbytes (lib.rs:387-406): whole blocks, rounded up; I2_S adds its f32 scale.
bool checked_nbytes(const TypeRow& t, uint64_t numel, uint64_t* out) {
    const uint64_t e = (uint64_t)t.elems;
    const uint64_t blocks = numel / e + (numel % e != 0);
    if (t.id == kI2S) {
        if (blocks > UINT64_MAX - 4) return false;
        *out = blocks + 4;
        return true;
    }
    return !__builtin_mul_overflow(blocks, (uint64_t)t.bytes, out);
}

// ── cursor over one mapped file ─────────────────────────────────────────────────────────────
struct Cursor {
    const uint8_t* buf;
    size_t len;
    size_t pos = 0;

    size_t remaining() const { return len - pos; }
    void need(uint64_t n) const {
        if (n > UINT64_MAX - pos) loader("GGUF: length " + u64s(n) + " at offset " + u64s(pos) + " overflows");
        if (pos + n > len)
            loader("GGUF: unexpected EOF at offset " + u64s(pos) + " (need " + u64s(n) +
                   " more bytes, file is " + u64s(len) + " bytes)");
    }
    template <typename T> T le() {
        need(sizeof(T));
        T v;
        std::memcpy(&v, buf + pos, sizeof(T));  // host is little-endian, as the file is
        pos += sizeof(T);
        return v;
    }
    std::string str() {
        const uint64_t n = le<uint64_t>();
        need(n);
        if (!valid_utf8(buf + pos, (size_t)n)) loader("GGUF: invalid UTF-8 string at offset " + u64s(pos));
        std::string s((const char*)buf + pos, (size_t)n);
        pos += (size_t)n;
        return s;
    }
    // read_meta_value_at_depth (lib.rs:278-316)
    void value(uint32_t vtype, size_t depth, infr_gguf_value& out) {
        switch (vtype) {
        case 0: out.kind = INFR_GGUF_U64; out.u = le<uint8_t>(); break;
        case 1: out.kind = INFR_GGUF_I64; out.i = le<int8_t>(); break;
        case 2: out.kind = INFR_GGUF_U64; out.u = le<uint16_t>(); break;
        case 3: out.kind = INFR_GGUF_I64; out.i = le<int16_t>(); break;
        case 4: out.kind = INFR_GGUF_U64; out.u = le<uint32_t>(); break;
        case 5: out.kind = INFR_GGUF_I64; out.i = le<int32_t>(); break;
        case 6: out.kind = INFR_GGUF_F64; out.f = (double)le<float>(); break;
        case 7: out.kind = INFR_GGUF_BOOL; out.b = le<uint8_t>() != 0; break;
        case 8: out.kind = INFR_GGUF_STR; out.s = str(); break;
        case 9: {
            if (depth >= kMaxMetaDepth)
                loader("GGUF: metadata array nesting exceeds the maximum depth of " + u64s(kMaxMetaDepth) +
                       " at offset " + u64s(pos));
            const uint32_t et = le<uint32_t>();
            const uint64_t count = le<uint64_t>();
            out.kind = INFR_GGUF_ARR;
            // `count` is whatever the file says: reserve a bounded amount and let the vector grow,
            // so a bogus count on a small file fails on the element read's EOF, not on the reserve
            out.arr.reserve((size_t)std::min<uint64_t>(std::min<uint64_t>(count, remaining()), 1u << 16));
            for (uint64_t k = 0; k < count; ++k) {
                out.arr.emplace_back();
                value(et, depth + 1, out.arr.back());
            }
            break;
        }
        case 10: out.kind = INFR_GGUF_U64; out.u = le<uint64_t>(); break;
        case 11: out.kind = INFR_GGUF_I64; out.i = le<int64_t>(); break;
        case 12: out.kind = INFR_GGUF_F64; out.f = le<double>(); break;
        default: loader("GGUF: unknown value type " + u64s(vtype));
        }
    }
};

struct Mapping {
    const uint8_t* data = nullptr;
    size_t len = 0;
    ~Mapping() {
        if (data && len) munmap((void*)data, len);
    }
};

struct Tensor {
    std::string name;
    int ggml_type = 0;
    int n_dims = 0;
    uint64_t shape[4] = {0, 0, 0, 0};
    uint64_t numel = 0;
    uint64_t offset = 0;
    uint64_t nbytes = 0;
};

struct Metadata {
    std::vector<std::string> keys;  // file order, first occurrence
    std::unordered_map<std::string, infr_gguf_value> kv;

    const infr_gguf_value* get(const std::string& k) const {
        auto it = kv.find(k);
        return it == kv.end() ? nullptr : &it->second;
    }
    bool u64(const char* k, uint64_t* out) const {
        const infr_gguf_value* v = get(k);
        return v && infr_gguf_value_u64(v, out);
    }
};

// One file parsed on its own (ShardParts, lib.rs:971-981): tensor offsets still relative to its
// own data region.
struct Part {
    std::unique_ptr<Mapping> map;
    Metadata meta;
    std::vector<Tensor> tensors;
    uint64_t data_start = 0;
    std::string path;
};

std::string shape_text(const Tensor& t) {
    std::string s = "[";
    for (int d = 0; d < t.n_dims; ++d) s += (d ? ", " : "") + u64s(t.shape[d]);
    return s + "]";
}

// map_and_parse (lib.rs:711-889)
Part parse_file(const std::string& path) {
    Part p;
    p.path = path;
    p.map.reset(new Mapping);
    const int fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) fail(INFR_HIP_ERR_IO, path + ": " + std::strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) {
        const int e = errno;
        close(fd);
        fail(INFR_HIP_ERR_IO, path + ": " + std::strerror(e));
    }
    if (st.st_size > 0) {
        void* m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_SHARED, fd, 0);
        const int e = errno;
        close(fd);
        if (m == MAP_FAILED) fail(INFR_HIP_ERR_IO, path + ": mmap: " + std::strerror(e));
        p.map->data = (const uint8_t*)m;
        p.map->len = (size_t)st.st_size;
        // Advisory only: start read-ahead of the whole file now and ask for huge pages; weight
        // bytes are re-read in full on every token, so no drop-behind hint (lib.rs:717-733).
        madvise(m, p.map->len, MADV_WILLNEED);
        madvise(m, p.map->len, MADV_HUGEPAGE);
    } else {
        close(fd);
    }

    Cursor r{p.map->data, p.map->len};
    const uint32_t magic = r.le<uint32_t>();
    if (magic != kMagic) {
        char b[96];
        std::snprintf(b, sizeof b, "not a GGUF file (magic 0x%08X, expected 0x%08X)", magic, kMagic);
        loader(b);
    }
    const uint32_t version = r.le<uint32_t>();
    if (version != 2 && version != 3)
        loader("unsupported GGUF version " + u64s(version) + " (supported: 2, 3)");
    const uint64_t tensor_count = r.le<uint64_t>();
    const uint64_t kv_count = r.le<uint64_t>();

    for (uint64_t k = 0; k < kv_count; ++k) {
        std::string key = r.str();
        const uint32_t vtype = r.le<uint32_t>();
        infr_gguf_value v;
        r.value(vtype, 0, v);
        auto it = p.meta.kv.find(key);
        if (it == p.meta.kv.end()) {
            p.meta.keys.push_back(key);
            p.meta.kv.emplace(std::move(key), std::move(v));
        } else {
            it->second = std::move(v);  // a repeated key keeps its last value
        }
    }

    uint64_t alignment = kDefaultAlignment;
    p.meta.u64("general.alignment", &alignment);
    if (alignment == 0 || (alignment & (alignment - 1)) != 0)
        loader("GGUF: invalid general.alignment " + u64s(alignment) + " (must be a positive power of two)");
    if (alignment > kMaxAlignment)
        loader("GGUF: invalid general.alignment " + u64s(alignment) + " (exceeds the " + u64s(kMaxAlignment) +
               "-byte cap)");

    p.tensors.reserve((size_t)std::min<uint64_t>(std::min<uint64_t>(tensor_count, r.remaining()), 1u << 16));
    for (uint64_t k = 0; k < tensor_count; ++k) {
        Tensor t;
        t.name = r.str();
        const uint32_t n_dims = r.le<uint32_t>();
        if (n_dims > kMaxDims)
            loader("GGUF: tensor '" + t.name + "' declares " + u64s(n_dims) + " dimensions (max " +
                   u64s(kMaxDims) + ")");
        t.n_dims = (int)n_dims;
        for (uint32_t d = 0; d < n_dims; ++d) t.shape[d] = r.le<uint64_t>();
        t.ggml_type = (int)r.le<uint32_t>();
        t.offset = r.le<uint64_t>();
        p.tensors.push_back(std::move(t));
    }

    p.data_start = ((uint64_t)r.pos + alignment - 1) / alignment * alignment;

    // Types and sizes are checked only after the whole directory has been read (lib.rs:810-871).
    for (Tensor& t : p.tensors) {
        const TypeRow* row = type_row(t.ggml_type);
        if (!row) fail(INFR_HIP_ERR_UNSUPPORTED, "ggml type " + u64s((uint32_t)t.ggml_type));
        uint64_t numel = 1;
        for (int d = 0; d < t.n_dims; ++d)
            if (__builtin_mul_overflow(numel, t.shape[d], &numel))
                loader("GGUF: tensor '" + t.name + "' shape " + shape_text(t) + " overflows");
        t.numel = numel;
        if (row->id == kI2S) {
            if (numel % 4 != 0)
                loader("GGUF: tensor '" + t.name + "' shape " + shape_text(t) + " has " + u64s(numel) +
                       " elements, not a multiple of 4 (i2_s packs 4 2-bit codes per byte)");
        } else if (numel % (uint64_t)row->elems != 0) {
            loader("GGUF: tensor '" + t.name + "' shape " + shape_text(t) + " has " + u64s(numel) +
                   " elements, not a whole number of " + row->name + " blocks (" + u64s((uint64_t)row->elems) +
                   " elements per block)");
        }
        if (!checked_nbytes(*row, numel, &t.nbytes))
            loader("GGUF: tensor '" + t.name + "' shape " + shape_text(t) + " byte size overflows");
    }
    return p;
}

struct ShardName {
    std::string base;
    uint32_t index = 0, total = 0;
    size_t width = 0;
};

bool all_digits(const std::string& s) {
    if (s.empty()) return false;
    for (char c : s)
        if (c < '0' || c > '9') return false;
    return true;
}

// parse_shard (gguf_split.rs:44-68)
bool parse_shard(const std::string& fname, ShardName* out) {
    if (fname.size() < 5) return false;
    const std::string suffix = fname.substr(fname.size() - 5);
    for (int k = 0; k < 5; ++k) {
        char c = suffix[(size_t)k];
        if (c >= 'A' && c <= 'Z') c = (char)(c - 'A' + 'a');
        if (c != ".gguf"[k]) return false;
    }
    const std::string stem = fname.substr(0, fname.size() - 5);
    const size_t of = stem.rfind("-of-");
    if (of == std::string::npos) return false;
    const std::string left = stem.substr(0, of), total_s = stem.substr(of + 4);
    const size_t dash = left.rfind('-');
    if (dash == std::string::npos) return false;
    const std::string idx_s = left.substr(dash + 1);
    if (!all_digits(total_s) || !all_digits(idx_s) || total_s.size() != idx_s.size() || total_s.size() > 5)
        return false;
    out->base = left.substr(0, dash);
    out->index = (uint32_t)std::stoul(idx_s);
    out->total = (uint32_t)std::stoul(total_s);
    out->width = total_s.size();
    return true;
}

std::string shard_file_name(const ShardName& s, uint32_t i) {
    char num[2][16];
    std::snprintf(num[0], sizeof num[0], "%0*u", (int)s.width, i);
    std::snprintf(num[1], sizeof num[1], "%0*u", (int)s.width, s.total);
    return s.base + "-" + num[0] + "-of-" + num[1] + ".gguf";
}

std::string base_name(const std::string& path) {
    const size_t slash = path.rfind('/');
    return slash == std::string::npos ? path : path.substr(slash + 1);
}

std::string dir_name(const std::string& path) {
    const size_t slash = path.rfind('/');
    if (slash == std::string::npos) return ".";
    return slash == 0 ? "/" : path.substr(0, slash);
}

// check_shard_position (lib.rs:591-622): `index0` is the position the file NAME claims.
void check_shard_position(const Part& p, size_t index0, uint64_t count) {
    const std::string where = p.path + " is named as shard " + u64s(index0 + 1) + " of " + u64s(count);
    uint64_t no;
    if (!p.meta.u64(kSplitNo, &no))
        loader("GGUF: " + where + " but carries no " + kSplitNo + " - it is not part of a `gguf-split` set");
    if (no != index0)
        loader("GGUF: " + where + " but declares " + kSplitNo + " = " + u64s(no) + " (shard " + u64s(no + 1) +
               ") - its name and its metadata disagree about which shard it is");
    uint64_t declared;
    if (!p.meta.u64(kSplitCount, &declared)) loader("GGUF: " + where + " but carries no " + kSplitCount);
    if (declared != count)
        loader("GGUF: " + p.path + " declares " + kSplitCount + " = " + u64s(declared) +
               " but the rest of the set declares " + u64s(count) + " - these files are not one model");
}

struct Shard {
    std::unique_ptr<Mapping> map;
    std::string path;
    uint64_t file_base = 0;
};

}  // namespace

struct infr_gguf {
    std::vector<Shard> shards;
    Metadata meta;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, size_t> by_name;
};

namespace {

// assemble (lib.rs:628-706): shards end to end, offsets rewritten into the concatenated space.
infr_gguf* assemble(std::vector<Part>& parts, const uint64_t* expect_tensors) {
    std::unique_ptr<infr_gguf> g(new infr_gguf);
    uint64_t file_base = 0;
    bool first = true;
    for (Part& p : parts) {
        uint64_t data_base;
        if (__builtin_add_overflow(file_base, p.data_start, &data_base))
            loader("GGUF: shard set is larger than u64 bytes");
        for (Tensor& t : p.tensors)
            if (__builtin_add_overflow(data_base, t.offset, &t.offset))
                loader("tensor '" + t.name + "' offset overflows u64");
        Shard s;
        s.path = p.path;
        s.file_base = file_base;
        if (__builtin_add_overflow(file_base, (uint64_t)p.map->len, &file_base))
            loader("GGUF: shard set is larger than u64 bytes");
        s.map = std::move(p.map);
        g->shards.push_back(std::move(s));
        for (Tensor& t : p.tensors) g->tensors.push_back(std::move(t));
        if (first) g->meta = std::move(p.meta);  // later shards carry only split.* keys
        first = false;
    }
    g->by_name.reserve(g->tensors.size());
    for (size_t i = 0; i < g->tensors.size(); ++i)
        if (!g->by_name.emplace(g->tensors[i].name, i).second)
            loader("GGUF: duplicate tensor name '" + g->tensors[i].name +
                   "' - the file declares it more than once, so which entry a lookup resolves to is ambiguous");
    if (expect_tensors && (uint64_t)g->tensors.size() != *expect_tensors)
        loader("GGUF: the " + u64s(g->shards.size()) + " shards hold " + u64s(g->tensors.size()) +
               " tensors between them but the model declares " + kSplitTensors + " = " + u64s(*expect_tensors) +
               " - the set is incomplete or mismatched");
    return g.release();
}

// open_split (lib.rs:496-583)
infr_gguf* open_split(Part opened, uint64_t count) {
    const std::string fname = base_name(opened.path);
    ShardName sn;
    if (!parse_shard(fname, &sn))
        loader("GGUF: " + fname + " declares " + kSplitCount + " = " + u64s(count) +
               ", but its name is not a `<base>-NNNNN-of-MMMMM.gguf` shard name, so the rest of the set cannot "
               "be found - rename the shards to the `gguf-split` convention");
    if ((uint64_t)sn.total != count)
        loader("GGUF: " + fname + " is named as one of " + u64s(sn.total) + " shards but declares " + kSplitCount +
               " = " + u64s(count) + " - the file's name and its metadata disagree about how many shards this "
               "model has");
    if (sn.index < 1 || (uint64_t)sn.index > count)
        loader("GGUF: " + fname + " is numbered " + u64s(sn.index) + " of " + u64s(count) +
               " - a shard's index runs from 1 to the total, so this file is not a member of the set its own "
               "name describes");
    const std::string dir = dir_name(opened.path);
    const size_t opened_idx = (size_t)sn.index - 1;
    check_shard_position(opened, opened_idx, count);

    std::vector<Part> parts;
    parts.reserve((size_t)count);
    for (size_t i = 0; i < (size_t)count; ++i) {
        if (i == opened_idx) {
            parts.push_back(std::move(opened));
            continue;
        }
        const std::string path = dir + "/" + shard_file_name(sn, (uint32_t)i + 1);
        try {
            parts.push_back(parse_file(path));
        } catch (Failure& f) {
            // every failure inside a sibling shard is a failure of the SET (lib.rs:553-559)
            loader("GGUF: shard " + u64s(i + 1) + " of " + u64s(count) + " (" + path + "): " + f.msg);
        }
        check_shard_position(parts.back(), i, count);
    }
    uint64_t expect;
    if (!parts[0].meta.u64(kSplitTensors, &expect))
        loader("GGUF: " + parts[0].path + " declares " + kSplitCount + " = " + u64s(count) + " but carries no " +
               kSplitTensors + ", so the assembled tensor index cannot be checked for completeness");
    return assemble(parts, &expect);
}

infr_gguf* open_model(const char* path) {
    Part first = parse_file(path);
    uint64_t count;
    if (first.meta.u64(kSplitCount, &count) && count > 1) return open_split(std::move(first), count);
    std::vector<Part> parts;
    parts.push_back(std::move(first));
    return assemble(parts, nullptr);
}

struct Resolved {
    const Shard* shard;
    size_t off, len;
};

// resolve (lib.rs:942-969)
Resolved resolve(const infr_gguf* g, const char* name) {
    auto it = g->by_name.find(name);
    if (it == g->by_name.end()) loader(std::string("tensor not found: '") + name + "'");
    const Tensor& t = g->tensors[it->second];
    // shards are ordered by file_base and cover their whole file: the owner is the last one
    // that starts at or before the offset
    size_t idx = 0;
    while (idx + 1 < g->shards.size() && g->shards[idx + 1].file_base <= t.offset) ++idx;
    const Shard& s = g->shards[idx];
    const uint64_t off = t.offset - s.file_base;
    uint64_t end;
    if (__builtin_add_overflow(off, t.nbytes, &end)) loader("tensor '" + t.name + "' byte range overflows");
    if (end > s.map->len)
        loader("tensor '" + t.name + "' byte range " + u64s(off) + ".." + u64s(end) + " exceeds the " +
               u64s(s.map->len) + " bytes of " + s.path);
    return Resolved{&s, (size_t)off, (size_t)t.nbytes};
}

template <typename F> int guarded(F&& body) {
    try {
        body();
        return INFR_HIP_OK;
    } catch (Failure& f) {
        g_last_error = std::move(f.msg);
        return f.status;
    } catch (std::bad_alloc&) {
        g_last_error = "out of host memory";
        return INFR_HIP_ERR_OTHER;
    }
}

int invalid(const char* msg) {
    g_last_error = msg;
    return INFR_HIP_ERR_INVALID;
}

}  // namespace

extern "C" {

int infr_gguf_open(const char* path, infr_gguf_t** out) {
    if (!path || !out) return invalid("infr_gguf_open: null argument");
    *out = nullptr;
    return guarded([&] { *out = open_model(path); });
}

void infr_gguf_close(infr_gguf_t* g) { delete g; }

const char* infr_gguf_last_error(void) { return g_last_error.c_str(); }

size_t infr_gguf_n_tensors(const infr_gguf_t* g) { return g ? g->tensors.size() : 0; }

int infr_gguf_tensor(const infr_gguf_t* g, size_t index, infr_gguf_tensor_t* out) {
    if (!g || !out || index >= g->tensors.size()) return invalid("infr_gguf_tensor: index out of range");
    const Tensor& t = g->tensors[index];
    out->name = t.name.c_str();
    out->ggml_type = t.ggml_type;
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; ++d) out->shape[d] = t.shape[d];
    out->numel = t.numel;
    out->offset = t.offset;
    out->nbytes = (size_t)t.nbytes;
    return INFR_HIP_OK;
}

int64_t infr_gguf_find(const infr_gguf_t* g, const char* name) {
    if (!g || !name) return -1;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? -1 : (int64_t)it->second;
}

int infr_gguf_tensor_bytes(const infr_gguf_t* g, const char* name, const void** data, size_t* len) {
    if (!g || !name || !data || !len) return invalid("infr_gguf_tensor_bytes: null argument");
    return guarded([&] {
        const Resolved r = resolve(g, name);
        *data = r.shard->map->data + r.off;
        *len = r.len;
    });
}

int infr_gguf_tensor_file_range(const infr_gguf_t* g, const char* name, uint64_t* offset, size_t* len) {
    if (!g || !name || !offset || !len) return invalid("infr_gguf_tensor_file_range: null argument");
    return guarded([&] {
        const Resolved r = resolve(g, name);
        *offset = r.shard->file_base + r.off;
        *len = r.len;
    });
}

size_t infr_gguf_n_shards(const infr_gguf_t* g) { return g ? g->shards.size() : 0; }

int infr_gguf_shard(const infr_gguf_t* g, size_t index, const char** path, uint64_t* len) {
    if (!g || index >= g->shards.size()) return invalid("infr_gguf_shard: index out of range");
    if (path) *path = g->shards[index].path.c_str();
    if (len) *len = g->shards[index].map->len;
    return INFR_HIP_OK;
}

size_t infr_gguf_n_meta(const infr_gguf_t* g) { return g ? g->meta.keys.size() : 0; }

const char* infr_gguf_meta_key(const infr_gguf_t* g, size_t index) {
    return g && index < g->meta.keys.size() ? g->meta.keys[index].c_str() : nullptr;
}

const infr_gguf_value_t* infr_gguf_meta_get(const infr_gguf_t* g, const char* key) {
    return g && key ? g->meta.get(key) : nullptr;
}

int infr_gguf_value_kind(const infr_gguf_value_t* v) { return v ? v->kind : -1; }

int infr_gguf_value_u64(const infr_gguf_value_t* v, uint64_t* out) {
    if (!v || !out) return 0;
    if (v->kind == INFR_GGUF_U64) { *out = v->u; return 1; }
    // a negative count is not a count: refuse it rather than wrap (loader.rs:23-26)
    if (v->kind == INFR_GGUF_I64 && v->i >= 0) { *out = (uint64_t)v->i; return 1; }
    return 0;
}

int infr_gguf_value_i64(const infr_gguf_value_t* v, int64_t* out) {
    if (!v || !out) return 0;
    if (v->kind == INFR_GGUF_I64) { *out = v->i; return 1; }
    if (v->kind == INFR_GGUF_U64 && v->u <= (uint64_t)INT64_MAX) { *out = (int64_t)v->u; return 1; }
    return 0;
}

int infr_gguf_value_f64(const infr_gguf_value_t* v, double* out) {
    if (!v || !out) return 0;
    if (v->kind == INFR_GGUF_F64) { *out = v->f; return 1; }
    if (v->kind == INFR_GGUF_U64) { *out = (double)v->u; return 1; }
    if (v->kind == INFR_GGUF_I64) { *out = (double)v->i; return 1; }
    return 0;
}

int infr_gguf_value_bool(const infr_gguf_value_t* v, int* out) {
    if (!v || !out || v->kind != INFR_GGUF_BOOL) return 0;
    *out = v->b ? 1 : 0;
    return 1;
}

int infr_gguf_value_str(const infr_gguf_value_t* v, const char** s, size_t* len) {
    if (!v || !s || v->kind != INFR_GGUF_STR) return 0;
    *s = v->s.c_str();
    if (len) *len = v->s.size();
    return 1;
}

int infr_gguf_value_arr_len(const infr_gguf_value_t* v, size_t* len) {
    if (!v || !len || v->kind != INFR_GGUF_ARR) return 0;
    *len = v->arr.size();
    return 1;
}

const infr_gguf_value_t* infr_gguf_value_arr_at(const infr_gguf_value_t* v, size_t index) {
    return v && v->kind == INFR_GGUF_ARR && index < v->arr.size() ? &v->arr[index] : nullptr;
}

const char* infr_gguf_chat_template(const infr_gguf_t* g) {
    const infr_gguf_value_t* v = infr_gguf_meta_get(g, "tokenizer.chat_template");
    return v && v->kind == INFR_GGUF_STR ? v->s.c_str() : nullptr;
}

int infr_gguf_block_layout(int ggml_type, int* elems, int* bytes) {
    const TypeRow* r = type_row(ggml_type);
    if (!r) return 0;
    if (elems) *elems = r->elems;
    if (bytes) *bytes = r->bytes;
    return 1;
}

size_t infr_gguf_nbytes(int ggml_type, uint64_t numel, int* ok) {
    const TypeRow* r = type_row(ggml_type);
    uint64_t n = 0;
    const bool good = r && checked_nbytes(*r, numel, &n);
    if (ok) *ok = good ? 1 : 0;
    return good ? (size_t)n : 0;
}

int infr_gguf_parse_shard(const char* fname, char* base, size_t base_cap, size_t* base_len, uint32_t* index,
                          uint32_t* total, size_t* width) {
    ShardName s;
    if (!fname || !parse_shard(fname, &s)) return 0;
    if (base && base_cap) {
        const size_t n = std::min(base_cap - 1, s.base.size());
        std::memcpy(base, s.base.data(), n);
        base[n] = 0;
    }
    if (base_len) *base_len = s.base.size();
    if (index) *index = s.index;
    if (total) *total = s.total;
    if (width) *width = s.width;
    return 1;
}

size_t infr_gguf_shard_set(const char* fname, size_t i, char* out, size_t out_cap) {
    if (!fname) return 0;
    ShardName s;
    std::string name = fname;
    size_t n = 1;
    if (parse_shard(fname, &s) && s.total >= 1) {
        n = s.total;
        if (i < n) name = shard_file_name(s, (uint32_t)i + 1);
    }
    if (out && out_cap && i < n) {
        const size_t c = std::min(out_cap - 1, name.size());
        std::memcpy(out, name.data(), c);
        out[c] = 0;
    }
    return n;
}

int infr_gguf_upload_concat(const infr_gguf_t* g, const char* const* names, size_t n, infr_hip_t* be,
                            infr_hip_buffer_t** out, size_t* offsets) {
    if (!g || !names || !n || !be || !out) return invalid("infr_gguf_upload: null argument");
    *out = nullptr;
    std::vector<Resolved> parts(n);
    size_t total = 0;
    int type = -1;
    const int st = guarded([&] {
        for (size_t i = 0; i < n; ++i) {
            if (!names[i]) fail(INFR_HIP_ERR_INVALID, "infr_gguf_upload: null tensor name");
            parts[i] = resolve(g, names[i]);
            const int t = g->tensors[g->by_name.find(names[i])->second].ggml_type;
            if (type >= 0 && t != type)
                fail(INFR_HIP_ERR_INVALID, std::string("infr_gguf_upload_concat: '") + names[i] + "' has ggml type " +
                                               u64s((uint64_t)t) + ", the tensors before it " + u64s((uint64_t)type));
            type = t;
            if (offsets) offsets[i] = total;
            total += parts[i].len;
        }
        if (total == 0) fail(INFR_HIP_ERR_INVALID, "infr_gguf_upload: nothing to upload (zero bytes)");
    });
    if (st != INFR_HIP_OK) return st;
    infr_hip_buffer_t* buf = nullptr;
    int rc = infr_hip_alloc_uninit(be, total, INFR_USAGE_WEIGHTS, &buf);
    size_t at = 0;
    for (size_t i = 0; rc == INFR_HIP_OK && i < n; ++i) {
        if (parts[i].len) rc = infr_hip_upload_at(be, buf, at, parts[i].shard->map->data + parts[i].off, parts[i].len);
        at += parts[i].len;
    }
    if (rc != INFR_HIP_OK) {
        g_last_error = std::string("upload failed: ") + infr_hip_last_error(be);
        if (buf) infr_hip_free(be, buf);
        return rc;
    }
    *out = buf;
    return INFR_HIP_OK;
}

int infr_gguf_upload(const infr_gguf_t* g, const char* name, infr_hip_t* be, infr_hip_buffer_t** out) {
    return infr_gguf_upload_concat(g, &name, 1, be, out, nullptr);
}

}  // extern "C"
