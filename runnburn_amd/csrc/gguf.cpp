// GGUF container reader for the quantized-matmul path: header and tensor table are parsed on the host, tensor
// payloads are never transformed — a tensor is (pointer into the caller's mapping, byte length, ggml type, shape)
// and goes to the device with the same untouched upload the operator entry points use.
//
// Follows crates/rnb-loader/src/gguf/parser.rs:247-407 (GGUFFile::parse: limits, checks and message texts),
// crates/rnb-loader/src/gguf/types.rs:5-41 (GGMLType ids), crates/rnb-loader/src/convert.rs:23-83 (block sizes,
// checked_tensor_size) and :99-178 (map_tensors: bounds of every tensor against the file length).
// Error texts are the reference's `LoaderError` Display strings (crates/rnb-loader/src/error.rs:4-16).
// A file opened by path whose metadata declares split.count > 1 is one shard of a split model: the other shards are
// found beside it, mapped and checked as crates/rnb-loader/src/gguf/sharded.rs:22-235 does, and the handle shows the
// union of their tensor tables with shard zero's metadata.
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <errno.h>
#include <stdlib.h>

#include <algorithm>
#include <limits>
#include <memory>
#include <set>
#include <string>
#include <unordered_set>
#include <vector>

#include "../../include/rnb_hip.h"
#include "state.h"

namespace rnb {

namespace {

constexpr uint64_t kMaxStringLength = 64ull * 1024 * 1024;
constexpr uint64_t kMaxArrayElements = 4ull * 1024 * 1024;
constexpr int kMaxArrayNesting = 64;
constexpr size_t kMaxMetadataKeyLength = 65535;
constexpr size_t kMaxTensorNameLength = 64;
constexpr uint64_t kMinMetadataRecordBytes = 13, kMinTensorInfoBytes = 24;

struct QuantParams {
    uint32_t id;
    uint64_t elems, bytes;
};
// ggml type id -> (elements per block, bytes per block), crates/rnb-loader/src/convert.rs:46-83
constexpr QuantParams kTypes[] = {
    {0, 1, 4},      {1, 1, 2},      {30, 1, 2},    {26, 1, 4},    {24, 1, 1},     {25, 1, 2},    {27, 1, 8},
    {28, 1, 8},     {2, 32, 18},    {3, 32, 20},   {6, 32, 22},   {7, 32, 24},    {8, 32, 34},   {9, 32, 36},
    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292}, {16, 256, 66},
    {17, 256, 74},  {18, 256, 98},  {19, 256, 50}, {20, 32, 18},  {21, 256, 110}, {22, 256, 82}, {23, 256, 136},
    {29, 256, 56},  {34, 256, 54},  {35, 256, 66}, {39, 32, 17},  {40, 64, 36},   {41, 128, 18}, {42, 64, 18},
};

const QuantParams *type_params(uint32_t id) {
    for (const QuantParams &t : kTypes)
        if (t.id == id) return &t;
    return nullptr;
}

struct Value {
    uint32_t type = 0;  // GGUF value type 0..12
    uint64_t u = 0;     // integers (zero/sign extended into 64 bits) and bool
    double f = 0.0;     // F32 / F64
    std::string s;      // String
    uint32_t elem_type = 0;  // Array: element type and count (elements themselves are validated, not kept,
    uint64_t count = 0;      // except strings and 32/64-bit numbers of flat arrays)
    std::vector<std::string> strings;
    std::vector<double> numbers;
};

struct Tensor {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t shape[4] = {0, 0, 0, 0};  // row-major: outermost first
    uint32_t ggml_type = 0;
    uint64_t offset = 0, file_offset = 0, n_bytes = 0;
    const rnb_hip_gguf *home = nullptr;  // the shard whose mapping holds the payload (null: the handle itself)
};

struct ParseFailure {
    std::string text;
};

[[noreturn]] void parse_error(size_t offset, const std::string &msg) {
    throw ParseFailure{"parse error at offset " + std::to_string(offset) + ": " + msg};
}

class Reader {
  public:
    Reader(const uint8_t *data, size_t len) : data_(data), len_(len) {}
    size_t pos() const { return pos_; }
    size_t remaining() const { return len_ - pos_; }
    const uint8_t *bytes(size_t n) {
        if (remaining() < n) parse_error(pos_, "need " + std::to_string(n) + " bytes, only " + std::to_string(remaining()) + " remain");
        const uint8_t *p = data_ + pos_;
        pos_ += n;
        return p;
    }
    template <typename T>
    T le() {  // little-endian host assumed (x86-64)
        T v;
        memcpy(&v, bytes(sizeof(T)), sizeof(T));
        return v;
    }
    std::string str() {
        const uint64_t len = le<uint64_t>();
        if (len > kMaxStringLength)
            parse_error(pos_ - 8, "string length " + std::to_string(len) + " exceeds maximum supported length " +
                                      std::to_string(kMaxStringLength));
        const size_t at = pos_;
        const uint8_t *p = bytes(static_cast<size_t>(len));
        std::string s(reinterpret_cast<const char *>(p), static_cast<size_t>(len));
        if (!valid_utf8(s)) parse_error(at, "invalid UTF-8 in string");
        return s;
    }

  private:
    static bool valid_utf8(const std::string &s) {
        const unsigned char *p = reinterpret_cast<const unsigned char *>(s.data());
        size_t i = 0, n = s.size();
        while (i < n) {
            const unsigned char c = p[i];
            size_t need;
            uint32_t cp;
            if (c < 0x80) { i++; continue; }
            if (c >= 0xC2 && c <= 0xDF) { need = 1; cp = c & 0x1F; }
            else if (c >= 0xE0 && c <= 0xEF) { need = 2; cp = c & 0x0F; }
            else if (c >= 0xF0 && c <= 0xF4) { need = 3; cp = c & 0x07; }
            else return false;
            if (i + need >= n) return false;  // truncated sequence
            for (size_t k = 1; k <= need; k++) {
                if ((p[i + k] & 0xC0) != 0x80) return false;
                cp = (cp << 6) | (p[i + k] & 0x3F);
            }
            if (need == 2 && (cp < 0x800 || (cp >= 0xD800 && cp <= 0xDFFF))) return false;
            if (need == 3 && (cp < 0x10000 || cp > 0x10FFFF)) return false;
            i += need + 1;
        }
        return true;
    }
    const uint8_t *data_;
    size_t len_, pos_ = 0;
};

void read_value(Reader &r, uint32_t type, int depth, Value *out, bool keep);

void read_scalar(Reader &r, uint32_t type, Value *v) {
    v->type = type;
    switch (type) {
        case 0: v->u = r.le<uint8_t>(); break;
        case 1: v->u = static_cast<uint64_t>(static_cast<int64_t>(r.le<int8_t>())); break;
        case 2: v->u = r.le<uint16_t>(); break;
        case 3: v->u = static_cast<uint64_t>(static_cast<int64_t>(r.le<int16_t>())); break;
        case 4: v->u = r.le<uint32_t>(); break;
        case 5: v->u = static_cast<uint64_t>(static_cast<int64_t>(r.le<int32_t>())); break;
        case 6: v->f = r.le<float>(); break;
        case 7: {
            const size_t at = r.pos();
            const uint8_t b = r.le<uint8_t>();
            if (b > 1) parse_error(at, "invalid GGUF boolean value " + std::to_string(b) + "; expected 0 or 1");
            v->u = b;
            break;
        }
        case 8: v->s = r.str(); break;
        case 10: v->u = r.le<uint64_t>(); break;
        case 11: v->u = static_cast<uint64_t>(r.le<int64_t>()); break;
        case 12: v->f = r.le<double>(); break;
        default: break;
    }
}

void read_value(Reader &r, uint32_t type, int depth, Value *out, bool keep) {
    if (type > 12) parse_error(r.pos(), "unknown GGUF value type: " + std::to_string(type));
    if (depth > kMaxArrayNesting)
        parse_error(r.pos(), "GGUF array nesting exceeds " + std::to_string(kMaxArrayNesting) + " levels");
    if (type != 9) {
        read_scalar(r, type, out);
        return;
    }
    out->type = 9;
    const uint32_t elem_type = r.le<uint32_t>();
    if (elem_type > 12) parse_error(r.pos() - 4, "unknown GGUF value type: " + std::to_string(elem_type));
    const uint64_t count = r.le<uint64_t>();
    if (count > kMaxArrayElements)
        parse_error(r.pos() - 8, "array element count " + std::to_string(count) + " exceeds maximum " +
                                     std::to_string(kMaxArrayElements));
    if (count > r.remaining())
        parse_error(r.pos(), "array element count " + std::to_string(count) + " exceeds " +
                                 std::to_string(r.remaining()) + " remaining bytes");
    out->elem_type = elem_type;
    out->count = count;
    for (uint64_t i = 0; i < count; i++) {
        Value e;
        read_value(r, elem_type, depth + 1, &e, false);
        if (!keep) continue;
        if (elem_type == 8)
            out->strings.push_back(std::move(e.s));
        else if (elem_type == 6 || elem_type == 12)
            out->numbers.push_back(e.f);
        else if (elem_type != 9)
            out->numbers.push_back(elem_type == 1 || elem_type == 3 || elem_type == 5 || elem_type == 11
                                       ? static_cast<double>(static_cast<int64_t>(e.u))
                                       : static_cast<double>(e.u));
    }
}

bool is_ascii(const std::string &s) {
    for (unsigned char c : s)
        if (c >= 0x80) return false;
    return true;
}

}  // namespace

}  // namespace rnb

struct rnb_hip_gguf {
    const uint8_t *data = nullptr;
    size_t len = 0;
    bool owns_mapping = false;
    uint32_t version = 0;
    uint64_t alignment = 32, data_start = 0;
    std::vector<std::pair<std::string, rnb::Value>> metadata;
    std::vector<rnb::Tensor> tensors;
    // a split file opened by path: the other shards (each owns its mapping); `tensors` above is then the union of all
    // shards' tables and `metadata` that of shard zero
    std::vector<std::unique_ptr<rnb_hip_gguf>> shards;
    ~rnb_hip_gguf() {
        if (owns_mapping && data != nullptr) munmap(const_cast<uint8_t *>(data), len);
    }
};

namespace rnb {

namespace {

int fail_gguf(int status, const std::string &msg) {
    set_last_error(msg);
    return status;
}

uint64_t metadata_alignment(const rnb_hip_gguf &g) {
    for (const auto &kv : g.metadata) {
        if (kv.first != "general.alignment") continue;
        const Value &v = kv.second;
        bool ok = false;
        uint64_t a = 0;
        switch (v.type) {
            case 0: case 2: case 4: case 10: ok = true; a = v.u; break;
            case 1: case 3: case 5: case 11: ok = static_cast<int64_t>(v.u) >= 0; a = v.u; break;
            default: break;
        }
        if (!ok) parse_error(0, "general.alignment must be a non-negative integer fitting usize");
        if (a == 0 || (a & (a - 1)) != 0)
            parse_error(0, "general.alignment " + std::to_string(a) + " must be a positive power of two");
        return a;
    }
    return 32;
}

// crates/rnb-loader/src/convert.rs:28-43
bool tensor_size(const uint64_t *shape, uint32_t n_dims, uint32_t ggml_type, uint64_t *bytes, std::string *why) {
    const QuantParams *qp = type_params(ggml_type);
    if (qp == nullptr) {
        *why = "unsupported GGML type: " + std::to_string(ggml_type);
        return false;
    }
    const uint64_t row = n_dims ? shape[n_dims - 1] : 1;
    if (row % qp->elems != 0) {
        *why = "row has " + std::to_string(row) + " elements, not divisible by block size " + std::to_string(qp->elems);
        return false;
    }
    uint64_t numel = 1;
    for (uint32_t i = 0; i < n_dims; i++) {
        if (shape[i] != 0 && numel > std::numeric_limits<uint64_t>::max() / shape[i]) {
            *why = "element count overflows usize";
            return false;
        }
        numel *= shape[i];
    }
    const uint64_t blocks = numel / qp->elems;
    if (blocks != 0 && qp->bytes > std::numeric_limits<uint64_t>::max() / blocks) {
        *why = "tensor byte size overflows usize";
        return false;
    }
    *bytes = blocks * qp->bytes;
    return true;
}

void parse_into(rnb_hip_gguf &g) {
    Reader r(g.data, g.len);
    if (memcmp(r.bytes(4), "GGUF", 4) != 0) throw ParseFailure{"invalid GGUF magic bytes"};
    const size_t version_at = r.pos();
    const uint8_t *vb = r.bytes(4);
    const uint32_t version = static_cast<uint32_t>(vb[0]) | (vb[1] << 8) | (vb[2] << 16) | (static_cast<uint32_t>(vb[3]) << 24);
    if (version != 2 && version != 3) {
        const uint32_t be = static_cast<uint32_t>(vb[3]) | (vb[2] << 8) | (vb[1] << 16) | (static_cast<uint32_t>(vb[0]) << 24);
        if (be == 2 || be == 3) parse_error(version_at, "big-endian GGUF is not supported by the mmap tensor runtime");
        throw ParseFailure{"unsupported GGUF version: " + std::to_string(version)};
    }
    g.version = version;
    const uint64_t tensor_count = r.le<uint64_t>();
    const uint64_t kv_count = r.le<uint64_t>();
    const unsigned __int128 need = static_cast<unsigned __int128>(kv_count) * kMinMetadataRecordBytes +
                                   static_cast<unsigned __int128>(tensor_count) * kMinTensorInfoBytes;
    if (need > std::numeric_limits<uint64_t>::max())
        parse_error(r.pos(), "tensor count " + std::to_string(tensor_count) + " and metadata count " +
                                 std::to_string(kv_count) + " overflow header size");
    if (need > r.remaining())
        parse_error(r.pos(), "tensor count " + std::to_string(tensor_count) + " and metadata count " +
                                 std::to_string(kv_count) + " cannot fit in " + std::to_string(r.remaining()) +
                                 " remaining bytes");

    std::unordered_set<std::string> keys;
    g.metadata.reserve(static_cast<size_t>(kv_count));
    for (uint64_t i = 0; i < kv_count; i++) {
        std::string key = r.str();
        if (key.empty() || key.size() > kMaxMetadataKeyLength || !is_ascii(key))
            parse_error(r.pos() - key.size(), "metadata key must be non-empty ASCII and at most " +
                                                  std::to_string(kMaxMetadataKeyLength) + " bytes");
        if (!keys.insert(key).second) parse_error(r.pos() - key.size(), "duplicate metadata key '" + key + "'");
        const uint32_t type = r.le<uint32_t>();
        Value v;
        read_value(r, type, 0, &v, true);
        g.metadata.emplace_back(std::move(key), std::move(v));
    }
    g.alignment = metadata_alignment(g);

    std::unordered_set<std::string> names;
    g.tensors.reserve(static_cast<size_t>(tensor_count));
    for (uint64_t i = 0; i < tensor_count; i++) {
        Tensor t;
        t.name = r.str();
        if (t.name.size() >= kMaxTensorNameLength)
            parse_error(r.pos() - t.name.size(), "tensor name is " + std::to_string(t.name.size()) +
                                                     " bytes; GGML requires fewer than " +
                                                     std::to_string(kMaxTensorNameLength));
        if (!names.insert(t.name).second) parse_error(r.pos() - t.name.size(), "duplicate tensor name '" + t.name + "'");
        t.n_dims = r.le<uint32_t>();
        if (t.n_dims > 4)
            parse_error(r.pos() - 4, "tensor '" + t.name + "' has " + std::to_string(t.n_dims) +
                                         " dimensions; GGUF supports at most 4");
        uint64_t dims[4] = {0, 0, 0, 0};
        for (uint32_t d = 0; d < t.n_dims; d++) dims[d] = r.le<uint64_t>();
        for (uint32_t d = 0; d < t.n_dims; d++) t.shape[d] = dims[t.n_dims - 1 - d];  // stored innermost first
        t.ggml_type = r.le<uint32_t>();
        if (type_params(t.ggml_type) == nullptr)
            throw ParseFailure{"unsupported GGML type: " + std::to_string(t.ggml_type)};
        t.offset = r.le<uint64_t>();
        if (t.offset % g.alignment != 0)
            parse_error(r.pos() - 8, "tensor '" + t.name + "' offset " + std::to_string(t.offset) +
                                         " is not aligned to " + std::to_string(g.alignment) + " bytes");
        g.tensors.push_back(std::move(t));
    }
    const uint64_t padding = (g.alignment - r.pos() % g.alignment) % g.alignment;
    g.data_start = r.pos() + padding;
    if (tensor_count > 0 && g.data_start > g.len)
        parse_error(r.pos(), "tensor data starts at " + std::to_string(g.data_start) + ", beyond file length " +
                                 std::to_string(g.len));
    for (Tensor &t : g.tensors) {  // sizes and absolute offsets where they are representable; checked by map_tensors
        std::string why;
        if (tensor_size(t.shape, t.n_dims, t.ggml_type, &t.n_bytes, &why) &&
            t.offset <= std::numeric_limits<uint64_t>::max() - g.data_start)
            t.file_offset = g.data_start + t.offset;
        else
            t.n_bytes = 0;
    }
}

// crates/rnb-loader/src/convert.rs:124-158: every tensor's shape is block-aligned and its bytes lie inside the file
void map_tensors(const rnb_hip_gguf &handle) {
    for (const Tensor &t : handle.tensors) {
        const rnb_hip_gguf &g = t.home != nullptr ? *t.home : handle;  // a split model: the tensor's own shard
        std::string why;
        uint64_t n_bytes = 0;
        if (!tensor_size(t.shape, t.n_dims, t.ggml_type, &n_bytes, &why))
            parse_error(static_cast<size_t>(g.data_start), "tensor '" + t.name + "' has invalid shape: " + why);
        if (t.offset > std::numeric_limits<uint64_t>::max() - g.data_start)
            parse_error(static_cast<size_t>(g.data_start), "tensor '" + t.name + "' absolute offset overflows usize");
        const uint64_t file_offset = g.data_start + t.offset;
        if (n_bytes > std::numeric_limits<uint64_t>::max() - file_offset)
            parse_error(static_cast<size_t>(file_offset), "tensor '" + t.name + "' data end overflows usize");
        if (file_offset + n_bytes > g.len)
            parse_error(static_cast<size_t>(file_offset), "tensor '" + t.name + "' ends at " +
                                                              std::to_string(file_offset + n_bytes) +
                                                              ", beyond file length " + std::to_string(g.len));
    }
}

bool tensor_in_bounds(const rnb_hip_gguf *g, const Tensor &t) {
    if (t.home != nullptr) g = t.home;
    std::string why;
    uint64_t n = 0;
    return tensor_size(t.shape, t.n_dims, t.ggml_type, &n, &why) && t.offset <= g->len && g->data_start <= g->len &&
           g->data_start + t.offset <= g->len && n <= g->len - (g->data_start + t.offset);
}

int finish_open(std::unique_ptr<rnb_hip_gguf> g, rnb_hip_gguf **out, bool map) {
    try {
        parse_into(*g);
        if (map) map_tensors(*g);
    } catch (const ParseFailure &f) {
        return fail_gguf(RNB_HIP_INVALID_REQUEST, f.text);
    } catch (const std::bad_alloc &) {
        return fail_gguf(RNB_HIP_EXECUTION_FAILED, "out of host memory while parsing GGUF header");
    }
    *out = g.release();
    return RNB_HIP_OK;
}

void fill_tensor(const rnb_hip_gguf *g, const Tensor &t, rnb_hip_gguf_tensor *out) {
    out->name = t.name.c_str();
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; d++) out->shape[d] = t.shape[d];
    out->ggml_type = t.ggml_type;
    out->offset = t.offset;
    out->file_offset = t.file_offset;
    out->n_bytes = t.n_bytes;
    out->data = tensor_in_bounds(g, t) ? (t.home != nullptr ? t.home : g)->data + t.file_offset : nullptr;
}

const Value *find_value(const rnb_hip_gguf *g, const char *key) {
    if (g == nullptr || key == nullptr) return nullptr;
    for (const auto &kv : g->metadata)
        if (kv.first == key) return &kv.second;
    return nullptr;
}

bool is_signed_type(uint32_t t) { return t == 1 || t == 3 || t == 5 || t == 11; }
bool is_integer_type(uint32_t t) { return t <= 5 || t == 10 || t == 11; }

// mmap + parse + map_tensors of one file
int open_one(const char *path, std::unique_ptr<rnb_hip_gguf> *out) {
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return fail_gguf(RNB_HIP_EXECUTION_FAILED, std::string("I/O error: ") + strerror(errno) + ": " + path);
    struct stat st;
    if (fstat(fd, &st) != 0) {
        const std::string msg = std::string("I/O error: ") + strerror(errno) + ": " + path;
        close(fd);
        return fail_gguf(RNB_HIP_EXECUTION_FAILED, msg);
    }
    auto g = std::make_unique<rnb_hip_gguf>();
    g->len = static_cast<size_t>(st.st_size);
    if (g->len > 0) {
        void *p = mmap(nullptr, g->len, PROT_READ, MAP_PRIVATE, fd, 0);
        if (p == MAP_FAILED) {
            const std::string msg = std::string("I/O error: mmap: ") + strerror(errno) + ": " + path;
            close(fd);
            return fail_gguf(RNB_HIP_EXECUTION_FAILED, msg);
        }
        g->data = static_cast<const uint8_t *>(p);
        g->owns_mapping = true;
    }
    close(fd);
    rnb_hip_gguf *raw = nullptr;
    if (int rc = finish_open(std::move(g), &raw, true); rc != RNB_HIP_OK) return rc;
    out->reset(raw);
    return RNB_HIP_OK;
}

// ---- split files: crates/rnb-loader/src/gguf/sharded.rs:22-235 (load_mapped_gguf), same checks, same texts ---------
[[noreturn]] void split_error(const std::string &msg) { parse_error(0, "invalid split GGUF: " + msg); }

// split_value, sharded.rs:153-178: absent -> false; any non-negative integer type
bool split_value(const rnb_hip_gguf &g, const char *key, uint64_t *out) {
    const Value *v = find_value(&g, key);
    if (v == nullptr) return false;
    const bool integer = v->type <= 5 || v->type == 10 || v->type == 11;  // u8 i8 u16 i16 u32 i32, u64 i64
    if (!integer || (is_signed_type(v->type) && static_cast<int64_t>(v->u) < 0))
        split_error(std::string("metadata key ") + key + " must be a non-negative integer");
    *out = v->u;
    return true;
}
uint64_t required_split_value(const rnb_hip_gguf &g, const char *key) {
    uint64_t v = 0;
    if (!split_value(g, key, &v)) split_error(std::string("missing metadata key ") + key);
    return v;
}

bool all_digits(const std::string &s) {
    return !s.empty() && std::all_of(s.begin(), s.end(), [](unsigned char c) { return c >= '0' && c <= '9'; });
}

// The shard files' names, made one at a time: a header may declare any 64-bit shard count, and a list of that many
// names would be allocated before the first missing file refuses the set.
struct ShardPaths {
    std::string parent, prefix, ext;
    size_t index_width, count_width;
    uint64_t split_count;
    std::string of(uint64_t no) const {  // shard `no`, counted from zero
        auto padded = [](uint64_t v, size_t width) {
            std::string t = std::to_string(v);
            return t.size() < width ? std::string(width - t.size(), '0') + t : t;
        };
        return parent + prefix + "-" + padded(no + 1, index_width) + "-of-" + padded(split_count, count_width) + ext;
    }
};

// resolve_shard_paths, sharded.rs:180-235: `<prefix>-<index>-of-<count>.gguf` beside the selected file, same digit widths
ShardPaths resolve_shard_paths(const std::string &selected, uint64_t selected_no, uint64_t split_count) {
    const size_t slash = selected.find_last_of('/');
    const std::string parent = slash == std::string::npos ? "" : selected.substr(0, slash + 1);
    const std::string file_name = slash == std::string::npos ? selected : selected.substr(slash + 1);
    const std::string ext = ".gguf";
    if (file_name.size() < ext.size() || file_name.compare(file_name.size() - ext.size(), ext.size(), ext) != 0)
        split_error("split GGUF file name must end in .gguf");
    const std::string stem = file_name.substr(0, file_name.size() - ext.size());
    const size_t of = stem.rfind("-of-");
    if (of == std::string::npos) split_error("split GGUF file name must end in -00001-of-00001.gguf");
    const std::string indexed_stem = stem.substr(0, of), file_count = stem.substr(of + 4);
    const size_t dash = indexed_stem.rfind('-');
    if (dash == std::string::npos) split_error("split GGUF file name is missing its shard index");
    const std::string prefix = indexed_stem.substr(0, dash), file_index = indexed_stem.substr(dash + 1);
    if (prefix.empty() || !all_digits(file_index) || !all_digits(file_count))
        split_error("split GGUF file name has an invalid shard suffix");
    errno = 0;
    const unsigned long long parsed_index = std::strtoull(file_index.c_str(), nullptr, 10);
    if (errno == ERANGE) split_error("split GGUF shard index is too large");
    const unsigned long long parsed_count = std::strtoull(file_count.c_str(), nullptr, 10);
    if (errno == ERANGE) split_error("split GGUF shard count is too large");
    if (parsed_index != selected_no + 1 || parsed_count != split_count)
        split_error("file name declares shard " + std::to_string(parsed_index) + " of " + std::to_string(parsed_count) +
                    ", metadata declares shard " + std::to_string(selected_no + 1) + " of " + std::to_string(split_count));
    return ShardPaths{parent, prefix, ext, file_index.size(), file_count.size(), split_count};
}

// The file that was opened declares split.count > 1: every shard is mapped and checked, `g` becomes shard zero with the
// union of the tensor tables (a tensor keeps pointing into its own shard's mapping).
void assemble_split(const char *path, std::unique_ptr<rnb_hip_gguf> &g) {
    uint64_t split_count = 1;
    if (split_value(*g, "split.count", &split_count) && split_count == 0) split_error("split.count must be positive");
    if (split_count == 1) return;
    const uint64_t selected_no = required_split_value(*g, "split.no");
    if (selected_no >= split_count)
        split_error("split.no " + std::to_string(selected_no) + " is outside split.count " + std::to_string(split_count));
    const uint64_t expected_tensors = required_split_value(*g, "split.tensors.count");
    const ShardPaths paths = resolve_shard_paths(path, selected_no, split_count);
    std::vector<std::unique_ptr<rnb_hip_gguf>> shards;  // grows with the shards that open: a wrong count ends at the first missing file
    for (uint64_t no = 0; no < split_count; no++) {
        shards.emplace_back();
        if (no == selected_no) {
            shards[no] = std::move(g);
        } else if (const std::string shard_path = paths.of(no); open_one(shard_path.c_str(), &shards[no]) != RNB_HIP_OK) {
            split_error("failed to load shard '" + shard_path + "': " + last_error_cstr());
        }
        // validate_shard, sharded.rs:113-138
        const rnb_hip_gguf &sh = *shards[no];
        const uint64_t shard_no = required_split_value(sh, "split.no"), shard_count = required_split_value(sh, "split.count"),
                       shard_tensors = required_split_value(sh, "split.tensors.count");
        if (shard_no != no)
            split_error("expected shard " + std::to_string(no) + ", but its metadata declares split.no " + std::to_string(shard_no));
        if (shard_count != split_count)
            split_error("shard " + std::to_string(shard_no) + " declares split.count " + std::to_string(shard_count) +
                        ", expected " + std::to_string(split_count));
        if (shard_tensors != expected_tensors)
            split_error("shard " + std::to_string(shard_no) + " declares split.tensors.count " + std::to_string(shard_tensors) +
                        ", expected " + std::to_string(expected_tensors));
    }
    // shard zero carries the metadata and becomes the handle; the tensors of all shards, in shard order
    std::unique_ptr<rnb_hip_gguf> head = std::move(shards[0]);
    std::vector<Tensor> all;
    std::set<std::string> names;
    auto take = [&](rnb_hip_gguf *from, const rnb_hip_gguf *home) {
        for (Tensor &t : from->tensors) {
            if (!names.insert(t.name).second) split_error("tensor '" + t.name + "' appears in more than one shard");
            t.home = home;
            all.push_back(std::move(t));
        }
        from->tensors.clear();
    };
    take(head.get(), nullptr);
    for (uint64_t no = 1; no < split_count; no++) take(shards[no].get(), shards[no].get());
    if (all.size() != expected_tensors)
        split_error("split.tensors.count declares " + std::to_string(expected_tensors) + " tensors but " +
                    std::to_string(all.size()) + " were loaded");
    head->tensors = std::move(all);
    for (uint64_t no = 1; no < split_count; no++) head->shards.push_back(std::move(shards[no]));
    g = std::move(head);
}

}  // namespace

}  // namespace rnb

using namespace rnb;

extern "C" {

int rnb_hip_gguf_open(const char *path, rnb_hip_gguf **out) {
    if (path == nullptr || out == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, "null argument");
    *out = nullptr;
    std::unique_ptr<rnb_hip_gguf> g;
    if (int st = open_one(path, &g); st != RNB_HIP_OK) return st;
    try {
        assemble_split(path, g);
    } catch (const ParseFailure &f) {
        return fail_gguf(RNB_HIP_INVALID_REQUEST, f.text);
    } catch (const std::bad_alloc &) {
        return fail_gguf(RNB_HIP_EXECUTION_FAILED, "out of host memory while parsing GGUF header");
    }
    *out = g.release();
    return RNB_HIP_OK;
}

int rnb_hip_gguf_parse(const uint8_t *data, size_t len, rnb_hip_gguf **out) {
    if (out == nullptr || (data == nullptr && len != 0)) return fail_gguf(RNB_HIP_INVALID_REQUEST, "null argument");
    *out = nullptr;
    auto g = std::make_unique<rnb_hip_gguf>();
    g->data = data;
    g->len = len;
    return finish_open(std::move(g), out, false);
}

int rnb_hip_gguf_map_tensors(const rnb_hip_gguf *g) {
    if (g == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, "null argument");
    try {
        map_tensors(*g);
    } catch (const ParseFailure &f) {
        return fail_gguf(RNB_HIP_INVALID_REQUEST, f.text);
    }
    return RNB_HIP_OK;
}

void rnb_hip_gguf_close(rnb_hip_gguf *g) { delete g; }

uint32_t rnb_hip_gguf_version(const rnb_hip_gguf *g) { return g ? g->version : 0; }
uint64_t rnb_hip_gguf_alignment(const rnb_hip_gguf *g) { return g ? g->alignment : 0; }
uint64_t rnb_hip_gguf_data_start(const rnb_hip_gguf *g) { return g ? g->data_start : 0; }
size_t rnb_hip_gguf_tensor_count(const rnb_hip_gguf *g) { return g ? g->tensors.size() : 0; }

int rnb_hip_gguf_tensor_at(const rnb_hip_gguf *g, size_t index, rnb_hip_gguf_tensor *out) {
    if (g == nullptr || out == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, "null argument");
    if (index >= g->tensors.size())
        return fail_gguf(RNB_HIP_INVALID_REQUEST, "tensor index " + std::to_string(index) + " out of range (" +
                                                      std::to_string(g->tensors.size()) + " tensors)");
    fill_tensor(g, g->tensors[index], out);
    return RNB_HIP_OK;
}

int rnb_hip_gguf_find_tensor(const rnb_hip_gguf *g, const char *name, rnb_hip_gguf_tensor *out) {
    if (g == nullptr || name == nullptr || out == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, "null argument");
    for (const Tensor &t : g->tensors)
        if (t.name == name) {
            fill_tensor(g, t, out);
            return RNB_HIP_OK;
        }
    return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("missing tensor: ") + name);
}

int rnb_hip_gguf_tensor_size(const uint64_t *shape, uint32_t n_dims, uint32_t ggml_type, uint64_t *bytes) {
    if (bytes == nullptr || (shape == nullptr && n_dims != 0) || n_dims > 4)
        return fail_gguf(RNB_HIP_INVALID_REQUEST, "bad shape argument");
    std::string why;
    if (!tensor_size(shape, n_dims, ggml_type, bytes, &why)) return fail_gguf(RNB_HIP_INVALID_REQUEST, why);
    return RNB_HIP_OK;
}

size_t rnb_hip_gguf_metadata_count(const rnb_hip_gguf *g) { return g ? g->metadata.size() : 0; }

const char *rnb_hip_gguf_metadata_key(const rnb_hip_gguf *g, size_t index) {
    return (g && index < g->metadata.size()) ? g->metadata[index].first.c_str() : nullptr;
}

int rnb_hip_gguf_metadata_type(const rnb_hip_gguf *g, const char *key) {
    const Value *v = find_value(g, key);
    return v ? static_cast<int>(v->type) : -1;
}

// crates/rnb-loader/src/error.rs:18-22 texts for absent keys and wrong types
int rnb_hip_gguf_metadata_u64(const rnb_hip_gguf *g, const char *key, uint64_t *out) {
    const Value *v = find_value(g, key);
    if (v == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("missing metadata key: ") + (key ? key : ""));
    if (out == nullptr || !(is_integer_type(v->type) || v->type == 7) ||
        (is_signed_type(v->type) && static_cast<int64_t>(v->u) < 0))
        return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("type mismatch for key '") + key + "': expected unsigned integer");
    *out = v->u;
    return RNB_HIP_OK;
}

int rnb_hip_gguf_metadata_i64(const rnb_hip_gguf *g, const char *key, int64_t *out) {
    const Value *v = find_value(g, key);
    if (v == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("missing metadata key: ") + (key ? key : ""));
    if (out == nullptr || !is_integer_type(v->type) ||
        (!is_signed_type(v->type) && v->u > static_cast<uint64_t>(std::numeric_limits<int64_t>::max())))
        return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("type mismatch for key '") + key + "': expected integer");
    *out = static_cast<int64_t>(v->u);
    return RNB_HIP_OK;
}

int rnb_hip_gguf_metadata_f64(const rnb_hip_gguf *g, const char *key, double *out) {
    const Value *v = find_value(g, key);
    if (v == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("missing metadata key: ") + (key ? key : ""));
    if (out == nullptr || !(v->type == 6 || v->type == 12))
        return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("type mismatch for key '") + key + "': expected float");
    *out = v->f;
    return RNB_HIP_OK;
}

const char *rnb_hip_gguf_metadata_str(const rnb_hip_gguf *g, const char *key) {
    const Value *v = find_value(g, key);
    return (v && v->type == 8) ? v->s.c_str() : nullptr;
}

int rnb_hip_gguf_metadata_array(const rnb_hip_gguf *g, const char *key, uint32_t *elem_type, uint64_t *count) {
    const Value *v = find_value(g, key);
    if (v == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("missing metadata key: ") + (key ? key : ""));
    if (v->type != 9)
        return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("type mismatch for key '") + key + "': expected array");
    if (elem_type) *elem_type = v->elem_type;
    if (count) *count = v->count;
    return RNB_HIP_OK;
}

const char *rnb_hip_gguf_metadata_array_str(const rnb_hip_gguf *g, const char *key, uint64_t index) {
    const Value *v = find_value(g, key);
    return (v && v->type == 9 && v->elem_type == 8 && index < v->strings.size()) ? v->strings[index].c_str() : nullptr;
}

int rnb_hip_gguf_metadata_array_f64(const rnb_hip_gguf *g, const char *key, uint64_t index, double *out) {
    const Value *v = find_value(g, key);
    if (v == nullptr || out == nullptr || v->type != 9 || index >= v->numbers.size())
        return fail_gguf(RNB_HIP_INVALID_REQUEST, std::string("no numeric array element ") + std::to_string(index) +
                                                      " under key '" + (key ? key : "") + "'");
    *out = v->numbers[index];
    return RNB_HIP_OK;
}

// Upload of one tensor's bytes exactly as stored (no requantisation, no repack) into the resident table, pinned:
// later operator calls that pass `data` (or a sub-range, e.g. one expert of a stacked tensor) find it on the device.
int rnb_hip_gguf_prewarm_tensor(const rnb_hip_gguf *g, size_t index) {
    if (g == nullptr) return fail_gguf(RNB_HIP_INVALID_REQUEST, "null argument");
    if (index >= g->tensors.size())
        return fail_gguf(RNB_HIP_INVALID_REQUEST, "tensor index " + std::to_string(index) + " out of range (" +
                                                      std::to_string(g->tensors.size()) + " tensors)");
    const Tensor &t = g->tensors[index];
    if (!tensor_in_bounds(g, t))
        return fail_gguf(RNB_HIP_INVALID_REQUEST, "tensor '" + t.name + "' does not lie inside the file");
    const uint8_t *ptr = (t.home != nullptr ? t.home : g)->data + t.file_offset;  // a split model: the tensor's own shard
    const size_t len = static_cast<size_t>(t.n_bytes);
    return rnb_hip_prewarm(&ptr, &len, 1);
}

}  // extern "C"
