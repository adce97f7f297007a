// Mutation fuzzer for the GGUF reader of include/rnb_hip.h, meant to be built with the address and
// undefined-behaviour sanitizers on the host side (see __graft_entry__.build): a valid file image is damaged in
// a few places per round (bit flips, extreme values over length and count fields, truncation) and every
// accessor is exercised on whatever the parser accepts.  The process must end normally: the sanitizers turn
// any out-of-bounds read, overflow or leak in the parser into a non-zero exit.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/rnb_hip.h"

namespace {

struct Rng {
    uint64_t s;
    uint64_t next() {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        return s;
    }
    uint64_t below(uint64_t n) { return n ? next() % n : 0; }
};

struct Image {
    std::vector<uint8_t> b;
    template <typename T>
    void num(T v) {
        const size_t at = b.size();
        b.resize(at + sizeof(T));
        std::memcpy(b.data() + at, &v, sizeof(T));
    }
    void str(const std::string &s) {
        num<uint64_t>(s.size());
        b.insert(b.end(), s.begin(), s.end());
    }
};

// a version-3 file with one value of every metadata type, nested string and number arrays and three tensors
std::vector<uint8_t> valid_image() {
    Image im;
    im.num<uint32_t>(0x46554747u);  // "GGUF"
    im.num<uint32_t>(3);
    im.num<uint64_t>(3);   // tensors
    im.num<uint64_t>(16);  // key/value pairs
    im.str("general.architecture"); im.num<uint32_t>(8); im.str("llama");
    im.str("general.alignment"); im.num<uint32_t>(4); im.num<uint32_t>(32);
    im.str("t.u8"); im.num<uint32_t>(0); im.num<uint8_t>(200);
    im.str("t.i8"); im.num<uint32_t>(1); im.num<int8_t>(-7);
    im.str("t.u16"); im.num<uint32_t>(2); im.num<uint16_t>(60000);
    im.str("t.i16"); im.num<uint32_t>(3); im.num<int16_t>(-30000);
    im.str("t.i32"); im.num<uint32_t>(5); im.num<int32_t>(-5);
    im.str("t.f32"); im.num<uint32_t>(6); im.num<float>(1.5f);
    im.str("t.bool"); im.num<uint32_t>(7); im.num<uint8_t>(1);
    im.str("t.u64"); im.num<uint32_t>(10); im.num<uint64_t>(1ull << 40);
    im.str("t.i64"); im.num<uint32_t>(11); im.num<int64_t>(-(1ll << 40));
    im.str("t.f64"); im.num<uint32_t>(12); im.num<double>(2.25);
    im.str("tokenizer.ggml.tokens"); im.num<uint32_t>(9); im.num<uint32_t>(8); im.num<uint64_t>(3);
    im.str("a"); im.str("bc"); im.str("");
    im.str("tokenizer.ggml.scores"); im.num<uint32_t>(9); im.num<uint32_t>(6); im.num<uint64_t>(4);
    for (int i = 0; i < 4; i++) im.num<float>(0.5f * static_cast<float>(i));
    im.str("t.arr_i32"); im.num<uint32_t>(9); im.num<uint32_t>(5); im.num<uint64_t>(2);
    im.num<int32_t>(1); im.num<int32_t>(-1);
    im.str("t.arr_u8"); im.num<uint32_t>(9); im.num<uint32_t>(0); im.num<uint64_t>(5);
    for (int i = 0; i < 5; i++) im.num<uint8_t>(static_cast<uint8_t>(i));
    // tensor infos: name, n_dims, dims innermost first, type, offset
    im.str("blk.0.ffn_up.weight"); im.num<uint32_t>(2); im.num<uint64_t>(256); im.num<uint64_t>(4); im.num<uint32_t>(12); im.num<uint64_t>(0);
    im.str("output.weight"); im.num<uint32_t>(2); im.num<uint64_t>(256); im.num<uint64_t>(2); im.num<uint32_t>(14); im.num<uint64_t>(576);
    im.str("norm.weight"); im.num<uint32_t>(1); im.num<uint64_t>(8); im.num<uint32_t>(0); im.num<uint64_t>(1024);
    while (im.b.size() % 32) im.b.push_back(0);
    im.b.resize(im.b.size() + 1024 + 32, 0x5a);
    return im.b;
}

int failures = 0;

void exercise(rnb_hip_gguf *g) {
    volatile uint64_t sink = 0;
    sink += rnb_hip_gguf_version(g) + rnb_hip_gguf_alignment(g) + rnb_hip_gguf_data_start(g);
    const size_t nt = rnb_hip_gguf_tensor_count(g);
    const int mapped = rnb_hip_gguf_map_tensors(g);
    for (size_t i = 0; i < nt + 1; i++) {
        rnb_hip_gguf_tensor t;
        if (rnb_hip_gguf_tensor_at(g, i, &t) != RNB_HIP_OK) continue;
        sink += std::strlen(t.name) + t.n_bytes + t.file_offset;
        for (uint32_t d = 0; d < t.n_dims && d < 4; d++) sink += t.shape[d];
        if (t.data && t.n_bytes) sink += t.data[0] + t.data[t.n_bytes - 1];  // in bounds by contract
        // a damaged name may hold a NUL byte, which a C string cannot carry; an intact name must be found
        const bool intact = !std::strcmp(t.name, "blk.0.ffn_up.weight") || !std::strcmp(t.name, "output.weight") ||
                            !std::strcmp(t.name, "norm.weight");
        rnb_hip_gguf_tensor again;
        if (rnb_hip_gguf_find_tensor(g, t.name, &again) != RNB_HIP_OK && intact) {
            failures++;
            if (failures < 5) std::printf("find_tensor(\"%s\") failed for tensor %zu: %s\n", t.name, i, rnb_hip_last_error());
        }
        uint64_t bytes = 0;
        (void)rnb_hip_gguf_tensor_size(t.shape, t.n_dims, t.ggml_type, &bytes);
    }
    (void)mapped;
    const size_t nm = rnb_hip_gguf_metadata_count(g);
    for (size_t i = 0; i < nm + 1; i++) {
        const char *key = rnb_hip_gguf_metadata_key(g, i);
        if (!key) continue;
        const int type = rnb_hip_gguf_metadata_type(g, key);
        uint64_t u = 0;
        int64_t s = 0;
        double f = 0;
        (void)rnb_hip_gguf_metadata_u64(g, key, &u);
        (void)rnb_hip_gguf_metadata_i64(g, key, &s);
        (void)rnb_hip_gguf_metadata_f64(g, key, &f);
        const char *str = rnb_hip_gguf_metadata_str(g, key);
        if (str) sink += std::strlen(str);
        uint32_t et = 0;
        uint64_t n = 0;
        if (type == 9 && rnb_hip_gguf_metadata_array(g, key, &et, &n) == RNB_HIP_OK) {
            for (uint64_t k = 0; k < n + 1 && k < 64; k++) {
                const char *e = rnb_hip_gguf_metadata_array_str(g, key, k);
                if (e) sink += std::strlen(e);
                (void)rnb_hip_gguf_metadata_array_f64(g, key, k, &f);
            }
        }
    }
    (void)rnb_hip_gguf_metadata_type(g, "no.such.key");
    (void)sink;
}

// ---- split models: rnb_hip_gguf_open on shard files (crates/rnb-loader/src/gguf/sharded.rs) -------------------------
// shard `no` of `count`: the three split keys as the given types/values, `n_tensors` F32 tensors of one element
std::vector<uint8_t> shard_image(uint64_t no, uint64_t count, uint64_t total, uint32_t key_type, int n_tensors, int name_base,
                                 bool with_no, bool with_total) {
    Image im;
    im.num<uint32_t>(0x46554747u);
    im.num<uint32_t>(3);
    im.num<uint64_t>(static_cast<uint64_t>(n_tensors));
    im.num<uint64_t>(2 + (with_no ? 1 : 0) + (with_total ? 1 : 0));
    im.str("general.architecture"); im.num<uint32_t>(8); im.str("llama");
    auto integer = [&](const char *key, uint64_t v) {
        im.str(key);
        im.num<uint32_t>(key_type);
        switch (key_type) {
        case 0: case 1: im.num<uint8_t>(static_cast<uint8_t>(v)); break;
        case 2: case 3: im.num<uint16_t>(static_cast<uint16_t>(v)); break;
        case 4: case 5: im.num<uint32_t>(static_cast<uint32_t>(v)); break;
        case 6: im.num<float>(static_cast<float>(v)); break;
        case 8: im.str(std::to_string(v)); break;
        default: im.num<uint64_t>(v); break;  // 10, 11
        }
    };
    if (with_no) integer("split.no", no);
    integer("split.count", count);
    if (with_total) integer("split.tensors.count", total);
    for (int t = 0; t < n_tensors; t++) {
        im.str("t" + std::to_string(name_base + t) + ".weight");
        im.num<uint32_t>(1); im.num<uint64_t>(1); im.num<uint32_t>(0); im.num<uint64_t>(32u * static_cast<uint64_t>(t));
    }
    while (im.b.size() % 32) im.b.push_back(0);
    for (int t = 0; t < n_tensors; t++) {
        const float v = static_cast<float>(name_base + t) + 0.25f;
        const size_t at = im.b.size();
        im.b.resize(at + 32, 0);
        std::memcpy(im.b.data() + at, &v, 4);
    }
    return im.b;
}

bool write_file(const std::string &path, const std::vector<uint8_t> &b) {
    FILE *f = std::fopen(path.c_str(), "wb");
    if (!f) return false;
    const bool ok = b.empty() || std::fwrite(b.data(), 1, b.size(), f) == b.size();
    std::fclose(f);
    return ok;
}

// Rounds of two to four shard files in `dir`, most of them consistent, some damaged in one place (a key's type or value,
// a missing key, a duplicate tensor name, a wrong total, a truncated or missing shard, a file name off the pattern);
// every shard path is opened.  A consistent set must open from every shard with all tensors, each carrying its own
// value; a damaged one must be refused with a message (or, where the damage is invisible from the selected shard,
// opened); the sanitizers watch the rest.
int split_rounds(const char *dir, long rounds, Rng &rng) {
    int bad = 0;
    long opened = 0, refused = 0;
    const uint32_t int_types[] = {0, 1, 2, 3, 4, 5, 10, 11};
    for (long r = 0; r < rounds; r++) {
        const uint64_t count = 2 + rng.below(3);
        const int damage = static_cast<int>(rng.below(12));  // 0..4: none
        const uint64_t victim = rng.below(count);
        std::vector<std::string> paths;
        uint64_t total = 0;
        std::vector<int> per(count);
        for (uint64_t i = 0; i < count; i++) total += static_cast<uint64_t>(per[i] = 1 + static_cast<int>(rng.below(3)));
        int base = 0;
        char name[96];
        for (uint64_t i = 0; i < count; i++) {
            uint32_t type = int_types[rng.below(8)];
            uint64_t no = i, cnt = count, tot = total;
            bool with_no = true, with_total = true;
            int nb = base;
            if (i == victim) {
                switch (damage) {
                case 5: type = 6; break;            // a float where an integer belongs
                case 6: type = 8; break;            // a string
                case 7: no = count + rng.below(3); break;
                case 8: cnt = rng.below(2) ? 0 : count + 1; break;
                case 9: tot = total + 1 + rng.below(2); break;
                case 10: with_no = false; break;
                case 11: nb = 0; break;             // names of shard zero again (no damage when the victim is shard zero)
                default: break;
                }
            }
            std::vector<uint8_t> img = shard_image(no, cnt, tot, type, per[i], nb, with_no, with_total);
            if (i == victim && damage == 4 && rng.below(2)) img.resize(rng.below(img.size()));  // truncated shard
            std::snprintf(name, sizeof name, "%s/f%ld-%05llu-of-%05llu.gguf", dir, r, static_cast<unsigned long long>(i + 1),
                          static_cast<unsigned long long>(count));
            paths.push_back(name);
            if (!write_file(name, img)) {
                std::printf("split rounds: cannot write %s\n", name);
                return 1;
            }
            base += per[i];
        }
        const bool consistent = damage < 4;
        for (uint64_t i = 0; i < count; i++) {
            rnb_hip_gguf *h = nullptr;
            const int rc = rnb_hip_gguf_open(paths[i].c_str(), &h);
            if (rc == RNB_HIP_OK && h) {
                opened++;
                exercise(h);
                if (consistent) {
                    if (rnb_hip_gguf_tensor_count(h) != total) bad++;
                    for (size_t t = 0; t < rnb_hip_gguf_tensor_count(h); t++) {
                        rnb_hip_gguf_tensor ti;
                        float v = 0.0f;
                        if (rnb_hip_gguf_tensor_at(h, t, &ti) != RNB_HIP_OK || !ti.data || ti.n_bytes != 4) { bad++; continue; }
                        std::memcpy(&v, ti.data, 4);
                        if (v != static_cast<float>(t) + 0.25f || ti.name != "t" + std::to_string(t) + ".weight") bad++;
                    }
                }
                rnb_hip_gguf_close(h);
            } else {
                refused++;
                if (consistent || std::strlen(rnb_hip_last_error()) == 0) {
                    bad++;
                    if (bad < 5) std::printf("split round %ld shard %llu: %s\n", r, static_cast<unsigned long long>(i), rnb_hip_last_error());
                }
            }
        }
        for (const std::string &p : paths) std::remove(p.c_str());
    }
    std::printf("gguf_fuzz split files: %ld rounds, %ld opened, %ld refused, %d failure(s)\n", rounds, opened, refused, bad);
    return bad;
}

}  // namespace

int main(int argc, char **argv) {
    const long rounds = argc > 1 ? std::atol(argv[1]) : 20000;
    const std::vector<uint8_t> good = valid_image();
    rnb_hip_gguf *g = nullptr;
    if (rnb_hip_gguf_parse(good.data(), good.size(), &g) != RNB_HIP_OK) {
        std::printf("FAIL: the unmodified image is rejected: %s\n", rnb_hip_last_error());
        return 1;
    }
    if (rnb_hip_gguf_tensor_count(g) != 3 || rnb_hip_gguf_metadata_count(g) != 16 ||
        rnb_hip_gguf_map_tensors(g) != RNB_HIP_OK) {
        std::printf("FAIL: the unmodified image is misread: %s\n", rnb_hip_last_error());
        return 1;
    }
    exercise(g);
    rnb_hip_gguf_close(g);

    const uint64_t extremes[] = {0, 1, 2, 0x7f, 0x80, 0xff, 0x7fffffffull, 0x80000000ull, 0xffffffffull,
                                 0x7fffffffffffffffull, 0x8000000000000000ull, 0xffffffffffffffffull,
                                 good.size(), good.size() - 1, good.size() + 1};
    Rng rng{0x9e3779b97f4a7c15ull};
    long accepted = 0, rejected = 0;
    // each round owns a heap copy of exactly the (possibly truncated) length, so reads past it are caught
    for (long r = 0; r < rounds; r++) {
        size_t len = good.size();
        if (rng.below(4) == 0) len = rng.below(good.size() + 1);
        const size_t header = len < 900 ? len : 900;  // most mutations land in the structured part
        uint8_t *buf = static_cast<uint8_t *>(std::malloc(len ? len : 1));
        std::memcpy(buf, good.data(), len);
        const int edits = static_cast<int>(rng.below(4));
        for (int e = 0; e < edits && len > 0; e++) {
            const size_t at = rng.below(rng.below(3) ? header : len);
            switch (rng.below(4)) {
            case 0: buf[at] ^= static_cast<uint8_t>(1u << rng.below(8)); break;
            case 1: buf[at] = static_cast<uint8_t>(rng.next()); break;
            case 2: {
                const uint32_t v = static_cast<uint32_t>(extremes[rng.below(sizeof(extremes) / sizeof(extremes[0]))]);
                if (at + 4 <= len) std::memcpy(buf + at, &v, 4);
                break;
            }
            default: {
                const uint64_t v = extremes[rng.below(sizeof(extremes) / sizeof(extremes[0]))];
                if (at + 8 <= len) std::memcpy(buf + at, &v, 8);
                break;
            }
            }
        }
        rnb_hip_gguf *h = nullptr;
        if (rnb_hip_gguf_parse(buf, len, &h) == RNB_HIP_OK && h) {
            accepted++;
            exercise(h);
            rnb_hip_gguf_close(h);
        } else {
            rejected++;
            if (std::strlen(rnb_hip_last_error()) == 0) {  // every rejection carries a message
                failures++;
                if (failures < 5) std::printf("round %ld: rejection without a message\n", r);
            }
        }
        std::free(buf);
    }
    std::printf("gguf_fuzz: %ld rounds, %ld accepted, %ld rejected, %d failure(s)\n", rounds, accepted, rejected, failures);
    if (argc > 2) failures += split_rounds(argv[2], rounds / 40 + 20, rng);
    return failures ? 1 : 0;
}
