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
    return failures ? 1 : 0;
}
