// Exercises include/rnb_backend_hip.hpp (the C++ mirror of the reference's operator functions) against
// librnb_hip.so.  Modes:
//   host_mirror_test validate            no GPU needed: error messages, capability facade
//   host_mirror_test run <golden_dir>    GPU: q4k/q6k/q8_0 gemv + batch on the committed raw fixtures
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <string>
#include <vector>

#include "../../include/rnb_backend_hip.hpp"

using namespace rnb_hip;

static int failures = 0;
#define EXPECT(cond, what)                                    \
    do {                                                      \
        if (!(cond)) {                                        \
            std::printf("FAIL: %s (%s)\n", what, #cond);      \
            failures++;                                       \
        }                                                     \
    } while (0)

template <typename T>
static std::vector<T> read_file(const std::string &path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) {
        std::printf("FAIL: cannot open %s\n", path.c_str());
        failures++;
        return {};
    }
    const size_t n = static_cast<size_t>(f.tellg());
    std::vector<T> v(n / sizeof(T));
    f.seekg(0);
    f.read(reinterpret_cast<char *>(v.data()), static_cast<std::streamsize>(v.size() * sizeof(T)));
    return v;
}

static int validate() {
    std::vector<uint8_t> w(144, 0);
    std::vector<float> x(256, 0.0f);
    auto r = q4k_gemv({w.data(), w.size()}, 1, 255, {x.data(), 255});
    EXPECT(!r && r.status == RNB_HIP_INVALID_REQUEST && r.error == "Q4_K cols must be divisible by 256, got 255", "cols message");
    r = q4k_gemv({w.data(), 143}, 1, 256, {x.data(), 256});
    EXPECT(!r && r.error == "Q4_K weight byte mismatch: got 143, expected 144", "weight bytes message");
    r = q6k_gemv({w.data(), 144}, 1, 256, {x.data(), 256});
    EXPECT(!r && r.error == "Q6_K weight byte mismatch: got 144, expected 210", "q6k weight bytes message");
    r = q5k_gemv({w.data(), 144}, 1, 256, {x.data(), 256});
    EXPECT(!r && r.error == "Q5_K weight byte mismatch: got 144, expected 176", "q5k weight bytes message");
    r = q8_0_gemv_batch({w.data(), 34}, 1, 32, {x.data(), 33});
    EXPECT(!r && r.error == "Q8_0 batch input length 33 is not divisible by cols 32", "q8_0 batch message");
    r = q8_0_head_gemv_batch({w.data(), 34}, 1, 1, 32, 2, {x.data(), 63});
    EXPECT(!r && r.error == "Q8_0 head batch input length mismatch: got 63, expected 64", "q8_0 head batch message");
    float out1 = 0;
    auto u = q4k_gemv_into({w.data(), 144}, 1, 256, {x.data(), 256}, &out1, 0);
    EXPECT(!u && u.error == "Q4_K shape mismatch: input=256 output=0 expected input=256 output>=1", "into message");
    auto eg = quant_embedding_gather(RNB_GGML_Q4_K, {w.data(), 144}, 1, 256, {0, 1});
    EXPECT(!eg && eg.status == RNB_HIP_INVALID_REQUEST && eg.error == "Q4K embedding token id 1 is out of range for 1 rows",
           "embedding id message");
    eg = quant_embedding_gather(RNB_GGML_Q6_K, {w.data(), 144}, 1, 256, {0});
    EXPECT(!eg && eg.error == "Q6K embedding weight byte mismatch: got 144, expected 210", "embedding weight bytes message");
    auto m = qwen35_sparse_experts_selected_base_by_token({w.data(), 144}, {w.data(), 144}, {w.data(), 144}, {0, 1}, {1.0f}, {0}, 1, 14, 256, 256, {x.data(), 256});
    EXPECT(!m && m.error.find("length mismatch") != std::string::npos, "moe slot arrays message");
    {
        std::vector<uint8_t> gw(256 * 144, 0), dw(256 * 210, 0);
        std::vector<float> xin(512, 0.0f);
        auto f1 = dense_q4k_silu_ffn_batch({gw.data(), gw.size()}, {gw.data(), gw.size()}, {dw.data(), dw.size()}, 14, 256,
                                           256, 1, {xin.data(), 256});
        EXPECT(!f1 && f1.error == "dense SiLU FFN batch requires seq_len > 1, got 1", "dense ffn seq_len message");
        auto f2 = dense_q4k_silu_ffn_batch({gw.data(), gw.size() - 1}, {gw.data(), gw.size()}, {dw.data(), dw.size()}, 14,
                                           256, 256, 2, {xin.data(), 512});
        EXPECT(!f2 && f2.error == "dense SiLU FFN batch gate byte mismatch: got 36863, expected 36864", "dense ffn gate bytes");
    }
    {  // GGUF header parse over the C ABI: a minimal v3 file with one key, then a wrong magic
        std::vector<uint8_t> f = {'G', 'G', 'U', 'F', 3, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0};
        const char key[] = "general.architecture", val[] = "llama";
        auto put_str = [&](const char *s) {
            const uint64_t n = std::strlen(s);
            for (int i = 0; i < 8; i++) f.push_back(static_cast<uint8_t>(n >> (8 * i)));
            f.insert(f.end(), s, s + n);
        };
        put_str(key);
        f.insert(f.end(), {8, 0, 0, 0});
        put_str(val);
        auto g = GgufFile::parse({f.data(), f.size()});
        EXPECT(g && g.value.version() == 3 && g.value.tensor_count() == 0 && g.value.alignment() == 32 &&
                   g.value.data_start() % 32 == 0 && g.value.metadata_str(key) == val,
               "minimal GGUF v3 header");
        f[0] = 'X';
        auto bad = GgufFile::parse({f.data(), f.size()});
        EXPECT(!bad && bad.error == "invalid GGUF magic bytes", "GGUF magic message");
    }
    HipBackend b;
    EXPECT(b.kind() == 6, "kind ordinal");
    const BackendCapabilities c = b.capabilities();
    EXPECT(c.matmul && c.moe && !c.attention && !c.gdn && !c.sampler, "capabilities");
    EXPECT(!b.execute(RNB_OP_MATMUL) && b.execute(RNB_OP_MATMUL).status == RNB_HIP_UNSUPPORTED_OP, "execute is a facade");
    return failures;
}

static void run_case(const std::string &dir, const char *name, size_t rows, size_t cols, size_t seq,
                     Result<std::vector<float>> (*fn)(Bytes, size_t, size_t, Floats)) {
    const auto w = read_file<uint8_t>(dir + "/" + name + "_w.bin");
    const auto x = read_file<float>(dir + "/" + name + "_x.bin");
    const auto want = read_file<float>(dir + "/" + name + "_out.bin");
    if (w.empty() || x.empty() || want.empty()) return;
    auto r = fn({w.data(), w.size()}, rows, cols, {x.data(), x.size()});
    if (!r) {
        std::printf("FAIL: %s: %s\n", name, r.error.c_str());
        failures++;
        return;
    }
    EXPECT(r.value.size() == seq * rows && want.size() == seq * rows, "output size");
    double ss = 0;
    for (float v : want) ss += double(v) * v;
    const double rms = std::sqrt(ss / double(want.size()));
    double worst = 0;
    for (size_t i = 0; i < want.size(); i++) {
        const double diff = std::fabs(double(r.value[i]) - want[i]);
        const double tol = std::fmax(1e-3 * rms, 1e-3 * std::fabs(want[i]));  // abs-or-rel, rel = 1e-3
        if (!(diff <= tol)) failures++;
        worst = std::fmax(worst, diff);
    }
    std::printf("%s: %zu outputs, max |diff| %.3g (rms %.3g)\n", name, want.size(), worst, rms);
}

// the golden Q8_0 batch read as a head batch: its 7 rows as one head, and as 7 heads of one row fed the same vector
static void head_case(const std::string &dir) {
    const size_t rows = 7, cols = 96, seq = 4;
    const auto w = read_file<uint8_t>(dir + "/q8_0_batch_w.bin");
    const auto x = read_file<float>(dir + "/q8_0_batch_x.bin");
    const auto want = read_file<float>(dir + "/q8_0_batch_out.bin");
    if (w.empty() || x.empty() || want.size() != seq * rows) return;
    auto plain = q8_0_gemv_batch({w.data(), w.size()}, rows, cols, {x.data(), x.size()});
    auto one = q8_0_head_gemv_batch({w.data(), w.size()}, 1, rows, cols, seq, {x.data(), x.size()});
    std::vector<float> xr(seq * rows * cols);
    for (size_t t = 0; t < seq; t++)
        for (size_t h = 0; h < rows; h++) std::memcpy(&xr[(t * rows + h) * cols], &x[t * cols], cols * sizeof(float));
    auto many = q8_0_head_gemv_batch({w.data(), w.size()}, rows, 1, cols, seq, {xr.data(), xr.size()});
    EXPECT(plain && one && many, "head batch calls");
    if (!(plain && one && many)) return;
    EXPECT(std::memcmp(one.value.data(), plain.value.data(), want.size() * sizeof(float)) == 0, "one head == plain batch");
    EXPECT(std::memcmp(many.value.data(), plain.value.data(), want.size() * sizeof(float)) == 0, "seven heads == plain batch");
    std::printf("q8_0_head_gemv_batch: %zu outputs, both layouts bit-identical to q8_0_gemv_batch\n", want.size());
}

// rows [last, 0, 2, 2] of a golden weight file, dequantised on the device: bit-identical to the fixture
static void embed_case(const std::string &dir, const char *name, uint32_t quant, size_t rows, size_t cols) {
    const auto w = read_file<uint8_t>(dir + "/" + name + "_w.bin");
    const auto want = read_file<float>(dir + "/embed_" + name + "_out.bin");
    if (w.empty() || want.empty()) return;
    auto r = quant_embedding_gather(quant, {w.data(), w.size()}, rows, cols, {static_cast<uint32_t>(rows - 1), 0, 2, 2});
    if (!r) {
        std::printf("FAIL: embed %s: %s\n", name, r.error.c_str());
        failures++;
        return;
    }
    EXPECT(r.value.size() == want.size() && want.size() == 4 * cols, "embedding output size");
    size_t differing = 0;
    for (size_t i = 0; i < want.size() && i < r.value.size(); i++)
        differing += std::memcmp(&r.value[i], &want[i], sizeof(float)) != 0;
    if (differing) failures++;
    std::printf("embed %s: %zu values, %zu differ\n", name, want.size(), differing);
}

int main(int argc, char **argv) {
    if (argc >= 2 && std::strcmp(argv[1], "validate") == 0) {
        const int f = validate();
        std::printf("validate: %d failure(s)\n", f);
        return f ? 1 : 0;
    }
    if (argc >= 3 && std::strcmp(argv[1], "run") == 0) {
        if (rnb_hip_init() != RNB_HIP_OK) {
            std::printf("SKIP: %s\n", rnb_hip_last_error());
            return 77;
        }
        const std::string dir = argv[2];
        run_case(dir, "q4k_gemv", 24, 1024, 1, q4k_gemv);
        run_case(dir, "q6k_gemv", 20, 768, 1, q6k_gemv);
        run_case(dir, "q8_0_gemv", 16, 544, 1, q8_0_gemv);
        run_case(dir, "q4k_batch", 40, 512, 19, q4k_gemv_batch);
        run_case(dir, "q6k_batch", 9, 512, 3, q6k_gemv_batch);
        run_case(dir, "q8_0_batch", 7, 96, 4, q8_0_gemv_batch);
        run_case(dir, "q5k_gemv", 22, 1280, 1, q5k_gemv);
        run_case(dir, "q5k_batch", 13, 512, 5, q5k_gemv_batch);
        run_case(dir, "q2k_gemv", 18, 768, 1, q2k_gemv);
        run_case(dir, "q3k_batch", 11, 512, 6, q3k_gemv_batch);
        run_case(dir, "q4_0_gemv", 21, 608, 1, q4_0_gemv);
        run_case(dir, "q5_1_batch", 10, 160, 3, q5_1_gemv_batch);
        run_case(dir, "q8_1_gemv", 19, 160, 1, q8_1_gemv);
        run_case(dir, "q6k_gemm", 33, 512, 20, q6k_gemv_batch);
        run_case(dir, "q5k_gemm", 40, 256, 17, q5k_gemv_batch);
        run_case(dir, "q8_0_gemm", 35, 96, 18, q8_0_gemv_batch);
        run_case(dir, "iq4_xs_gemv", 17, 768, 1, iq4_xs_gemv);
        run_case(dir, "iq2_xxs_batch", 12, 512, 3, iq2_xxs_gemv_batch);
        run_case(dir, "iq3_xxs_gemv", 14, 512, 1, iq3_xxs_gemv);
        run_case(dir, "iq2_s_batch", 9, 256, 2, iq2_s_gemv_batch);
        head_case(dir);
        embed_case(dir, "q4k_gemv", RNB_GGML_Q4_K, 24, 1024);
        embed_case(dir, "q6k_gemv", RNB_GGML_Q6_K, 20, 768);
        embed_case(dir, "q8_0_gemv", RNB_GGML_Q8_0, 16, 544);
        embed_case(dir, "iq2_s_batch", RNB_GGML_IQ2_S, 9, 256);
        std::printf("run: %d failure(s)\n", failures);
        return failures ? 1 : 0;
    }
    std::printf("usage: host_mirror_test validate | run <golden_dir>\n");
    return 2;
}
