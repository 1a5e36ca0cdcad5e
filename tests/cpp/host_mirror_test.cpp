// Exercises the C++ host-side mirror (izwi_amd/host/izwi_qmm.hpp) the way the
// reference's own unit tests exercise its Rust types.
//   host_mirror_test cpu [fixture]   host logic only: byte-size rule and its errors, GGUF
//                          container parse of tests/golden/tiny.gguf
//   host_mirror_test gpu   the reference's packed-projection test
//                          (crates/izwi-core/src/models/architectures/qwen3/core.rs:3099-3142)
//                          and a Q4_K projection, the folded calls (norm, activation,
//                          residual) and the hooks' namespace, checked against the CPU oracle
// Test infrastructure: links the oracle (liboracle_qmm.so) as the checker.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "izwi_qmm.hpp"

extern "C" {
int oracle_qmatmul(int dtype, int64_t m, int64_t k, int64_t n, const float* lhs, const void* rhs_t, float* dst);
int oracle_quantize(int dtype, int64_t rows, int64_t cols, const float* src, void* dst);
int64_t oracle_storage_bytes(int dtype, int64_t rows, int64_t cols);
void oracle_fill_normal(uint64_t seed, int64_t offset, int64_t count, float mean, float std, float* out);
void oracle_rms_norm(const float* x, const float* weight, int64_t rows, int64_t hidden, float eps, float* y);
void oracle_argmax(const float* x, int64_t rows, int64_t n, uint32_t* out);
}

static int failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);     \
            failures++;                                                     \
        }                                                                   \
    } while (0)

template <class F>
static bool throws(izwi::Error::Kind kind, const char* needle, F&& f) {
    try {
        f();
    } catch (const izwi::Error& e) {
        if (e.kind() != kind) std::printf("  wrong kind, message: %s\n", e.what());
        if (needle && !std::strstr(e.what(), needle)) std::printf("  message lacks '%s': %s\n", needle, e.what());
        return e.kind() == kind && (!needle || std::strstr(e.what(), needle));
    }
    return false;
}

static std::vector<uint8_t> quantize(izwi::GgmlDType dt, const std::vector<float>& w, int64_t n, int64_t k) {
    std::vector<uint8_t> blocks((size_t)oracle_storage_bytes((int)dt, n, k));
    if (oracle_quantize((int)dt, n, k, w.data(), blocks.data())) std::printf("oracle_quantize rejected the shape\n");
    return blocks;
}

static float max_rel(const std::vector<float>& a, const std::vector<float>& b) {
    float mx = 0.0f, scale = 0.0f;
    for (size_t i = 0; i < b.size(); i++) scale = std::fmax(scale, std::fabs(b[i]));
    for (size_t i = 0; i < b.size(); i++) mx = std::fmax(mx, std::fabs(a[i] - b[i]));
    return mx / (scale > 0 ? scale : 1.0f);
}

static void host_logic() {
    using izwi::GgmlDType;
    EXPECT(izwi::quantized_storage_bytes(3072, 1024, GgmlDType::Q8_0) == 3342336u);
    EXPECT(izwi::quantized_storage_bytes(12288, 4096, GgmlDType::Q4K) == 28311552u);
    EXPECT(izwi::quantized_storage_bytes(0, 4096, GgmlDType::Q4K) == 0u);
    EXPECT(throws(izwi::Error::Kind::InvalidInput, "not divisible by block size",
                  [] { izwi::quantized_storage_bytes(3, 100, GgmlDType::Q4K); }));
    EXPECT(throws(izwi::Error::Kind::ModelLoadError, "not supported",
                  [] { izwi::quantized_storage_bytes(4, 256, (GgmlDType)13); }));
    EXPECT(izwi::block_size(GgmlDType::Q4K) == 256 && izwi::type_size(GgmlDType::Q4K) == 144);
    EXPECT(izwi::block_size(GgmlDType::Q8_0) == 32 && izwi::type_size(GgmlDType::Q8_0) == 34);
    EXPECT(izwi::block_size(GgmlDType::Q6K) == 256 && izwi::type_size(GgmlDType::Q6K) == 210);
    EXPECT(izwi::quantized_storage_bytes(4096, 12288, GgmlDType::Q6K) == 4096u * 48u * 210u);
}

static void no_device_is_loud() {
    std::vector<uint8_t> blocks(34 * 2, 0);
    EXPECT(throws(izwi::Error::Kind::ModelLoadError, "no CPU fallback", [&] {
        izwi::QTensor::from_blocks(izwi::GgmlDType::Q8_0, blocks.data(), blocks.size(), 2, 32);
    }));
}

static void packed_matches_separate_q8_0() {
    using izwi::GgmlDType;
    std::vector<float> w1(64), w2(32), x(32);
    for (int i = 0; i < 64; i++) w1[i] = (float)(i - 31) / 8.0f;
    for (int i = 0; i < 32; i++) w2[i] = (float)(15 - i) / 7.0f;
    for (int i = 0; i < 32; i++) x[i] = (float)(i + 1) / 16.0f;
    auto b1 = quantize(GgmlDType::Q8_0, w1, 2, 32), b2 = quantize(GgmlDType::Q8_0, w2, 1, 32);
    auto q1 = izwi::QTensor::from_blocks(GgmlDType::Q8_0, b1.data(), b1.size(), 2, 32);
    auto q2 = izwi::QTensor::from_blocks(GgmlDType::Q8_0, b2.data(), b2.size(), 1, 32);
    EXPECT(q1->data() == b1 && q2->data() == b2);
    // the reference's test builds its tensors with QTensor::quantize: the same blocks
    EXPECT(izwi::QTensor::quantize(w1, 2, 32, GgmlDType::Q8_0)->data() == b1);
    EXPECT(izwi::QTensor::quantize(w2, 1, 32, GgmlDType::Q8_0)->data() == b2);
    auto y1 = izwi::QMatMul::from_arc(q1).forward(x);
    auto y2 = izwi::QMatMul::from_qtensor(q2).forward(x);
    auto packed = izwi::Qwen3Projection::packed_quantized({q1, q2});
    EXPECT(packed.qmatmul().out_features() == 3 && packed.qmatmul().in_features() == 32);
    auto yp = packed.forward(x);
    EXPECT(yp.size() == 3);
    // the reference asserts packed == cat(separate) within 1e-5
    EXPECT(std::fabs(yp[0] - y1[0]) < 1e-5f && std::fabs(yp[1] - y1[1]) < 1e-5f && std::fabs(yp[2] - y2[0]) < 1e-5f);
    // absolute values of candle-core's algorithm on this input
    const float want[3] = {-42.692207f, 89.229607f, -26.613434f};
    for (int i = 0; i < 3; i++) EXPECT(std::fabs(yp[i] - want[i]) < 1e-4f);
    // error texts of the packing rule
    EXPECT(throws(izwi::Error::Kind::ModelLoadError, "empty", [] { izwi::packed_qmatmul_from_qtensors({}); }));
    std::vector<float> w3(64, 0.5f);
    auto b3 = quantize(GgmlDType::Q8_0, w3, 1, 64);
    auto q3 = izwi::QTensor::from_blocks(GgmlDType::Q8_0, b3.data(), b3.size(), 1, 64);
    EXPECT(throws(izwi::Error::Kind::InvalidInput, nullptr, [&] { izwi::packed_qmatmul_from_qtensors({q1, q3}); }));
    EXPECT(throws(izwi::Error::Kind::InvalidInput, "multiple of k", [&] { izwi::QMatMul::from_arc(q1).forward(std::vector<float>(33, 1.0f)); }));
}

static void q4k_projection_matches_oracle() {
    using izwi::GgmlDType;
    const int64_t n = 200, k = 1280, m = 5;
    std::vector<float> w((size_t)n * k), x((size_t)m * k);
    oracle_fill_normal(11, 0, (int64_t)w.size(), 0.0f, 0.02f, w.data());
    oracle_fill_normal(12, 0, (int64_t)x.size(), 0.0f, 1.0f, x.data());
    auto blocks = quantize(GgmlDType::Q4K, w, n, k);
    auto q = izwi::QTensor::from_blocks(GgmlDType::Q4K, blocks.data(), blocks.size(), n, k);
    EXPECT(q->dtype() == GgmlDType::Q4K && q->dims2().first == n && q->dims2().second == k);
    EXPECT(q->data() == blocks);
    EXPECT(izwi::QTensor::quantize(w, n, k, GgmlDType::Q4K)->data() == blocks);
    auto y = izwi::Qwen3Projection::quantized(q).forward(x);
    std::vector<float> want((size_t)m * n);
    EXPECT(oracle_qmatmul((int)GgmlDType::Q4K, m, k, n, x.data(), blocks.data(), want.data()) == 0);
    EXPECT(max_rel(y, want) < 1e-4f);
}

// The folded calls of a decode step through the mirror, host pointers: the norm inside the
// projection, the activation inside gate/up, the residual inside down, the greedy argmax.
static void folded_calls_match_oracle() {
    using izwi::GgmlDType;
    using izwi::MemSpace;
    const int64_t hidden = 512, inter = 768, m = 1;
    std::vector<float> wg((size_t)inter * hidden), wu(wg.size()), wd((size_t)hidden * inter), x((size_t)m * hidden),
        nw((size_t)hidden);
    oracle_fill_normal(21, 0, (int64_t)wg.size(), 0.0f, 0.05f, wg.data());
    oracle_fill_normal(22, 0, (int64_t)wu.size(), 0.0f, 0.05f, wu.data());
    oracle_fill_normal(23, 0, (int64_t)wd.size(), 0.0f, 0.05f, wd.data());
    oracle_fill_normal(24, 0, (int64_t)x.size(), 0.0f, 2.0f, x.data());
    oracle_fill_normal(25, 0, (int64_t)nw.size(), 1.0f, 0.1f, nw.data());
    auto bg = quantize(GgmlDType::Q4K, wg, inter, hidden), bu = quantize(GgmlDType::Q4K, wu, inter, hidden),
         bd = quantize(GgmlDType::Q4K, wd, hidden, inter);
    auto gate = izwi::QMatMul::from_arc(izwi::QTensor::from_blocks(GgmlDType::Q4K, bg.data(), bg.size(), inter, hidden));
    auto up = izwi::QMatMul::from_arc(izwi::QTensor::from_blocks(GgmlDType::Q4K, bu.data(), bu.size(), inter, hidden));
    auto down = izwi::QMatMul::from_arc(izwi::QTensor::from_blocks(GgmlDType::Q4K, bd.data(), bd.size(), hidden, inter));

    // the oracle's composition: norm, two products, silu(g) * u, product, + x
    std::vector<float> xn(x.size()), g((size_t)m * inter), u(g.size()), h(g.size()), want((size_t)m * hidden);
    oracle_rms_norm(x.data(), nw.data(), m, hidden, 1e-6f, xn.data());
    EXPECT(oracle_qmatmul((int)GgmlDType::Q4K, m, hidden, inter, xn.data(), bg.data(), g.data()) == 0);
    EXPECT(oracle_qmatmul((int)GgmlDType::Q4K, m, hidden, inter, xn.data(), bu.data(), u.data()) == 0);
    for (size_t i = 0; i < h.size(); i++) h[i] = g[i] / (1.0f + std::exp(-g[i])) * u[i];
    EXPECT(oracle_qmatmul((int)GgmlDType::Q4K, m, inter, hidden, h.data(), bd.data(), want.data()) == 0);
    for (size_t i = 0; i < want.size(); i++) want[i] += x[i];

    std::vector<float> got_n(xn.size()), got_g(g.size()), got_h(h.size()), got((size_t)m * hidden);
    izwi::kernels::rms_norm(x.data(), nw.data(), m, hidden, 1e-6f, got_n.data(), MemSpace::Host);
    EXPECT(max_rel(got_n, xn) < 1e-5f);
    gate.forward_normed(x.data(), m, nw.data(), 1e-6f, got_g.data(), MemSpace::Host);
    EXPECT(max_rel(got_g, g) < 3e-4f);
    izwi::forward_gate_up_silu(gate, up, x.data(), m, got_h.data(), MemSpace::Host, nullptr, nw.data(), 1e-6f);
    EXPECT(max_rel(got_h, h) < 3e-4f);
    down.forward_fused(got_h.data(), false, m, x.data(), got.data(), false, MemSpace::Host);
    EXPECT(max_rel(got, want) < 1e-3f);
    std::vector<float*> ys = {got_g.data(), got_h.data()};
    izwi::forward_group_normed({&gate, &up}, x.data(), m, nw.data(), 1e-6f, ys, MemSpace::Host);
    EXPECT(max_rel(got_g, g) < 3e-4f && max_rel(got_h, u) < 3e-4f);
    {
        // Qwen3Mlp::forward as one call: the two calls' bits (no norm, no residual here)
        std::vector<float> h2(h.size()), y2((size_t)m * hidden), y1((size_t)m * hidden);
        izwi::forward_gate_up_silu(gate, up, x.data(), m, h2.data(), MemSpace::Host);
        down.forward(h2.data(), m, y2.data(), MemSpace::Host);
        izwi::mlp_forward(gate, up, down, x.data(), m, y1.data(), MemSpace::Host);
        EXPECT(y1 == y2);
    }
    uint32_t best = 0, best_want = 1;
    izwi::kernels::argmax(got.data(), m, hidden, &best, MemSpace::Host);
    oracle_argmax(got.data(), m, hidden, &best_want);
    EXPECT(best == best_want);
    EXPECT(throws(izwi::Error::Kind::InvalidInput, nullptr,
                  [&] { izwi::kernels::rms_norm(x.data(), nw.data(), 1, 0, 1e-6f, got_n.data(), MemSpace::Host); }));
}

// The committed GGUF fixture (tests/golden/tiny.gguf, laid out by hand from the container
// format): three tensors, alignment 64.  Parsing needs no GPU.
static void gguf_parse(const std::string& fixture) {
    EXPECT(izwi::is_gguf_file(fixture));
    EXPECT(!izwi::is_gguf_file(fixture + ".absent"));
    auto g = izwi::GgufLoader::from_path(fixture);
    EXPECT(g->tensor_count() == 3);
    const std::vector<std::string> names = g->tensor_names();
    EXPECT(names.size() == 3 && names[0] == "a" && names[1] == "blk.q" && names[2] == "hand.q4k");
    EXPECT(g->has_tensor("blk.q") && !g->has_tensor("blk.k"));
    EXPECT((g->tensor_shape("hand.q4k") == std::vector<int64_t>{1, 256}));
    bool found = true;
    EXPECT(g->tensor_shape("nope", &found).empty() && !found);
    std::string arch;
    uint64_t v = 0;
    EXPECT(g->get_metadata_string("general.architecture", &arch) && arch == "qwen3");
    EXPECT(g->get_metadata_u64("general.alignment", &v) && v == 64);
    EXPECT(!g->get_metadata_string("general.alignment", &arch) && !g->get_metadata_u64("absent", &v));
    EXPECT(throws(izwi::Error::Kind::ModelLoadError, "Failed to open GGUF file",
                  [&] { izwi::GgufLoader::from_path(fixture + ".absent"); }));
    EXPECT(throws(izwi::Error::Kind::ModelLoadError, "not supported", [&] { g->load_qtensor("a"); }));
    EXPECT(throws(izwi::Error::Kind::ModelLoadError, "tensor not found", [&] { g->load_qtensor("nope"); }));
    // the reader policy of backends/model_io.rs: auto maps, "off" reads with buffered I/O, same contents
    EXPECT(g->reader_kind() == izwi::GgufReaderKind::Mapped);
    izwi::GgufMmapMode mode = izwi::GgufMmapMode::Auto;
    EXPECT(izwi::parse_gguf_mmap_mode("no", &mode) && mode == izwi::GgufMmapMode::Off);
    EXPECT(izwi::parse_gguf_mmap_mode(" TRUE ", &mode) && mode == izwi::GgufMmapMode::On);
    EXPECT(!izwi::parse_gguf_mmap_mode("", &mode) && !izwi::parse_gguf_mmap_mode("invalid", &mode));
    const izwi::GgufMmapMode off = izwi::GgufMmapMode::Off;
    auto b = izwi::GgufLoader::from_path(fixture, &off);
    EXPECT(b->reader_kind() == izwi::GgufReaderKind::Buffered && b->tensor_names() == names);
}

// ... and its tensors on the GPU: the Q4_K tensor is the hand-built block whose closed form
// sums to 32224; the Q8_0 block is d = 1, q = -16 .. 15.
// `logits_for_tokens` (core.rs:745-758): the selected ids of the full product, bit for bit.
static void selected_token_logits() {
    using izwi::GgmlDType;
    const int64_t n = 4000, k = 1024;
    std::vector<float> w((size_t)n * k), x((size_t)k);
    oracle_fill_normal(71, 0, (int64_t)w.size(), 0.0f, 0.02f, w.data());
    oracle_fill_normal(72, 0, k, 0.0f, 1.0f, x.data());
    std::vector<uint8_t> blocks((size_t)oracle_storage_bytes((int)GgmlDType::Q4K, n, k));
    EXPECT(oracle_quantize((int)GgmlDType::Q4K, n, k, w.data(), blocks.data()) == 0);
    auto proj = izwi::Qwen3Projection::quantized(izwi::QTensor::from_blocks(GgmlDType::Q4K, blocks.data(), blocks.size(), n, k));
    const std::vector<float> full = proj.forward(x);
    const std::vector<uint32_t> ids = {3999, 0, 17, 17, 2048, 1};
    const auto pairs = proj.logits_for_tokens(x, ids);
    EXPECT(pairs.size() == ids.size());
    for (size_t i = 0; i < pairs.size(); i++) EXPECT(pairs[i].first == ids[i] && pairs[i].second == full[ids[i]]);
    EXPECT(proj.logits_for_tokens(x, {}).empty());
    EXPECT(throws(izwi::Error::Kind::InvalidInput, "out of range", [&] { proj.logits_for_tokens(x, {4000}); }));
}

static void gguf_load(const std::string& fixture) {
    auto g = izwi::GgufLoader::from_path(fixture);
    auto q4 = g->load_qtensor("hand.q4k");
    EXPECT(q4->dtype() == izwi::GgmlDType::Q4K && q4->rows() == 1 && q4->cols() == 256);
    const std::vector<float> deq = q4->dequantize();
    double sum = 0;
    for (float f : deq) sum += f;
    EXPECT(sum == 32224.0 && deq[224] == 346.5f && deq[32] == -2.5f);
    EXPECT(g->load_tensor("hand.q4k") == deq);
    EXPECT(q4->dequantize_rows({0, 0}) == [&] { std::vector<float> two = deq; two.insert(two.end(), deq.begin(), deq.end()); return two; }());
    EXPECT(q4->dequantize_rows({}).empty());
    EXPECT(throws(izwi::Error::Kind::InvalidInput, "out of range", [&] { q4->dequantize_rows({1}); }));
    const std::vector<float> q8 = g->load_tensor("blk.q");
    EXPECT(q8.size() == 32 && q8[0] == -16.0f && q8[31] == 15.0f);
    EXPECT((g->load_tensor("a") == std::vector<float>{1.0f, 2.0f, 3.0f, 4.0f}));
    // a projection loaded from the file: y = x . w with x = ones gives the row sum
    std::vector<float> x(32, 1.0f);
    const std::vector<float> y = izwi::QMatMul::from_qtensor(g->load_qtensor("blk.q")).forward(x);
    EXPECT(y.size() == 1 && std::fabs(y[0] - (-16.0f)) < 1e-3f);
}

int main(int argc, char** argv) {
    const std::string mode = argc > 1 ? argv[1] : "cpu";
    const std::string fixture = argc > 2 ? argv[2] : "tests/golden/tiny.gguf";
    host_logic();
    gguf_parse(fixture);
    if (mode == "gpu") {
        packed_matches_separate_q8_0();
        q4k_projection_matches_oracle();
        folded_calls_match_oracle();
        selected_token_logits();
        gguf_load(fixture);
    } else if (mode == "nodevice") {
        no_device_is_loud();
    }
    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
