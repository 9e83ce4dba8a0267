// Drives a bare mixture-of-experts layer through the C++ host mirror, the way the
// reference's tutorial does (tutorials/code/15_mixture_of_experts.rs:58-120): the
// total-vs-active parameter table, then the load fractions and the two auxiliary losses
// for varied and for identical tokens.  It also asserts the reference's own unit-test
// expectations, so it doubles as the test of the C++ host side.
//
//   moe_tutorial --cpu-checks   configuration, accounting and error paths only (no GPU)
//   moe_tutorial                everything, on GPU 0
//   moe_tutorial --rbw FILE     parses a `.rbw` weight snapshot and prints what it holds (no GPU)
//   moe_tutorial --rbw FILE ROWS.f32 TOKENS OUT
//                               also loads its sparse blocks onto GPU 0 and runs the block step
//                               x + layer(rmsnorm(x)) on the rows of ROWS.f32 ([TOKENS, d_model] f32),
//                               writing each block's output to OUT.<block> (f32)
#include <cmath>
#include <cstdio>
#include <cstring>

#include "rbw.hpp"
#include "rusting_brain_moe.hpp"

using namespace rusting_brain;

static int failures = 0;
#define EXPECT(cond)                                                   \
    do {                                                               \
        if (!(cond)) {                                                 \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                \
        }                                                              \
    } while (0)

template <typename E, typename F>
static bool throws(F f) {
    try {
        f();
    } catch (const E&) {
        return true;
    } catch (...) {
        return false;
    }
    return false;
}

// small deterministic generator (values in [-1, 1)); the tutorial's StdRng stream cannot be reproduced
static float unit(uint64_t& s) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((s >> 40) & 0xffffff) / 8388608.0f - 1.0f;
}
static Matrix random_matrix(size_t r, size_t c, float bound, uint64_t seed) {
    Matrix m(r, c);
    uint64_t s = seed * 2654435761ull + 12345;
    for (float& v : m.data) v = unit(s) * bound;
    return m;
}

static void cpu_checks() {
    // reference src/moe.rs:704-710
    EXPECT(throws<InvalidConfig>([] { MoeConfig(4, 0, 6).validate(); }));
    EXPECT(throws<InvalidConfig>([] { MoeConfig(4, 5, 6).validate(); }));
    EXPECT(throws<InvalidConfig>([] { MoeConfig(0, 1, 6).validate(); }));
    MoeConfig(4, 4, 6).validate();
    // reference README.md:96: 55.2M total / 35.7M active for the default configuration
    const ParameterCounts c = TransformerBuilder().parameter_counts();
    EXPECT(c.total == 55181824ull && c.active == 35717632ull);
    // reference src/transformer.rs:3020-3026
    auto tiny = [] { return TransformerBuilder().n_layers(2).moe_layers({1}).experts(4, 2); };
    EXPECT(throws<InvalidConfig>([&] { tiny().heads(4, 3, 4).validate(); }));
    EXPECT(throws<InvalidConfig>([&] { tiny().heads(4, 2, 5).validate(); }));
    EXPECT(throws<InvalidConfig>([&] { tiny().moe_layers({9}).validate(); }));
    EXPECT(throws<InvalidConfig>([&] { tiny().experts(2, 4).validate(); }));
    // reference src/batch.rs:254-268
    std::vector<bool> mask = {true, false, true};
    Layout bad;
    bad.valid = &mask;
    EXPECT(throws<InvalidConfig>([&] { bad.check(4); }));
    Layout seq;
    seq.seq_len = 4;
    EXPECT(throws<InvalidConfig>([&] { seq.check(9); }));

    std::printf("== Total vs active, as experts are added ==\n\nexperts   total    active    ratio\n");
    for (size_t n : {1, 2, 4, 8, 16, 32}) {
        const ParameterCounts p = TransformerBuilder().experts(n, n < 2 ? n : 2).parameter_counts();
        std::printf("%7zu %6.1fM %7.1fM %7.2fx\n", n, p.total / 1e6, p.active / 1e6, (double)p.total / p.active);
    }
}

static void report(const char* label, MoeLayer& layer, const Matrix& tokens, size_t experts) {
    auto result = layer.forward_train(tokens, Layout{});
    const MoeCache& cache = result.second;
    const std::vector<float> loads = cache.load_fractions();
    float busiest = 0.0f;
    size_t dead = 0;
    std::printf("%s\n  routing ", label);
    for (float share : loads) {
        std::printf("%6.1f%%", share * 100.0f);
        busiest = std::fmax(busiest, share);
        dead += share < 0.01f;
    }
    std::printf("\n  busiest %.1f%%   dead experts %zu/%zu   aux %.4f   z %.4f\n", busiest * 100.0f, dead, experts,
                cache.aux_loss(), cache.z_loss());
}

static void gpu_checks() {
    const size_t D = 64, E = 8, K = 2, F = 32, ROWS = 512;
    auto device = Device::open(0);
    MoeLayer layer(D, MoeConfig(E, K, F), device, ROWS);
    const float bound = std::sqrt(6.0f / (float)(D + F));
    layer.set_router(random_matrix(E, D, std::sqrt(6.0f / (float)(D + E)), 7));
    for (size_t e = 0; e < E; ++e)
        layer.set_expert(e, random_matrix(F, D, bound, 100 + 3 * e), random_matrix(F, D, bound, 101 + 3 * e),
                         random_matrix(D, F, bound, 102 + 3 * e));

    std::printf("\n== What the load-balancing loss measures ==\n\n");
    const Matrix varied = random_matrix(ROWS, D, 1.0f, 11);
    report("varied tokens, balanced routing:", layer, varied, E);
    Matrix same(ROWS, D);
    const Matrix one = random_matrix(1, D, 1.0f, 13);
    for (size_t r = 0; r < ROWS; ++r) std::memcpy(same.row_mut(r), one.data.data(), D * sizeof(float));
    report("identical tokens, collapsed routing:", layer, same, E);

    // reference tutorials/15_mixture_of_experts.md:310-312: exactly two experts at 50 %, six dead
    {
        auto r = layer.forward_train(same, Layout{});
        size_t half = 0, zero = 0;
        for (float f : r.second.load_fractions()) {
            half += f == 0.5f;
            zero += f == 0.0f;
        }
        EXPECT(half == 2 && zero == E - 2);
    }
    // reference src/moe.rs:696-702, :726-741, :757-765
    {
        auto r = layer.forward_train(varied, Layout{});
        EXPECT(r.first.rows == ROWS && r.first.cols == D);
        size_t routed = 0;
        for (const auto& v : r.second.expert_tokens) routed += v.size();
        EXPECT(routed == ROWS * K);
        bool sums_ok = true;
        for (size_t t = 0; t < ROWS; ++t) {
            float total = 0.0f;
            for (size_t q = 0; q < K; ++q) total += r.second.assignments[t * K + q].second;
            sums_ok = sums_ok && std::fabs(total - 1.0f) < 1e-5f;
        }
        EXPECT(sums_ok);
        EXPECT(r.second.aux_loss() >= 0.01f - 1e-6f && r.second.aux_loss() <= (float)E * 0.01f + 1e-6f);
        EXPECT(r.second.z_loss() > 0.0f);
    }
    // reference src/moe.rs:248-253
    EXPECT(throws<InvalidInput>([&] { layer.forward(Matrix(3, D + 1)); }));
    // padding rows are routed nowhere (reference src/moe.rs:559-562)
    {
        std::vector<bool> mask(ROWS, true);
        mask[5] = false;
        Layout layout;
        layout.valid = &mask;
        auto r = layer.forward_train(varied, layout);
        EXPECT(r.second.assignments[5 * K].first == UNROUTED && r.second.assignments[5 * K].second == 0.0f);
        EXPECT(r.second.valid_tokens == ROWS - 1);
        bool zero_row = true;
        for (size_t c = 0; c < D; ++c) zero_row = zero_row && r.first.row(5)[c] == 0.0f;
        EXPECT(zero_row);
    }
    // the builder surface hands out one layer per index in moe_layers
    {
        auto layers = TransformerBuilder().d_model(16).n_layers(4).experts(4, 2).moe_layers({1, 3}).moe_d_ff(12)
                          .shared_expert(true).build_moe_layers(device, 8);
        EXPECT(layers.size() == 2 && layers.count(1) && layers.count(3));
        EXPECT(layers[1]->num_parameters() == 4 * 16 + 5 * 3 * 16 * 12);
    }
    // training through the C++ mirror: the block step (norm, layer, residual) forward and backward on an all-f32 layer
    {
        const size_t TD = 64, TE = 4, TF = 32, TR = 48;
        MoeLayer train(TD, MoeConfig(TE, 2, TF).with_aux_loss_weight(0.0f).with_router_z_loss_weight(0.0f), device, TR);
        train.enable_training();
        std::vector<float> norm_w(TD);
        for (size_t c = 0; c < TD; ++c) norm_w[c] = 0.75f + 0.01f * (float)c;
        train.set_feed_forward_norm(norm_w, 1e-6f);
        const float tb = std::sqrt(6.0f / (float)(TD + TF));
        train.set_router(random_matrix(TE, TD, 0.5f, 21));
        for (size_t e = 0; e < TE; ++e)
            train.set_expert(e, random_matrix(TF, TD, tb, 200 + 3 * e), random_matrix(TF, TD, tb, 201 + 3 * e),
                             random_matrix(TD, TF, tb, 202 + 3 * e));
        const Matrix x = random_matrix(TR, TD, 1.0f, 23);
        Matrix ones(TR, TD);
        for (float& v : ones.data) v = 1.0f;
        const Matrix out = train.forward_block(x);
        const Matrix grad = train.backward_block(ones);
        EXPECT(grad.rows == TR && grad.cols == TD);
        // finite differences of sum(out) in a few coordinates (reference src/moe.rs:895-925: epsilon 1e-3, 2e-2)
        double sum0 = 0.0;
        for (float v : out.data) sum0 += v;
        (void)sum0;
        bool fd_ok = true;
        for (size_t idx : {size_t(0), size_t(7 * TD + 3), size_t(40 * TD + 60)}) {
            Matrix hi = x, lo = x;
            hi.data[idx] += 1e-3f;
            lo.data[idx] -= 1e-3f;
            double sh = 0.0, sl = 0.0;
            for (float v : train.forward_block(hi).data) sh += v;
            for (float v : train.forward_block(lo).data) sl += v;
            const double numeric = (sh - sl) / (double)(hi.data[idx] - lo.data[idx]);
            fd_ok = fd_ok && std::fabs(numeric - grad.data[idx]) < 2e-2 * std::fmax(1.0, std::fabs(numeric));
        }
        EXPECT(fd_ok);
        // gradients accumulate until cleared (Param.grad), and the norm's scale has one too
        train.forward_block(x);
        const Matrix g1 = train.weight_grad(RBMOE_W_DOWN, 1);
        train.backward_block(ones);
        const Matrix g2 = train.weight_grad(RBMOE_W_DOWN, 1);
        bool doubled = true, any = false;
        for (size_t i = 0; i < g1.data.size(); ++i) {
            doubled = doubled && std::fabs(g2.data[i] - 2.0f * g1.data[i]) <= 1e-5f * (1.0f + std::fabs(g2.data[i]));
            any = any || g1.data[i] != 0.0f;
        }
        EXPECT(doubled && any);
        EXPECT(train.weight_grad(RBMOE_W_NORM).cols == TD);
        train.zero_grads();
        bool cleared = true;
        for (float v : train.weight_grad(RBMOE_W_DOWN, 1).data) cleared = cleared && v == 0.0f;
        EXPECT(cleared);
        // no backward pass for a layer that is not in training mode
        EXPECT(throws<InvalidConfig>([&] { layer.backward(Matrix(ROWS, D)); }));
    }
    // TransformerLm::quantize on the layer (reference src/transformer.rs:899-910): a router quantized at upload by
    // the in-memory rule routes exactly as the same int8 rows and scales handed over as they are
    {
        const size_t QD = 64, QE = 8, QF = 32, QR = 96;
        MoeLayer at_upload(QD, MoeConfig(QE, 2, QF), device, QR, RBMOE_F32, RBMOE_I8);
        MoeLayer as_stored(QD, MoeConfig(QE, 2, QF), device, QR, RBMOE_F32, RBMOE_I8);
        at_upload.quantize_on_upload(true, true);
        as_stored.quantize_on_upload(true, false);
        const Matrix router = random_matrix(QE, QD, 0.5f, 31);
        std::vector<int8_t> q(QE * QD);
        std::vector<float> scales(QE);
        for (size_t e = 0; e < QE; ++e) {   // Quantized::from_matrix, reference src/quantized.rs:29-51
            float absmax = 0.0f;
            for (size_t c = 0; c < QD; ++c) absmax = std::fmax(absmax, std::fabs(router.row(e)[c]));
            const float scale = absmax / 127.0f, inv = scale > 0.0f ? 1.0f / scale : 0.0f;
            scales[e] = scale;
            for (size_t c = 0; c < QD; ++c)
                q[e * QD + c] = (int8_t)std::fmin(127.0f, std::fmax(-127.0f, std::round(router.row(e)[c] * inv)));
        }
        at_upload.set_router(router);
        as_stored.set_router_q8(q.data(), scales.data());
        const float qb = std::sqrt(6.0f / (float)(QD + QF));
        for (size_t e = 0; e < QE; ++e) {
            const Matrix g = random_matrix(QF, QD, qb, 300 + 3 * e), u = random_matrix(QF, QD, qb, 301 + 3 * e),
                         d = random_matrix(QD, QF, qb, 302 + 3 * e);
            at_upload.set_expert(e, g, u, d);
            as_stored.set_expert(e, g, u, d);
        }
        const Matrix x = random_matrix(QR, QD, 1.0f, 33);
        auto a = at_upload.forward_train(x, Layout{});
        auto b = as_stored.forward_train(x, Layout{});
        EXPECT(a.second.assignments == b.second.assignments);
        EXPECT(a.second.probabilities.data == b.second.probabilities.data);
        EXPECT(a.first.data == b.first.data);
    }
    // a budget that cannot hold the layer is refused before anything is allocated
    EXPECT(throws<MemoryBudget>([&] {
        auto small = Device::open(0, 1);
        MoeLayer big(768, MoeConfig(8, 2, 1408), small, 1024);
    }));
}

// sum of the values `load_bin` would restore, in double: a checksum that the Python reader can reproduce
static double checksum(const rbw::Param& p) {
    double s = 0.0;
    if (p.q.empty()) {
        for (float v : p.values) s += (double)v;
    } else {
        for (size_t r = 0; r < p.rows; ++r)
            for (size_t c = 0; c < p.cols; ++c) s += (double)((float)p.q[r * p.cols + c] * p.scales[r]);
    }
    return s;
}

static int rbw_mode(int argc, char** argv) {
    const std::string path = argv[2];
    const rbw::Snapshot snap = rbw::read(path);
    std::printf("precision %s parameters %zu optimizer_step %llu\n", snap.precision.c_str(), snap.params.size(),
                (unsigned long long)snap.optimizer_step);
    const std::vector<rbw::MoeBlock> blocks = rbw::moe_blocks(snap);
    for (const rbw::MoeBlock& b : blocks) {
        std::printf("block %zu experts %zu shared %d norm %.9g router %.9g gate0 %.9g down_last %.9g\n", b.block,
                    b.experts.size(), b.has_shared ? 1 : 0, b.norm ? checksum(*b.norm) : 0.0, checksum(*b.router),
                    checksum(*b.experts.front().gate),
                    checksum(b.has_shared ? *b.shared.down : *b.experts.back().down));
    }
    if (argc < 6) return 0;
    const size_t tokens = (size_t)std::atol(argv[4]);
    const size_t d = snap.config.at("d_model").as_size("d_model");
    Matrix x(tokens, d);
    std::FILE* f = std::fopen(argv[3], "rb");
    if (!f || std::fread(x.data.data(), 4, x.data.size(), f) != x.data.size()) {
        std::printf("FAILED: cannot read %zu x %zu f32 from %s\n", tokens, d, argv[3]);
        return 2;
    }
    std::fclose(f);
    auto layers = rbw::load_moe_layers(path, Device::open(0), tokens);
    for (size_t i = 0; i < layers.size(); ++i) {
        const Matrix out = layers[i]->forward_block(x);
        const std::string name = std::string(argv[5]) + "." + std::to_string(blocks[i].block);
        std::FILE* o = std::fopen(name.c_str(), "wb");
        if (!o || std::fwrite(out.data.data(), 4, out.data.size(), o) != out.data.size()) {
            std::printf("FAILED: cannot write %s\n", name.c_str());
            return 2;
        }
        std::fclose(o);
        std::printf("block %zu ran on %s\n", blocks[i].block, layers[i]->kernel_name().c_str());
    }
    return 0;
}

int main(int argc, char** argv) {
    const bool cpu_only = argc > 1 && std::strcmp(argv[1], "--cpu-checks") == 0;
    if (argc > 2 && std::strcmp(argv[1], "--rbw") == 0) {
        try {
            return rbw_mode(argc, argv);
        } catch (const std::exception& e) {
            std::printf("FAILED with exception: %s\n", e.what());
            return 2;
        }
    }
    try {
        cpu_checks();
        if (!cpu_only) gpu_checks();
    } catch (const std::exception& e) {
        std::printf("FAILED with exception: %s\n", e.what());
        return 2;
    }
    std::printf(failures ? "\n%d check(s) FAILED\n" : "\nall checks passed%.0d\n", failures);
    return failures ? 1 : 0;
}
