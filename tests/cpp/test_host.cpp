// Tests of the C++ host mirror (include/wrq.hpp).  `--cpu`: everything that needs no device
// (token schedule against the literal expectations of src/runtime/infer/rnn.rs:362-569,
// op-build shape errors, the on-disk form of packed matrices against RFC 8949's examples).  Without flag: the same API driving the GPU, checked against a
// float64 product on host-dequantised weights.
#include <cmath>
#include <cstdio>
#include <chrono>
#include <cstdlib>
#include <fstream>
#include <random>

#include "../../include/wrq.hpp"
#include "../../include/wrq_serde.hpp"
#include "../../include/wrq_loader.hpp"

using namespace wrq;

static int failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);     \
            failures++;                                                     \
        }                                                                   \
    } while (0)

using Opt = std::optional<RnnOption>;
static const Opt NONE = std::nullopt, LAST = RnnOption::Last, FULL = RnnOption::Full;

static bool same(const RnnInfo &info, std::vector<std::pair<size_t, Opt>> want) {
    if (info.batches.size() != want.size()) return false;
    for (size_t i = 0; i < want.size(); i++)
        if (info.batches[i].len != want[i].first || info.batches[i].option != want[i].second) return false;
    return true;
}

static void test_run_iter() { // rnn.rs:362-454
    RnnInput run({{139, RnnOption::Last}, {1, RnnOption::Last}, {0, RnnOption::Full}, {65, RnnOption::Full}}, 128);
    auto it = run.iter();
    EXPECT(same(it.next(), {{65, NONE}, {1, LAST}, {0, FULL}, {62, FULL}}));
    EXPECT(same(it.next(), {{60, NONE}, {1, LAST}, {0, FULL}, {3, FULL}}));
    EXPECT(same(it.next(), {{14, LAST}, {1, LAST}, {0, FULL}, {1, FULL}}));
    EXPECT(same(it.next(), {{1, LAST}, {1, LAST}, {0, FULL}, {1, FULL}}));
    EXPECT(same(it.next(), {{1, LAST}, {1, LAST}, {0, FULL}, {1, FULL}}));
}

static void test_advance() { // rnn.rs:456-507
    RnnInput run({{139, RnnOption::Last}, {1, RnnOption::Last}, {0, RnnOption::Full}, {65, RnnOption::Full}}, 128);
    run.step();
    EXPECT(same(run.iter().next(), {{61, NONE}, {0, LAST}, {0, FULL}, {3, FULL}}));
    RnnInput again({{61, RnnOption::Last}, {1, RnnOption::Last}, {0, RnnOption::Full}, {3, RnnOption::Full}}, 128);
    EXPECT(same(again.iter().next(), {{60, NONE}, {1, LAST}, {0, FULL}, {3, FULL}}));
}

static void test_redirect() { // rnn.rs:509-569
    RnnInput run({{61, RnnOption::Last}, {0, RnnOption::Last}, {0, RnnOption::Full}, {3, RnnOption::Full}}, 128);
    auto r = run.iter().next().redirect();
    EXPECT((r.headers == std::vector<size_t>{60, 61, 62, 63}));
    EXPECT((r.inputs == std::vector<std::pair<size_t, size_t>>{{0, 61}, {61, 61}, {61, 61}, {61, 64}}));
    EXPECT((r.outputs == std::vector<std::pair<size_t, size_t>>{{0, 1}, {1, 1}, {1, 1}, {1, 4}}));
    std::vector<RnnInput::Batch> eight;
    for (int rep = 0; rep < 2; rep++)
        for (size_t n : {11, 8, 9, 4}) eight.push_back({n, RnnOption::Last});
    RnnInput run2(eight, 32);
    auto r2 = run2.iter().next().redirect();
    EXPECT((r2.headers == std::vector<size_t>{15, 31}));
    EXPECT((r2.inputs == std::vector<std::pair<size_t, size_t>>{{0, 4}, {4, 8}, {8, 12}, {12, 16}, {16, 20}, {20, 24}, {24, 28}, {28, 32}}));
    EXPECT((r2.outputs == std::vector<std::pair<size_t, size_t>>{{0, 0}, {0, 0}, {0, 0}, {0, 1}, {1, 1}, {1, 1}, {1, 1}, {1, 2}}));
}

static void test_schedule_of_the_configs() {
    // config 4: 512-token prompt in chunks of 128, then decode -> T = 128 x 4 (chunk kernels), then T = 1
    RnnInput c4({{512, RnnOption::Last}}, 128);
    for (int i = 0; i < 4; i++) {
        auto info = c4.iter().next();
        EXPECT(info.num_token() == 128 && turbo(info.num_token()));
        c4.step();
    }
    EXPECT(c4.iter().next().num_token() == 0);
    // token_chunk_size is rounded up to a multiple of 32 (rnn.rs:203-212); a 40-token prompt runs 32 + 8
    RnnInput odd({{40, RnnOption::Last}}, 33);
    EXPECT(odd.token_chunk_size() == 64);
    EXPECT(odd.iter().next().num_token() == 32);
    odd.step();
    EXPECT(odd.iter().next().num_token() == 8 && !turbo(8));
    EXPECT(turbo(32) && turbo(256) && !turbo(1) && !turbo(31));
}

static void test_build_time_errors() {
    // op constructors fail like the reference's: TensorErrorKind::Shape(got, want)
    const uint32_t K = 256, R = 8;
    auto fake = reinterpret_cast<void *>(0x10000);
    auto w = TensorGpu<uint8_t>::wrap(fake, Shape(K, R, 1, 1));
    auto mm = TensorGpu<f16>::wrap(fake, Shape(2 * K * R / 128, 1, 1, 1));
    auto x = TensorGpu<f16>::wrap(fake, Shape(K, 1, 1, 1));
    auto out = TensorGpu<f16>::wrap(fake, Shape(R, 1, 1, 1));
    bool threw = false;
    try {
        auto bad = TensorGpu<f16>::wrap(fake, Shape(7, 1, 1, 1));
        TensorOp::matmul_vec_int8(w, bad, TensorGpuView<f16>(x), TensorGpuView<f16>(out), Activation::None, false);
    } catch (const TensorError &e) {
        threw = e.status == WRQ_ERR_SHAPE && std::string(e.what()) == "tensor shape not match: (7, 1, 1, 1) vs. (32, 1, 1, 1)";
    }
    EXPECT(threw);
    threw = false;
    try {
        auto x2 = TensorGpu<f16>::wrap(fake, Shape(K, 2, 1, 1));
        TensorOp::matmul_vec_int8(w, mm, TensorGpuView<f16>(x2), TensorGpuView<f16>(out), Activation::None, false);
    } catch (const TensorError &e) {
        threw = e.status == WRQ_ERR_SHAPE;
    }
    EXPECT(threw);
    threw = false;
    try {
        view_of(x, {{{0, K}, {0, 2}, {0, 1}, {0, 1}}}); // slice past the parent
    } catch (const TensorError &e) {
        threw = e.status == WRQ_ERR_SHAPE;
    }
    EXPECT(threw);
    // a well-formed op builds without touching a device
    auto ok = TensorOp::matmul_vec_int8(w, mm, TensorGpuView<f16>(x), TensorGpuView<f16>(out), Activation::SquaredRelu, true);
    EXPECT(ok.kind() == TensorOp::Kind::Atom);
    EXPECT(TensorOp::INT8_BLOCK_SIZE == 128 && TensorOp::NF4_BLOCK_SIZE == 64);
    EXPECT(float4_quant().size() == 16 && float4_quant()[7] == 0.0f);
    {   // SF4 table (src/tensor/matrix.rs:29-44): nu = 5, values from scipy.stats.t.ppf
        const auto sf4 = float4_quant_student(5.0);
        EXPECT(sf4.size() == 16 && sf4[0] == -1.0f && sf4[7] == 0.0f && sf4[15] == 1.0f);
        EXPECT(std::fabs(sf4[1] - -0.62778056f) < 2e-7 && std::fabs(sf4[2] - -0.454736f) < 2e-7);
        for (int i = 1; i < 16; i++) EXPECT(sf4[i] > sf4[i - 1]);
    }
}

// ------------------------------------------------------------------ GPU

static uint16_t to_h(float f) { // round to nearest even, normal range only (test data)
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    int32_t e = (int32_t)((x >> 23) & 0xff) - 127 + 15;
    uint32_t m = x & 0x7fffffu;
    if (e <= 0) return (uint16_t)sign;
    uint32_t r = ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}
static float from_h(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu;
    if (e == 0) return (sign ? -1.0f : 1.0f) * std::ldexp((float)m, -24);
    uint32_t bits = sign | ((e + 112u) << 23) | (m << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

static void test_gpu_layer() {
    check(wrq_init());
    const uint32_t C = 512, H = 1024, T = 1;
    std::mt19937 rng(42);
    std::normal_distribution<float> nw(0.0f, 0.02f), nx(0.0f, 1.0f);
    auto rand_h = [&](size_t n, std::normal_distribution<float> &d) {
        std::vector<f16> v(n);
        for (auto &e : v) e.bits = to_h(d(rng));
        return v;
    };
    Queue queue;
    // five [C, C] products reading slices of one [C, T, 5] tensor, as v6 does, plus ffn.key with squared ReLU
    std::vector<std::vector<f16>> wh;
    std::vector<Matrix> mats;
    for (int j = 0; j < 4; j++) {
        wh.push_back(rand_h((size_t)C * C, nw));
        auto t = TensorGpu<f16>::from_data(Shape(C, C, 1, 1), wh.back());
        mats.push_back(j % 2 ? Matrix::quant_nf4(t, queue) : Matrix::quant_u8(t, queue));
    }
    wh.push_back(rand_h((size_t)C * H, nw));
    mats.push_back(Matrix::quant_u8(TensorGpu<f16>::from_data(Shape(C, H, 1, 1), wh.back()), queue));
    auto sx_h = rand_h((size_t)C * T * 5, nx);
    auto sx = TensorGpu<f16>::from_data(Shape(C, T, 5, 1), sx_h);
    std::vector<TensorGpu<float>> outs;
    std::vector<TensorOp> ops;
    for (uint32_t j = 0; j < 4; j++) {
        outs.push_back(TensorGpu<float>::init(Shape(C, T, 1, 1)));
        ops.push_back(mats[j].matmul_op(view_of(sx, {{{0, C}, {0, T}, {j + 1, j + 2}, {0, 1}}}), TensorGpuView<float>(outs[j]),
                                        Activation::None, turbo(T)));
    }
    auto ffn = TensorGpu<f16>::init(Shape(H, T, 1, 1));
    ops.push_back(TensorOp::Sep());
    ops.push_back(mats[4].matmul_op(view_of(sx, {{{0, C}, {0, T}, {0, 1}, {0, 1}}}), TensorGpuView<f16>(ffn), Activation::SquaredRelu,
                                    turbo(T)));
    queue.submit(TensorOp::List(ops));
    queue.sync();

    // host check: dequantise the packed bytes the device produced, multiply in double
    auto close = [](double a, double b) { return std::fabs(a - b) <= std::max(2e-3, 2e-3 * std::max(std::fabs(a), std::fabs(b))); };
    for (uint32_t j = 0; j < 5; j++) {
        const uint32_t R = j < 4 ? C : H;
        const auto wb = mats[j].w.back();
        const auto sb = mats[j].m.back();
        std::vector<double> got;
        if (j < 4)
            for (float v : outs[j].back()) got.push_back(v);
        else
            for (f16 v : ffn.back()) got.push_back(from_h(v.bits));
        const uint32_t slice = j < 4 ? j + 1 : 0;
        int bad = 0;
        for (uint32_t r = 0; r < R; r++) {
            double acc = 0;
            for (uint32_t k = 0; k < C; k++) {
                const size_t e = (size_t)r * C + k;
                double wv;
                if (mats[j].kind == Matrix::Kind::Int8) {
                    const double mn = from_h(sb[2 * (e / 128)].bits), mx = from_h(sb[2 * (e / 128) + 1].bits);
                    wv = wb[e] / 255.0 * (mx - mn) + mn;
                } else {
                    const uint8_t byte = wb[e / 2];
                    const int nib = (e & 1) ? byte >> 4 : byte & 15;
                    wv = (double)float4_quant()[nib] * from_h(sb[e / 64].bits);
                }
                acc += wv * from_h(sx_h[(size_t)slice * C * T + k].bits);
                // the packed value stays close to the source weight
                if (k == 0 && r == 0) EXPECT(std::fabs(wv - from_h(wh[j][e].bits)) < 0.02);
            }
            if (j == 4) acc = acc > 0 ? acc * acc : 0.0;
            bad += !close(acc, got[r]);
        }
        EXPECT(bad == 0);
    }
}

// The head (src/runtime/v6.rs:982-987): an f16 matrix behind the same Matrix interface, one token.
static void test_gpu_head() {
    check(wrq_init());
    const uint32_t C = 512, V = 2048;
    std::mt19937 rng(7);
    std::normal_distribution<float> nw(0.0f, 0.02f), nx(0.0f, 1.0f);
    std::vector<f16> wh((size_t)C * V), xh(C);
    for (auto &e : wh) e.bits = to_h(nw(rng));
    for (auto &e : xh) e.bits = to_h(nx(rng));
    Queue queue;
    const Matrix head = Matrix::fp16(TensorGpu<f16>::from_data(Shape(C, V, 1, 1), wh));
    auto x = TensorGpu<f16>::from_data(Shape(C, 1, 1, 1), xh);
    auto out = TensorGpu<float>::init(Shape(V, 1, 1, 1));
    queue.submit(head.matmul_op(TensorGpuView<f16>(x), TensorGpuView<float>(out), Activation::None, turbo(1)));
    queue.sync();
    const auto got = out.back();
    int bad = 0;
    for (uint32_t r = 0; r < V; r++) {
        double acc = 0;
        for (uint32_t k = 0; k < C; k++) acc += (double)from_h(wh[(size_t)r * C + k].bits) * from_h(xh[k].bits);
        bad += std::fabs(acc - got[r]) > std::max(2e-3, 2e-3 * std::fabs(acc));
    }
    EXPECT(bad == 0);
    bool threw = false;
    try {
        auto wrong = TensorGpu<float>::init(Shape(V + 4, 1, 1, 1));
        head.matmul_op(TensorGpuView<f16>(x), TensorGpuView<float>(wrong), Activation::None, false);
    } catch (const TensorError &e) {
        threw = e.status == WRQ_ERR_SHAPE;
    }
    EXPECT(threw);
}

// The ops between the products through the same Queue: layer norm against its closed form, the
// literal buffer of the reference's test_blit (src/tensor/ops.rs:3302-3336), a rejected shape.
static void test_gpu_layer_ops() {
    check(wrq_init());
    const uint32_t C = 1000, T = 3;
    std::mt19937 rng(11);
    std::uniform_real_distribution<float> ux(-5.0f, 5.0f), uw(-0.5f, 0.5f);
    std::vector<float> xh((size_t)C * T);
    std::vector<f16> wh(C), bh(C);
    for (auto &e : xh) e = ux(rng);
    for (auto &e : wh) e.bits = to_h(uw(rng));
    for (auto &e : bh) e.bits = to_h(uw(rng));
    Queue queue;
    auto x = TensorGpu<float>::from_data(Shape(C, T, 1, 1), xh);
    auto w = TensorGpu<f16>::from_data(Shape(C, 1, 1, 1), wh);
    auto b = TensorGpu<f16>::from_data(Shape(C, 1, 1, 1), bh);
    queue.submit(TensorOp::layer_norm(w, b, x, 1.0e-5f));
    queue.sync();
    const auto got = x.back();
    int bad = 0;
    for (uint32_t t = 0; t < T; t++) {
        double mean = 0, var = 0;
        for (uint32_t i = 0; i < C; i++) mean += xh[t * C + i];
        mean /= C;
        for (uint32_t i = 0; i < C; i++) var += (xh[t * C + i] - mean) * (xh[t * C + i] - mean);
        var /= C;
        for (uint32_t i = 0; i < C; i++) {
            const double want = (xh[t * C + i] - mean) / std::sqrt(var + 1.0e-5) * from_h(wh[i].bits) + from_h(bh[i].bits);
            bad += std::fabs(want - got[t * C + i]) > std::max(1e-3, 1e-3 * std::fabs(want));
        }
    }
    EXPECT(bad == 0);

    auto out = TensorGpu<float>::from_data(Shape(4, 3, 2, 1), std::vector<float>(24, 0.0f));
    std::vector<float> a(8), c(4);
    for (int i = 0; i < 8; i++) a[i] = (float)i;
    for (int i = 0; i < 4; i++) c[i] = (float)(8 + i);
    auto in0 = TensorGpu<float>::from_data(Shape(4, 1, 2, 1), a);
    auto in1 = TensorGpu<float>::from_data(Shape(4, 1, 1, 1), c);
    queue.submit(TensorOp::blit(TensorGpuView<float>(in0), view_of(out, {{{0, 4}, {1, 2}, {0, 2}, {0, 1}}})));
    queue.submit(TensorOp::blit(TensorGpuView<float>(in1), view_of(out, {{{0, 4}, {2, 3}, {1, 2}, {0, 1}}})));
    queue.sync();
    const std::vector<float> want = {0, 0, 0, 0, 0, 1, 2, 3, 0, 0, 0, 0, 0, 0, 0, 0, 4, 5, 6, 7, 8, 9, 10, 11};
    EXPECT(out.back() == want);

    // rows of unit length after l2_norm (src/tensor/ops.rs:642-700), k (1 + (a - 1) p) after control_k_v7 (:1800-1858)
    {
        std::vector<float> rows(64 * 5), av(64 * 5, 0.25f);
        for (auto &e : rows) e = ux(rng);
        std::vector<f16> ph(64);
        for (auto &e : ph) e.bits = to_h(0.5f);
        auto xr = TensorGpu<float>::from_data(Shape(64, 5, 1, 1), rows);
        auto kr = TensorGpu<float>::from_data(Shape(64, 5, 1, 1), rows);
        auto ar = TensorGpu<float>::from_data(Shape(64, 5, 1, 1), av);
        auto pr = TensorGpu<f16>::from_data(Shape(64, 1, 1, 1), ph);
        queue.submit(TensorOp::l2_norm(xr, 1.0e-12f));
        queue.submit(TensorOp::control_k_v7(pr, TensorGpuView<float>(ar), TensorGpuView<float>(kr)));
        queue.sync();
        const auto unit = xr.back(), kc = kr.back();
        int off = 0;
        for (int t = 0; t < 5; t++) {
            double sq = 0, in = 0;
            for (int i = 0; i < 64; i++) sq += (double)unit[t * 64 + i] * unit[t * 64 + i], in += (double)rows[t * 64 + i] * rows[t * 64 + i];
            off += std::fabs(sq - 1.0) > 1e-5;
            for (int i = 0; i < 64; i++) off += std::fabs(unit[t * 64 + i] - rows[t * 64 + i] / std::sqrt(in)) > 1e-6;
            for (int i = 0; i < 64; i++) off += std::fabs(kc[t * 64 + i] - rows[t * 64 + i] * 0.625) > 1e-6 * std::max(1.0, (double)std::fabs(rows[t * 64 + i]));
        }
        EXPECT(off == 0);
    }

    bool threw = false;
    try {
        queue.submit(TensorOp::transpose(TensorGpuView<float>(in0), TensorGpuView<float>(out)));
    } catch (const TensorError &e) {
        threw = e.status == WRQ_ERR_SHAPE;
    }
    EXPECT(threw);
}


// The ops of the v4 / v5 / v7 layers and of the loader: a mis-shaped operand is refused with the reference's
// shape error when the op is submitted, before anything is launched (no device needed).
static void test_layer_op_shape_errors() {
    auto fake = reinterpret_cast<void *>(0x10000);
    const uint32_t S = 64, H = 2, A = 3, B = 2, C = S * H;
    auto cursors = TensorGpu<uint32_t>::wrap(fake, Shape(A, 1, 1, 1));
    auto heads = TensorGpu<f16>::wrap(fake, Shape(S, H, A, 1));
    auto heads32 = TensorGpu<float>::wrap(fake, Shape(S, H, A, 1));
    auto n4 = TensorGpu<f16>::wrap(fake, Shape(S, H, A, 4)), n3 = TensorGpu<f16>::wrap(fake, Shape(S, H, A, 3));
    auto u = TensorGpu<f16>::wrap(fake, Shape(S, H, 1, 1));
    auto chan = TensorGpu<f16>::wrap(fake, Shape(C, 1, 1, 1));
    auto decay = TensorGpu<float>::wrap(fake, Shape(S, H, 1, 1)), decay_t = TensorGpu<float>::wrap(fake, Shape(S, H, A, 1));
    auto flat = TensorGpu<f16>::wrap(fake, Shape(C, A, 1, 1)), flat2 = TensorGpu<f16>::wrap(fake, Shape(C, A + 1, 1, 1));
    auto vec32 = TensorGpu<float>::wrap(fake, Shape(C, 1, 1, 1));
    auto state = TensorGpu<float>::wrap(fake, Shape(C, S + 2, B, 1));
    const auto att = view_of(state, {{{0, C}, {0, S + 1}, {0, B}, {0, 1}}}), ffn = view_of(state, {{{0, C}, {S + 1, S + 2}, {0, B}, {0, 1}}});
    auto factor = TensorGpu<float>::wrap(fake, Shape(4, 1, 1, 1));
    Queue queue;
    const std::pair<const char *, TensorOp> bad[] = {
        {"time_mix_v4", TensorOp::time_mix_v4(cursors, vec32, vec32, att, flat, flat, flat, flat)},               // the v4 state has 4 rows
        {"time_mix_v5", TensorOp::time_mix_v5(cursors, decay_t, decay, att, heads32, heads32, heads32, heads32)}, // a decay per token is v6's
        {"time_mix_v6", TensorOp::time_mix_v6(cursors, decay, decay, att, heads32, heads32, heads32, heads32)},   // a decay per channel is v5's
        {"time_mix_v7", TensorOp::time_mix_v7(cursors, att, heads, heads, n3, heads)},
        {"time_first_v7", TensorOp::time_first_v7(chan, heads, n4, heads)},
        {"control_k_v7", TensorOp::control_k_v7(u, TensorGpuView<f16>(flat), TensorGpuView<f16>(flat))},
        {"channel_mix_v7", TensorOp::channel_mix_v7(cursors, att, flat, flat)},                                  // the feed-forward state is one row
        {"l2_norm", TensorOp::l2_norm(n4, 1e-12f)},
        {"rms_norm", TensorOp::rms_norm(u, u, flat, 1e-5f)},
        {"broadcast", TensorOp::broadcast(TensorGpuView<f16>(u), TensorGpuView<f16>(flat))},
        {"blend", TensorOp::blend(factor, flat, flat2)},
        {"blend_lora", TensorOp::blend_lora(factor, TensorGpuView<f16>(flat), TensorGpuView<f16>(flat), TensorGpuView<f16>(flat))},
    };
    for (const auto &kv : bad) {
        bool threw = false;
        try {
            queue.submit(kv.second);
        } catch (const TensorError &e) {
            threw = e.status == WRQ_ERR_SHAPE && std::string(e.what()).find(kv.first) == 0;
        }
        if (!threw) std::printf("not refused: %s\n", kv.first);
        EXPECT(threw);
    }
    // a state view without slots (or, for token_shift, without rows) leaves the cursors nothing to be clamped into
    const auto no_slots = view_of(state, {{{0, C}, {0, S + 1}, {0, 0}, {0, 1}}}), no_slots_ffn = view_of(state, {{{0, C}, {S + 1, S + 2}, {0, 0}, {0, 1}}});
    const auto no_rows = view_of(state, {{{0, C}, {0, 0}, {0, B}, {0, 1}}});
    const auto mix = TensorGpuView<f16>(chan);
    const std::pair<const char *, TensorOp> empty_state[] = {
        {"token_shift", TensorOp::token_shift(cursors, mix, no_slots_ffn, flat, flat, false)},
        {"token_shift", TensorOp::token_shift(cursors, mix, no_rows, flat, flat, false)},
        {"channel_mix", TensorOp::channel_mix(cursors, no_slots_ffn, flat, flat, flat)},
        {"channel_mix_v7", TensorOp::channel_mix_v7(cursors, no_slots_ffn, flat, flat)},
        {"time_mix_v5", TensorOp::time_mix_v5(cursors, decay, decay, no_slots, heads32, heads32, heads32, heads32)},
        {"time_mix_v6", TensorOp::time_mix_v6(cursors, decay_t, decay, no_slots, heads32, heads32, heads32, heads32)},
        {"time_mix_v7", TensorOp::time_mix_v7(cursors, no_slots, heads, heads, n4, heads)},
    };
    for (const auto &kv : empty_state) {
        bool threw = false;
        try {
            queue.submit(kv.second);
        } catch (const TensorError &e) {
            threw = e.status == WRQ_ERR_SHAPE && std::string(e.what()).find(kv.first) == 0;
        }
        if (!threw) std::printf("empty state not refused: %s\n", kv.first);
        EXPECT(threw);
    }
    (void)ffn;
}

// ---------------------------------------------------------------- on-disk form of a Matrix

static std::vector<uint8_t> hex(const char *s) {
    std::vector<uint8_t> out;
    for (; s[0] && s[1]; s += 2) {
        unsigned v = 0;
        std::sscanf(s, "%2x", &v);
        out.push_back((uint8_t)v);
    }
    return out;
}

// The items the format is made of, against the examples of RFC 8949, Appendix A.
static void test_cbor_items() {
    const std::pair<uint64_t, const char *> ints[] = {{0, "00"}, {1, "01"}, {10, "0a"}, {23, "17"}, {24, "1818"}, {25, "1819"}, {100, "1864"},
                                                      {1000, "1903e8"}, {1000000, "1a000f4240"}, {1000000000000ull, "1b000000e8d4a51000"},
                                                      {18446744073709551615ull, "1bffffffffffffffff"}};
    for (const auto &kv : ints) {
        serde::Writer w;
        w.uint(kv.first);
        EXPECT(w.out == hex(kv.second));
        const auto bytes = hex(kv.second);
        serde::Reader r(bytes.data(), bytes.size());
        EXPECT(r.uint() == kv.first && r.remaining() == 0);
    }
    {
        serde::Writer w;
        const uint8_t b[4] = {1, 2, 3, 4};
        w.bytes(b, 4); // h'01020304'
        EXPECT(w.out == hex("4401020304"));
        serde::Writer e;
        e.bytes(b, 0); // h''
        EXPECT(e.out == hex("40"));
    }
    {
        serde::Writer w;
        w.text("IETF");
        EXPECT(w.out == hex("6449455446"));
        serde::Writer e;
        e.text("");
        EXPECT(e.out == hex("60"));
    }
    {
        serde::Writer w; // [1, 2, 3]
        w.array(3), w.uint(1), w.uint(2), w.uint(3);
        EXPECT(w.out == hex("83010203"));
        serde::Writer l; // [1 .. 25]
        l.array(25);
        for (int i = 1; i <= 25; i++) l.uint(i);
        EXPECT(l.out == hex("98190102030405060708090a0b0c0d0e0f101112131415161718181819"));
    }
    {
        serde::Writer w; // {"a": 1, "b": [2, 3]}
        w.map(2), w.text("a"), w.uint(1), w.text("b"), w.array(2), w.uint(2), w.uint(3);
        EXPECT(w.out == hex("a26161016162820203"));
        // the same value with open-ended containers: {_ "a": 1, "b": [_ 2, 3]}
        for (const char *form : {"a26161016162820203", "bf61610161629f0203ffff"}) {
            const auto bytes = hex(form);
            serde::Reader r(bytes.data(), bytes.size());
            std::vector<uint64_t> seen;
            std::string keys;
            r.each(5, "a map", [&](uint64_t) {
                keys += r.text();
                if (keys == "a") seen.push_back(r.uint());
                else r.each(4, "an array", [&](uint64_t) { seen.push_back(r.uint()); });
            });
            EXPECT(keys == "ab" && seen == (std::vector<uint64_t>{1, 2, 3}) && r.remaining() == 0);
        }
    }
}

static void test_matrix_blob() {
    using serde::MatrixBlob;
    using serde::TensorBlob;
    // one tensor, written out by hand from the rules: map(2) "shape" [2, 300, 1, 1] "data" h'0a0b'
    {
        serde::Writer w;
        serde::write(w, TensorBlob{Shape(2, 300, 1, 1), {0x0a, 0x0b}});
        EXPECT(w.out == hex("a2" "657368617065" "84" "02" "19012c" "01" "01" "6464617461" "42" "0a0b"));
    }
    std::mt19937 rng(3);
    auto blob = [&](Shape s, size_t elem) {
        TensorBlob t{s, std::vector<uint8_t>(s.len() * elem)};
        for (auto &b : t.data) b = (uint8_t)rng();
        return t;
    };
    MatrixBlob i8{Matrix::Kind::Int8, blob(Shape(128, 2, 1, 1), 1), blob(Shape(4, 1, 1, 1), 2), {}};
    MatrixBlob f4{Matrix::Kind::Fp4, blob(Shape(64, 2, 1, 1), 1), blob(Shape(4, 1, 1, 1), 2), blob(Shape(16, 1, 1, 1), 4)};
    MatrixBlob h{Matrix::Kind::Fp16, blob(Shape(8, 3, 1, 1), 2), {}, {}};
    for (const MatrixBlob *mb : {&i8, &f4, &h}) {
        const auto bytes = serde::to_vec(*mb);
        EXPECT(serde::from_slice(bytes.data(), bytes.size()) == *mb);
    }
    // the head of an Int8 matrix: {"Int8": {"w": {"shape": [128, 2, 1, 1], "data": h'(256 bytes)...
    const auto bytes = serde::to_vec(i8);
    const auto head = hex("a1" "64496e7438" "a2" "6177" "a2" "657368617065" "84" "1880" "02" "01" "01" "6464617461" "590100");
    EXPECT(bytes.size() > head.size() && std::equal(head.begin(), head.end(), bytes.begin()));
    EXPECT(bytes.size() == head.size() + 256 + hex("616d" "a2" "657368617065" "84" "04" "01" "01" "01" "6464617461" "48").size() + 8);
    // `Nf4` is read as `Fp4` (src/tensor/matrix.rs:88)
    auto alias = serde::to_vec(f4);
    EXPECT(alias[1] == 0x63 && alias[2] == 'F' && alias[3] == 'p' && alias[4] == '4');
    alias[2] = 'N', alias[3] = 'f';
    EXPECT(serde::from_slice(alias.data(), alias.size()) == f4);
    // the same matrix spelled with open-ended maps and arrays, the fields of the variant in another order and an
    // integer in a longer form than needed: read as the same value
    {
        serde::Writer w;
        auto open_tensor = [&](const TensorBlob &t) {
            w.out.push_back(0xbf);
            w.text("data"), w.bytes(t.data.data(), t.data.size());
            w.text("shape");
            w.out.push_back(0x9f);
            w.out.push_back(0x19), w.out.push_back(0x00), w.out.push_back((uint8_t)t.shape[0]); // 16-bit form of a small extent
            for (int d = 1; d < 4; d++) w.uint(t.shape[d]);
            w.out.push_back(0xff);
            w.out.push_back(0xff);
        };
        w.out.push_back(0xbf);
        w.text("Int8");
        w.out.push_back(0xbf);
        w.text("m"), open_tensor(i8.m);
        w.text("w"), open_tensor(i8.w);
        w.out.push_back(0xff);
        w.out.push_back(0xff);
        EXPECT(serde::from_slice(w.out.data(), w.out.size()) == i8);
    }
    // what must be refused: a cut file, another variant, scales that do not fit the weights, trailing bytes
    auto refused = [](const std::vector<uint8_t> &b) {
        try {
            serde::from_slice(b.data(), b.size());
        } catch (const serde::Error &) {
            return true;
        }
        return false;
    };
    EXPECT(refused(std::vector<uint8_t>(bytes.begin(), bytes.end() - 1)));
    EXPECT(refused(std::vector<uint8_t>(bytes.begin(), bytes.begin() + 40)));
    auto other = bytes;
    other[2] = 'J';
    EXPECT(refused(other));
    MatrixBlob wrong = i8;
    wrong.m = blob(Shape(6, 1, 1, 1), 2);
    EXPECT(refused(serde::to_vec(wrong)));
    auto longer = bytes;
    longer.push_back(0);
    EXPECT(refused(longer));
    EXPECT(!refused(bytes));
}

// A packed matrix written to its on-disk form and read back gives the same bytes and the same product.
static void test_gpu_matrix_round_trip() {
    check(wrq_init());
    const uint32_t C = 256, R = 384;
    std::mt19937 rng(5);
    std::normal_distribution<float> nw(0.0f, 0.02f), nx(0.0f, 1.0f);
    std::vector<f16> wh((size_t)C * R), xh(C);
    for (auto &e : wh) e.bits = to_h(nw(rng));
    for (auto &e : xh) e.bits = to_h(nx(rng));
    Queue queue;
    auto src = TensorGpu<f16>::from_data(Shape(C, R, 1, 1), wh);
    auto x = TensorGpu<f16>::from_data(Shape(C, 1, 1, 1), xh);
    const Matrix mats[3] = {Matrix::quant_u8(src, queue), Matrix::quant_nf4(src, queue), Matrix::fp16(src)};
    queue.sync();
    for (const Matrix &mx : mats) {
        const auto bytes = serde::to_vec(mx);
        const Matrix back = serde::matrix_from_slice(bytes.data(), bytes.size());
        EXPECT(back.kind == mx.kind);
        EXPECT(serde::to_blob(back) == serde::to_blob(mx));
        auto o0 = TensorGpu<float>::init(Shape(R, 1, 1, 1)), o1 = TensorGpu<float>::init(Shape(R, 1, 1, 1));
        queue.submit(mx.matmul_op(TensorGpuView<f16>(x), TensorGpuView<float>(o0), Activation::None, false));
        queue.submit(back.matmul_op(TensorGpuView<f16>(x), TensorGpuView<float>(o1), Activation::None, false));
        queue.sync();
        EXPECT(o0.back() == o1.back());
    }
}

// ------------------------------------------------------------------------- the loader

static std::vector<uint8_t> file_bytes(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    return std::vector<uint8_t>(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
}

// every f16 value survives the trip through f32, and the rounding of f32 -> f16 at its critical points
static void test_f16_conversions() {
    int bad = 0;
    for (uint32_t b = 0; b < 65536; b++) {
        f16 h;
        h.bits = (uint16_t)b;
        const bool nan = (b & 0x7c00) == 0x7c00 && (b & 0x3ff);
        const f16 r = f16_from_f32(f16_to_f32(h));
        bad += nan ? ((r.bits & 0x7c00) != 0x7c00 || !(r.bits & 0x3ff)) : r.bits != h.bits;
    }
    EXPECT(bad == 0);
    EXPECT(f16_to_f32(f16{0x3c00}) == 1.0f && f16_to_f32(f16{0x0001}) == 5.9604644775390625e-8f && f16_to_f32(f16{0xfbff}) == -65504.0f);
    EXPECT(f16_from_f32(1.0f + 0x1p-11f).bits == 0x3c00);          // tie: to even (down)
    EXPECT(f16_from_f32(1.0f + 0x1p-10f + 0x1p-11f).bits == 0x3c02); // tie: to even (up)
    EXPECT(f16_from_f32(1.0f + 0x1p-11f + 0x1p-20f).bits == 0x3c01); // above the tie
    EXPECT(f16_from_f32(65519.0f).bits == 0x7bff && f16_from_f32(65520.0f).bits == 0x7c00);
    EXPECT(f16_from_f32(0x1p-25f).bits == 0x0000 && f16_from_f32(0x1.000002p-25f).bits == 0x0001); // smallest subnormal's tie
    EXPECT(f16_from_f32(0x1.8p-24f).bits == 0x0002 && f16_from_f32(-0x1p-14f).bits == 0x8400);
    EXPECT(f16_from_f32(0x1.ffcp-15f).bits == 0x0400); // largest subnormal's upper neighbour rounds into the normal range
}

// argv: the model file and the folder of what a numpy reading of the same file expects
static void test_loader_host(const std::string &model_path, const std::string &dir) {
    SafeTensors model(model_path);
    Queue queue; // holds a stream handle only; the host-side functions never launch
    Loader loader(model, queue);
    EXPECT(model.contains("blocks.6.att.output.weight") && model.contains("blocks.6.ffn.value.weight") && model.contains("blocks.6.att.time_first"));
    EXPECT(!model.contains("blocks.7.att.output.weight") && model.names().size() == 3);
    EXPECT(model.shape("blocks.6.ffn.value.weight") == (std::vector<uint64_t>{256, 384}));
    EXPECT(loader.tensor_shape("blocks.6.ffn.value.weight") == Shape(384, 256, 1, 1)); // [out, in] -> x = in
    EXPECT(loader.tensor_shape("blocks.6.att.time_first") == Shape(64, 4, 1, 1));
    EXPECT(model.metadata().count("note") && model.metadata().at("note") == "a \"quoted\" word");
    for (const char *name : {"blocks.6.att.output.weight", "blocks.6.ffn.value.weight"}) {
        const auto got = loader.discounted(name, 0.5f);
        const auto want = file_bytes(dir + "/" + name + ".half.f16");
        EXPECT(want.size() == got.size() * 2 && std::memcmp(want.data(), got.data(), want.size()) == 0);
        const auto got3 = loader.discounted(name, 0.3f);
        const auto want3 = file_bytes(dir + "/" + name + ".x03.f16");
        EXPECT(want3.size() == got3.size() * 2 && std::memcmp(want3.data(), got3.data(), want3.size()) == 0);
    }
    bool threw = false;
    try {
        loader.discounted("blocks.6.att.time_first", 1.0f); // an f32 tensor
    } catch (const TensorError &e) {
        threw = e.status == WRQ_ERR_TYPE;
    }
    EXPECT(threw);
    threw = false;
    try {
        model.tensor("blocks.0.nothing");
    } catch (const LoaderError &) {
        threw = true;
    }
    EXPECT(threw);
    threw = false;
    try {
        SafeTensors cut(dir + "/cut.st"); // the same file without its last bytes
    } catch (const LoaderError &) {
        threw = true;
    }
    EXPECT(threw);
    threw = false;
    try {
        SafeTensors wraps(dir + "/wraps.st"); // extents 2^31 x 2^31 x 4 of F16: the byte size wraps to 0 and would match offsets [0, 0]
    } catch (const LoaderError &) {
        threw = true;
    }
    EXPECT(threw);
}

// Adapter plumbing on the host: which pattern counts, how a matrix name maps to the adapter's tensor names (loader.rs:328-386)
static void test_lora_host(const std::string &model_path, const std::string &dir) {
    SafeTensors model(model_path), adapter(dir + "/lora.st");
    Queue queue;
    EXPECT(Loader::lora_stem("blocks.6.att.output.weight") == "blocks.6.att.output");
    EXPECT(Loader::lora_stem("head.weight") == "head");
    float a = 0.0f;
    EXPECT(LoraBlend::full(0.25f).factor_of("blocks.6.att.output.weight", a) && a == 0.25f); // the last matching pattern counts
    EXPECT(LoraBlend::full(0.25f).factor_of("blocks.6.att.time_first", a) && a == 1.0f);     // only the nominal pattern matches
    EXPECT(!LoraBlend().add_layer(5, 0.5f).factor_of("blocks.6.att.output.weight", a));
    EXPECT(LoraBlend().add_layer(6, 0.5f).factor_of("blocks.6.ffn.value.weight", a) && a == 0.5f);
    Loader loader(model, queue, {Lora{&adapter, LoraBlend::full(0.5f)}});
    const auto ms = loader.lora_matrices("blocks.6.ffn.value.weight");
    EXPECT(ms.size() == 1 && ms[0].rank == 8 && ms[0].alpha == 0.5f && ms[0].x == "blocks.6.ffn.value.lora.0" && ms[0].y == "blocks.6.ffn.value.lora.1");
    EXPECT(loader.lora_matrices("blocks.6.att.output.weight").empty()); // the adapter file has no halves for it
    const auto vs = loader.lora_vectors("blocks.6.att.output.weight");
    EXPECT(vs.size() == 1 && vs[0].alpha == 0.5f); // ... but a whole tensor of that name
    EXPECT(loader.lora_vectors("blocks.6.ffn.value.weight").empty());
}

// An adapter blended in while loading: out = f16(alpha / rank * xa^T xb + w) for the low-rank halves, f16(alpha * v + w) for a
// whole tensor, with the discount in both factors; against numpy's float32 evaluation of the same expressions (one f16 ulp:
// the order of the rank-8 sum is free)
static void test_lora_gpu(const std::string &model_path, const std::string &dir) {
    SafeTensors model(model_path), adapter(dir + "/lora.st");
    Queue queue;
    Loader loader(model, queue, {Lora{&adapter, LoraBlend::full(0.5f)}});
    struct Case {
        const char *name, *tag;
        float discount;
    };
    for (const Case &c : {Case{"blocks.6.ffn.value.weight", ".lora.f16", 1.0f}, Case{"blocks.6.ffn.value.weight", ".lora_half.f16", 0.5f},
                          Case{"blocks.6.att.output.weight", ".lora.f16", 1.0f}, Case{"blocks.6.att.output.weight", ".lora_half.f16", 0.5f}}) {
        const TensorGpu<f16> t = c.discount == 1.0f ? loader.load_matrix_f16(c.name) : loader.load_matrix_f16_discount(c.name, c.discount);
        queue.sync();
        const auto got = t.back();
        const auto want = file_bytes(dir + "/" + c.name + c.tag);
        EXPECT(want.size() == got.size() * 2);
        int off = 0;
        for (size_t i = 0; i < got.size() && want.size() == got.size() * 2; i++) {
            f16 w;
            std::memcpy(&w.bits, want.data() + 2 * i, 2);
            const float g = f16_to_f32(got[i]), e = f16_to_f32(w);
            off += std::fabs(g - e) > 1e-3f * std::max(1.0f, std::fabs(e)) * 0.5f + 6e-8f ? 1 : 0; // half a per mille: an f16 ulp is 4.9e-4 relative
        }
        EXPECT(off == 0);
    }
    // packed through the same path: an Int8 matrix of the blended weights loads without error
    const Matrix mx = loader.load_matrix(std::string("blocks.6.ffn.value.weight"), Quant::Int8);
    queue.sync();
    EXPECT(mx.kind == Matrix::Kind::Int8);
}

// file -> discount -> pack on the device, against the packed bytes the CPU restatement gives for numpy's discount
static void test_loader_gpu(const std::string &model_path, const std::string &dir) {
    check(wrq_init());
    SafeTensors model(model_path);
    Queue queue;
    Loader loader(model, queue);
    const std::string name = "blocks.6.ffn.value.weight";
    struct Case {
        Quant quant;
        const char *tag;
    };
    for (const Case &c : {Case{Quant::Int8, "int8"}, Case{Quant::NF4, "nf4"}}) {
        const Matrix mx = loader.load_matrix_discount(name, c.quant, 0.5f);
        queue.sync();
        const serde::MatrixBlob blob = serde::to_blob(mx);
        EXPECT(blob.w.data == file_bytes(dir + "/" + name + "." + c.tag + ".w"));
        EXPECT(blob.m.data == file_bytes(dir + "/" + name + "." + c.tag + ".m"));
        EXPECT(blob.w.shape == (c.quant == Quant::Int8 ? Shape(384, 256, 1, 1) : Shape(192, 256, 1, 1)));
    }
    const Matrix plain = loader.load_matrix(name, Quant::None);
    const auto bytes = model.tensor(name);
    const auto back = plain.h.back();
    EXPECT(plain.kind == Matrix::Kind::Fp16 && back.size() * 2 == bytes.second && std::memcmp(back.data(), bytes.first, bytes.second) == 0);
    const Matrix sf4 = loader.load_matrix(name, Quant::SF4);
    queue.sync();
    EXPECT(sf4.kind == Matrix::Kind::Fp4 && sf4.q.back() == float4_quant_student(5.0));
}

// Timing of the loader on a model file (bench.py --loader): every 2-axis F16 tensor into an Int8 matrix,
// once as it is and once with a discount (the host-side f32 multiply and f16 rounding in between).
static int loader_bench(const std::string &model_path) {
    check(wrq_init());
    SafeTensors model(model_path);
    Queue queue;
    Loader loader(model, queue);
    std::vector<std::string> names;
    uint64_t bytes = 0;
    for (const auto &name : model.names())
        if (model.entry(name).dtype == "F16" && model.shape(name).size() == 2) names.push_back(name), bytes += model.tensor(name).second;
    for (int pass = 0; pass < 3; pass++) { // pass 0 warms the page cache and the library
        const bool discount = pass == 2;
        const auto t0 = std::chrono::steady_clock::now();
        for (const auto &name : names) {
            const Matrix mx = discount ? loader.load_matrix_discount(name, Quant::Int8, 0.5f) : loader.load_matrix(name, Quant::Int8);
            (void)mx;
        }
        queue.sync();
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        if (pass) std::printf("{\"loader\": \"%s\", \"matrices\": %zu, \"f16_bytes\": %llu, \"ms\": %.2f, \"GBps\": %.2f}\n", discount ? "int8 with discount" : "int8",
                              names.size(), (unsigned long long)bytes, ms, bytes / ms / 1e6);
    }
    return 0;
}

int main(int argc, char **argv) {
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu";
    if (argc > 2 && std::string(argv[1]) == "--loader-bench") {
        try {
            return loader_bench(argv[2]);
        } catch (const std::exception &e) {
            std::printf("FAIL: %s\n", e.what());
            return 1;
        }
    }
    if (argc > 3 && (std::string(argv[1]) == "--loader" || std::string(argv[1]) == "--loader-gpu")) {
        // the loader against a model file and its expectations, both written by tests/test_loader.py
        try {
            test_f16_conversions();
            test_loader_host(argv[2], argv[3]);
            test_lora_host(argv[2], argv[3]);
            if (std::string(argv[1]) == "--loader-gpu") {
                test_loader_gpu(argv[2], argv[3]);
                test_lora_gpu(argv[2], argv[3]);
            }
        } catch (const std::exception &e) {
            std::printf("FAIL: %s\n", e.what());
            failures++;
        }
        std::printf(failures ? "%d FAILED\n" : "host tests ok%.0d\n", failures);
        return failures ? 1 : 0;
    }
    test_run_iter();
    test_advance();
    test_redirect();
    test_schedule_of_the_configs();
    test_build_time_errors();
    test_layer_op_shape_errors();
    test_cbor_items();
    test_matrix_blob();
    if (!cpu_only) {
        try {
            test_gpu_layer();
            test_gpu_head();
            test_gpu_layer_ops();
            test_gpu_matrix_round_trip();
        } catch (const TensorError &e) {
            std::printf("FAIL: TensorError %d: %s\n", e.status, e.what());
            failures++;
        }
    }
    std::printf(failures ? "%d FAILED\n" : "host tests ok%.0d\n", failures);
    return failures ? 1 : 0;
}
