// Exercises the C++ classes the way the reference's own C++ tests do
// (tests_cpp/test_against_eigen1.cpp:70-213 of the reference: build a network from JSON,
// create and initialise the parameter tensor, run inference / forward / adjoint, compare with
// a plain evaluation on the host). Usage: test_cpp_api [--host]. With --host only the part
// that needs no GPU runs. Exit code 0 = all checks passed.
#include <qmlp/fused_network.h>
#include <qmlp/qmlp.h>
#include <qmlp/tmp_memory.h>
#include <qmlp/utils.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

using namespace qmlp;

static int failures = 0;
#define CHECK(cond)                                                            \
    do {                                                                       \
        if (!(cond)) {                                                         \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
            ++failures;                                                        \
        }                                                                      \
    } while (0)

static const char* SPEC = R"json({
    "num_inputs": 5, "num_outputs": 3,
    "activation_specification": ["qmlp/builtin-activations.json"],
    "encodings": [{"id": "Identity", "start_in": 0, "n_in": 5}],
    "network": [
        {"n_out": 20, "bias": true, "activation": "celu"},
        {"n_out": 3, "bias": false, "activation": "identity"}
    ]
})json";

static float halfToFloat(half h) { return static_cast<float>(h); }   // the host-side half is _Float16

static void hostPart()
{
    auto cfg = json::parse(SPEC);
    FusedNetwork net(cfg, ".");
    CHECK(net.channelsIn() == 5 && net.channelsOut() == 3 && net.numLayers() == 2);
    CHECK(net.numEncodings() == 1 && net.encoding(0)->id() == "Identity");
    // padded layout: W0 (32,16), W1 (16,32), then b0 (32)
    CHECK(net.networkParameterCount() == 32 * 16 + 16 * 32 + 32);
    CHECK(net.networkParameterPrecision(Tensor::INFERENCE) == Tensor::HALF);
    CHECK(net.networkParameterPrecision(Tensor::GRADIENTS) == Tensor::FLOAT);
    CHECK(net.forwardMemory(100, FusedNetwork::GRADIENTS_INPUT) == size_t(128) * 2 * (16 + 32 + 16));
    CHECK(FusedNetwork::MATRIX_SIZE == 16 && FusedNetwork::WARP_SIZE == 64);
    // views into a parameter buffer
    std::vector<half> dummy(net.networkParameterCount());
    Tensor w1 = net.networkParameter(1, false, dummy.data(), Tensor::HALF);
    CHECK(w1.ndim() == 2 && w1.size(0) == 16 && w1.size(1) == 32 && w1.stride(0) == 32);
    CHECK(static_cast<half*>(w1.rawPtr()) - dummy.data() == 32 * 16);
    Tensor b0 = net.networkParameter(0, true, dummy.data(), Tensor::HALF);
    CHECK(b0.ndim() == 1 && b0.size(0) == 32);
    bool thrown = false;
    try {
        auto bad = json::parse(SPEC);
        bad["num_outputs"] = 4;
        FusedNetwork n2(bad, ".");
    } catch (const configuration_error&) {
        thrown = true;
    }
    CHECK(thrown);
    // the kernels of this network compile for gfx950 without a device
    net.precompile(FusedNetwork::GRADIENTS_INPUT | FusedNetwork::GRADIENTS_NETWORK_WEIGHTS);

    // Which grids offer a slab key for sorting inference batches: a dense 32^4 grid with 8 fp16
    // features (16.8 MB) does, in 31 x 31 slabs of one cell over its box [1,3] x [0,4];
    // a 16-level hash grid whose dense levels are small offers one (32 x 32 slabs of its second and third coordinate
    // along a Z curve) when asked whether an order exists, never for a batch size (its sort costs more than it
    // gains); a small dense grid has none.
    {
        auto dense = EncodingFactory::Instance().create(json::parse(R"json({"id": "HashGrid", "start_in": 1, "n_in": 4,
            "n_levels": 1, "n_features_per_level": 8, "log2_hashmap_size": -1, "min_resolution": 32, "max_resolution": 32,
            "combination_mode": "concat", "bounding_box_min": [1, 0, 0, 0], "bounding_box_size": [2, 4, 1, 1],
            "parameter_precision": "half"})json"));
        kernel::PointOrderKey key{};
        CHECK(dense->pointOrderKey(key));
        CHECK(key.channel0 == 1 && key.channel1 == 2 && key.slabs0 == 31 && key.slabs1 == 31 && key.slabs2 == 1);
        CHECK(key.min0 == 1.f && key.min1 == 0.f && key.scale0 == 15.5f && key.scale1 == 7.75f);
        auto hashed = EncodingFactory::Instance().create(json::parse(R"json({"id": "HashGrid", "start_in": 0, "n_in": 3,
            "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 19, "min_resolution": 16, "max_resolution": 4096,
            "combination_mode": "concat", "bounding_box_min": [0, 0, 0], "bounding_box_size": [1, 1, 1]})json"));
        CHECK(hashed->pointOrderKey(key));
        CHECK(key.slabs0 == 1 && key.slabs1 == 32 && key.slabs2 == 32 && key.interleave12 == 1);
        CHECK(key.channel1 == 1 && key.channel2 == 2 && key.scale1 == 32.f && key.min2 == 0.f);
        CHECK(!hashed->pointOrderKey(key, 1 << 20) && !hashed->pointOrderKey(key, 1 << 24));
        auto small = EncodingFactory::Instance().create(json::parse(R"json({"id": "HashGrid", "start_in": 0, "n_in": 3,
            "n_levels": 1, "n_features_per_level": 2, "log2_hashmap_size": -1, "min_resolution": 64, "max_resolution": 64,
            "combination_mode": "concat", "bounding_box_min": [0, 0, 0], "bounding_box_size": [1, 1, 1]})json"));
        CHECK(!small->pointOrderKey(key));
        // a wide dense 3-D grid: 300 cells per coordinate in 30 slabs of 10 cells
        auto wide = EncodingFactory::Instance().create(json::parse(R"json({"id": "HashGrid", "start_in": 0, "n_in": 3,
            "n_levels": 1, "n_features_per_level": 2, "log2_hashmap_size": -1, "min_resolution": 301, "max_resolution": 301,
            "combination_mode": "concat", "bounding_box_min": [0, 0, 0], "bounding_box_size": [1, 1, 1]})json"));
        CHECK(wide->pointOrderKey(key));
        CHECK(key.slabs0 == 30 && key.slabs1 == 30 && key.scale0 == 30.f);
        // with a batch size the answer also weighs the gain: 4 gathered lines per point against
        // the 218 MB of the wide grid (1.7 M lines) need 10 M points, the 16.8 MB of the 4-D grid
        // (8 lines per point) 2^19
        CHECK(!wide->pointOrderKey(key, 1 << 22) && wide->pointOrderKey(key, 11 << 20));
        CHECK(dense->pointOrderKey(key, 1 << 19) && !dense->pointOrderKey(key, 1 << 18));
    }
}

static float celu(float x) { return x > 0 ? x : std::exp(x) - 1; }
static float celuAdjoint(float x, float adjz) { return x > 0 ? adjz : adjz * std::exp(x); }

static void gpuPart()
{
    auto cfg = json::parse(SPEC);
    auto net = std::make_shared<FusedNetwork>(cfg, ".");
    const int N = 777, CIN = 5, COUT = 3, H = 32, K = 16;
    const int P = net->networkParameterCount();

    Tensor params(net->networkParameterPrecision(Tensor::INFERENCE), {P});
    net->setNetworkParameter(params, Tensor::INFERENCE);
    std::default_random_engine rng(42);
    net->initializeInferenceParameters(rng);
    std::vector<half> hp(P);
    params.copyToHost(hp.data(), sizeof(half) * P);
    std::vector<float> p(P);
    for (int i = 0; i < P; ++i) p[i] = halfToFloat(hp[i]);
    {
        // the draw order of initializeInferenceParameters (src_cpp/src/fused_network.cpp:280-312 of
        // the reference): per layer the weight matrix row by row, then the bias, one engine,
        // U(-1/sqrt(padded fan-in), +1/sqrt(padded fan-in)) rounded to half
        std::default_random_engine again(42);
        std::vector<float> expected(P, 0.f);
        const int fanIn[2] = {K, H}, fanOut[2] = {H, K};
        const int weightStart[2] = {0, H * K}, biasStart[2] = {2 * H * K, -1};
        for (int layer = 0; layer < 2; ++layer) {
            const float bound = static_cast<float>(1.0f / std::sqrt(static_cast<double>(fanIn[layer])));
            std::uniform_real_distribution<float> distr(-bound, +bound);
            for (int i = 0; i < fanOut[layer] * fanIn[layer]; ++i)
                expected[weightStart[layer] + i] = halfToFloat(static_cast<half>(distr(again)));
            if (biasStart[layer] >= 0)
                for (int i = 0; i < fanOut[layer]; ++i) expected[biasStart[layer] + i] = halfToFloat(static_cast<half>(distr(again)));
        }
        int different = 0;
        for (int i = 0; i < P; ++i) different += p[i] != expected[i];
        CHECK(different == 0);
    }
    const float* W0 = p.data();            // (32, 16)
    const float* W1 = p.data() + H * K;    // (16, 32)
    const float* b0 = p.data() + 2 * H * K;

    std::vector<float> x(N * CIN), adjOut(N * COUT);
    std::uniform_real_distribution<float> uni(-1.f, 1.f);
    for (auto& v : x) v = uni(rng);
    for (auto& v : adjOut) v = uni(rng) / N;
    Tensor input(Tensor::FLOAT, {N, CIN}), output(Tensor::FLOAT, {N, COUT}), adjOutput(Tensor::FLOAT, {N, COUT});
    Tensor adjInput(Tensor::FLOAT, {N, CIN});
    input.copyFromHost(x.data(), sizeof(float) * x.size());
    adjOutput.copyFromHost(adjOut.data(), sizeof(float) * adjOut.size());
    adjInput.zero_();
    Tensor grads(net->networkParameterPrecision(Tensor::GRADIENTS), {P});
    grads.zero_();
    net->setNetworkParameter(grads, Tensor::GRADIENTS);

    // host evaluation in fp32
    std::vector<float> ref(N * COUT), refAdjIn(N * CIN, 0.f), refGrad(P, 0.f);
    for (int n = 0; n < N; ++n) {
        float pre[H], hid[H], dhid[H];
        for (int o = 0; o < H; ++o) {
            float a = b0[o];
            for (int k = 0; k < CIN; ++k) a += W0[o * K + k] * x[n * CIN + k];
            pre[o] = a;
            hid[o] = celu(a);
            dhid[o] = 0.f;
        }
        for (int o = 0; o < COUT; ++o) {
            float a = 0.f;
            for (int k = 0; k < H; ++k) a += W1[o * H + k] * hid[k];
            ref[n * COUT + o] = a;
            const float d = adjOut[n * COUT + o];
            for (int k = 0; k < H; ++k) {
                refGrad[H * K + o * H + k] += d * hid[k];
                dhid[k] += W1[o * H + k] * d;
            }
        }
        for (int o = 0; o < H; ++o) {
            const float d = celuAdjoint(pre[o], dhid[o]);
            refGrad[2 * H * K + o] += d;
            for (int k = 0; k < CIN; ++k) {
                refGrad[o * K + k] += d * x[n * CIN + k];
                refAdjIn[n * CIN + k] += W0[o * K + k] * d;
            }
        }
    }
    auto close = [](float a, float e) { return std::fabs(a - e) <= 1e-3f + 1e-2f * std::fabs(e); };

    net->inference(input, output, nullptr);
    std::vector<float> out(N * COUT);
    output.copyToHost(out.data(), sizeof(float) * out.size());
    int bad = 0;
    for (size_t i = 0; i < out.size(); ++i) bad += !close(out[i], ref[i]);
    CHECK(bad == 0);

    const int flags = FusedNetwork::GRADIENTS_INPUT | FusedNetwork::GRADIENTS_NETWORK_WEIGHTS;
    TmpMemory fwd(net->forwardMemory(input, flags));
    output.zero_();
    net->forward(input, output, fwd.get(), nullptr);
    output.copyToHost(out.data(), sizeof(float) * out.size());
    bad = 0;
    for (size_t i = 0; i < out.size(); ++i) bad += !close(out[i], ref[i]);
    CHECK(bad == 0);

    TmpMemory adj(net->adjointMemory(input, flags));
    net->adjoint(input, adjOutput, flags, adjInput, fwd.get(), adj.get(), nullptr);
    std::vector<float> adjIn(N * CIN), grad(P);
    adjInput.copyToHost(adjIn.data(), sizeof(float) * adjIn.size());
    grads.copyToHost(grad.data(), sizeof(float) * P);
    bad = 0;
    for (size_t i = 0; i < adjIn.size(); ++i) bad += !close(adjIn[i], refAdjIn[i]);
    CHECK(bad == 0);
    bad = 0;
    for (int i = 0; i < P; ++i) bad += !close(grad[i], refGrad[i]);
    CHECK(bad == 0);

    // gradients accumulate: a second adjoint call doubles them
    net->adjoint(input, adjOutput, flags, adjInput, fwd.get(), adj.get(), nullptr);
    grads.copyToHost(grad.data(), sizeof(float) * P);
    bad = 0;
    for (int i = 0; i < P; ++i) bad += !close(grad[i], 2 * refGrad[i]);
    CHECK(bad == 0);
    net->zeroGradients();
    grads.copyToHost(grad.data(), sizeof(float) * P);
    bad = 0;
    for (int i = 0; i < P; ++i) bad += grad[i] != 0.f;
    CHECK(bad == 0);
}

// Utils::fractionalPullpush (src_cpp/include/qmlp/utils.h:50-85 of the reference) on closed forms:
// one known pixel floods a power-of-two image, a full mask returns the data, and the data
// gradient under a full mask is the output gradient.
static void pullpushPart()
{
    const int B = 2, C = 3, S = 16;
    std::vector<float> mask(B * S * S, 0.f), data(B * C * S * S), out(B * C * S * S), adjOut(B * C * S * S);
    std::default_random_engine rng(7);
    std::uniform_real_distribution<float> uni(-1.f, 1.f);
    for (auto& v : data) v = uni(rng);
    for (auto& v : adjOut) v = uni(rng);
    for (int b = 0; b < B; ++b) mask[(b * S + 5) * S + 11] = 1.f;
    Tensor tMask(Tensor::FLOAT, {B, S, S}), tData(Tensor::FLOAT, {B, C, S, S}), tOut(Tensor::FLOAT, {B, C, S, S});
    tMask.copyFromHost(mask.data(), sizeof(float) * mask.size());
    tData.copyFromHost(data.data(), sizeof(float) * data.size());
    Utils::fractionalPullpush(tMask, tData, tOut, nullptr);
    tOut.copyToHost(out.data(), sizeof(float) * out.size());
    int bad = 0;
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c) {
            const float known = data[((b * C + c) * S + 5) * S + 11];
            for (int i = 0; i < S * S; ++i) bad += std::fabs(out[(b * C + c) * S * S + i] - known) > 1e-5f;
        }
    CHECK(bad == 0);

    std::fill(mask.begin(), mask.end(), 1.f);
    tMask.copyFromHost(mask.data(), sizeof(float) * mask.size());
    Utils::fractionalPullpush(tMask, tData, tOut, nullptr);
    tOut.copyToHost(out.data(), sizeof(float) * out.size());
    bad = 0;
    for (size_t i = 0; i < out.size(); ++i) bad += out[i] != data[i];
    CHECK(bad == 0);

    Tensor tAdjOut(Tensor::FLOAT, {B, C, S, S}), tAdjMask(Tensor::FLOAT, {B, S, S}), tAdjData(Tensor::FLOAT, {B, C, S, S});
    tAdjOut.copyFromHost(adjOut.data(), sizeof(float) * adjOut.size());
    tAdjMask.zero_();
    tAdjData.zero_();
    Utils::adjointFractionalPullpush(tMask, tData, tAdjOut, tAdjMask, tAdjData, nullptr);
    tAdjData.copyToHost(out.data(), sizeof(float) * out.size());
    bad = 0;
    for (size_t i = 0; i < out.size(); ++i) bad += out[i] != adjOut[i];
    CHECK(bad == 0);

    bool thrown = false;
    try {
        Tensor wide(Tensor::FLOAT, {B, 16, S, S}), wideOut(Tensor::FLOAT, {B, 16, S, S});
        Utils::fractionalPullpush(tMask, wide, wideOut, nullptr);
    } catch (const std::runtime_error&) {
        thrown = true;
    }
    CHECK(thrown);
}

int main(int argc, char** argv)
{
    const bool hostOnly = argc > 1 && std::strcmp(argv[1], "--host") == 0;
    try {
        QuickMLP::Instance().setLogLevel("error");
        hostPart();
        if (!hostOnly) {
            QuickMLP::Instance().checkHipAvailable();
            gpuPart();
            pullpushPart();
        }
    } catch (const std::exception& e) {
        std::printf("FAILED with exception: %s\n", e.what());
        return 2;
    }
    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
