// Passes of single layers through the nz:: API (Model::forward(), backward(), update()), timed on the host around a device
// synchronisation: Linear 4096 x 1024 -> 4096 + ReLU, and Conv2d 16 x 64 x 128 x 128 -> 128 (3x3, stride 1, pad 1)
// + ReLU with the reference's parameters (one weight copy per sample, per-pixel bias; src/Model.cu:244-263).
// Each layer twice: weights untouched between the passes (the fused layers keep the fp16 image of their weights),
// and weights rewritten before every pass (the image is rebuilt every time). The device is first kept busy for 1.5 s
// (after an idle period its power management takes about a second to settle, and whatever is measured first looks
// slow), then the two variants alternate three times and the median of each is reported. A third figure per layer is
// a whole training pass: forward(), backward() (the output gradient seeded with ones, as the reference's
// Model::backward does without a loss node) and update() with SGD. Prints one JSON line.
//   layer_bench [steps] [warmup]
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "NeuZephyr/Model.cuh"
#include "NeuZephyr/Optimizer.cuh"
#include "nzhip.h"

using namespace nz::nodes;
using namespace nz::nodes::io;

struct LinearLayer : nz::Model {
    InputNode input;
    LinearLayer(size_t batch, size_t in, size_t out) : input({batch, 1, in, 1}) { defaultOutput(ReLU(Linear(&input, out))); }
};

struct ConvLayer : nz::Model {
    InputNode input;
    ConvLayer(size_t n, size_t c, size_t h, size_t w, size_t o) : input({n, c, h, w}) {
        defaultOutput(ReLU(Conv2d(&input, o, 3, 3, 1, 1)));
    }
};

template <typename M>
static void fill(M& model, std::mt19937& gen, float scale) {
    std::uniform_real_distribution<float> u(-1.f, 1.f);
    std::vector<float> x(model.input.output->size());
    for (auto& v : x) v = u(gen);
    model.input.dataInject(x.begin(), x.end());
    for (auto* p : model.parameters()) {
        std::vector<float> v(p->output->size());
        for (auto& e : v) e = u(gen) * scale;
        p->dataInject(v.begin(), v.end());
    }
}

template <typename M>
static double timeForward(M& model, int steps, int warmup, bool touchWeights) {
    auto pass = [&] {
        if (touchWeights) (void)model.parameters()[0]->output->data();     // a writable pointer was handed out
        model.forward();
    };
    for (int i = 0; i < warmup; ++i) pass();
    nzhip_sync_all();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) pass();
    nzhip_sync_all();
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
}

template <typename M>
static void settle(M& model, double seconds) {
    const auto t0 = std::chrono::steady_clock::now();
    while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds) {
        for (int i = 0; i < 50; ++i) model.forward();
        nzhip_sync_all();
    }
}

// kept / rebuilt alternate three times; medians
template <typename M>
static void measure(M& model, int steps, int warmup, double& kept, double& rebuilt, unsigned long long& buildsInKeptLoops) {
    settle(model, 1.5);
    double k[3], r[3];
    buildsInKeptLoops = 0;
    for (int round = 0; round < 3; ++round) {
        model.forward();                                             // the image is current before a kept loop starts
        const unsigned long long before = model.graph().weightImageBuilds();
        k[round] = timeForward(model, steps, warmup, false);
        buildsInKeptLoops += model.graph().weightImageBuilds() - before;
        r[round] = timeForward(model, steps, warmup, true);
    }
    std::sort(k, k + 3);
    std::sort(r, r + 3);
    kept = k[1];
    rebuilt = r[1];
}

template <typename M>
static double timeTraining(M& model, int steps, int warmup) {
    nz::opt::SGD sgd(1e-7f);
    auto pass = [&] {
        model.forward();
        model.backward();
        model.update(&sgd);
    };
    double t[3];
    for (int round = 0; round < 3; ++round) {
        for (int i = 0; i < warmup; ++i) pass();
        nzhip_sync_all();
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; ++i) pass();
        nzhip_sync_all();
        t[round] = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
    }
    std::sort(t, t + 3);
    return t[1];
}

int main(int argc, char** argv) {
    const int steps = argc > 1 ? atoi(argv[1]) : 200, warmup = argc > 2 ? atoi(argv[2]) : 20;
    try {
        std::mt19937 gen(11);
        double linKept, linRebuilt, convKept, convRebuilt, linTrain, convTrain;
        unsigned long long linBuilds, convBuilds;
        {
            LinearLayer m(4096, 1024, 4096);
            fill(m, gen, 0.0765f);
            measure(m, steps, warmup, linKept, linRebuilt, linBuilds);
            linTrain = timeTraining(m, steps, warmup);
        }
        {
            ConvLayer m(16, 64, 128, 128, 128);
            fill(m, gen, 0.06f);
            measure(m, steps, warmup, convKept, convRebuilt, convBuilds);
            convTrain = timeTraining(m, steps, warmup);
        }
        printf("{\"workload\": \"single layers through nz::Model, host wall clock per pass (forward(); forward() + backward() + update())\", \"steps\": %d, \"warmup\": %d, "
               "\"linear_4096x1024_to_4096_relu\": {\"ms_weight_image_kept\": %.4f, \"ms_weight_image_rebuilt_every_pass\": %.4f, "
               "\"image_builds_in_kept_loops\": %llu, \"ms_training_pass\": %.4f}, "
               "\"conv2d_16x64x128x128_to_128_relu_per_sample_weights_per_pixel_bias\": {\"ms_weight_image_kept\": %.4f, "
               "\"ms_weight_image_rebuilt_every_pass\": %.4f, \"image_builds_in_kept_loops\": %llu, \"ms_training_pass\": %.4f}}\n",
               steps, warmup, linKept, linRebuilt, linBuilds, linTrain, convKept, convRebuilt, convBuilds, convTrain);
    } catch (const std::exception& e) {
        fprintf(stderr, "layer_bench: %s\n", e.what());
        return 1;
    }
    return 0;
}
