// The example network of the reference's README (README.md:62-90) on this build's nz:: API:
//   Conv2d(3 -> 1, 3x3) -> ReLU -> Conv2d(1 -> 1, 3x3) -> AvgPool2d(5, 2) -> Linear(16) -> Softmax -> BCELoss,
// trained with Adam. Prints one JSON line with the time of a training step (forward + backward + update,
// host wall clock around a device synchronisation) and the loss before and after.
//   readme_example [steps] [warmup] [batch] [height] [width]
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

struct SegmentationModel : nz::Model {
    InputNode input, target;
    SegmentationModel(size_t n, size_t h, size_t w) : input({n, 3, h, w}), target({1, 1, 16, 1}) {
        Node* x = Conv2d(&input, 1, 3, 3, 1, 1);
        x = ReLU(x);
        x = Conv2d(x, 1, 3, 3, 1, 1);
        x = AvgPool2d(x, 5, 2);
        x = Linear(x, 16);
        x = Softmax(x);
        BCELoss(x, &target);
    }
};

int main(int argc, char** argv) {
    const int steps = argc > 1 ? atoi(argv[1]) : 10, warmup = argc > 2 ? atoi(argv[2]) : 3;
    const size_t n = argc > 3 ? (size_t)atol(argv[3]) : 10, h = argc > 4 ? (size_t)atol(argv[4]) : 1024,
                 w = argc > 5 ? (size_t)atol(argv[5]) : 1024;
    try {
        SegmentationModel model(n, h, w);
        std::mt19937 gen(7);
        std::uniform_real_distribution<float> pixel(0.f, 1.f);
        std::vector<float> x(n * 3 * h * w);
        for (auto& v : x) v = pixel(gen);
        model.input.dataInject(x.begin(), x.end());
        std::vector<float> labels(16, 0.02f);
        labels[3] = 0.7f;
        model.target.dataInject(labels.begin(), labels.end());
        // small positive parameters: the ReLU stays alive and the softmax away from saturation
        for (auto* p : model.parameters()) {
            const float hi = 2.0f / static_cast<float>(p->output->shape()[2] * p->output->shape()[3]) + 1e-4f;
            std::uniform_real_distribution<float> init(0.f, hi);
            std::vector<float> v(p->output->size());
            for (auto& e : v) e = init(gen);
            p->dataInject(v.begin(), v.end());
        }
        // Adam moves every weight by about lr per step whatever the gradient's size, so a logit of the Linear
        // layer moves by about fan-in x lr x mean input; keep that near 0.1 (fan-in 260 100 at full size)
        const size_t fanIn = ((h + 2 - 3 + 1 - 5) / 2 + 1) * ((w + 2 - 3 + 1 - 5) / 2 + 1);
        nz::opt::Adam optimizer(0.25f / static_cast<float>(fanIn), 0.9f, 0.999f);
        model.forward();
        const float first = model.getLoss();
        auto step = [&] {
            model.forward();
            model.backward();
            model.update(&optimizer);
        };
        for (int i = 0; i < warmup; i++) step();
        nzhip_sync_all();
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; i++) step();
        nzhip_sync_all();
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
        model.forward();
        printf("{\"workload\": \"README example network, batch %zu x 3 x %zu x %zu, one Adam training step\", "
               "\"ms_per_step\": %.4f, \"steps\": %d, \"warmup\": %d, \"loss_first\": %.6f, \"loss_last\": %.6f, "
               "\"fused_groups\": %zu}\n",
               n, h, w, ms, steps, warmup, first, model.getLoss(), model.graph().fusedGroupCount());
    } catch (const std::exception& e) {
        fprintf(stderr, "readme_example: %s\n", e.what());
        return 1;
    }
    return 0;
}
