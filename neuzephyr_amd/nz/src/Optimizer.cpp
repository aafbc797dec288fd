#include "NeuZephyr/Optimizer.cuh"

#include "NeuZephyr/NeuZephyrCudaErrorHandling.cuh"
#include "nzhip.h"

namespace nz::opt {
    SGD::SGD(const Tensor::value_type learning_rate) { this->learning_rate = learning_rate; }

    void SGD::step(Node* input) {
        NZ_CHECK(nzhip_sgd_step(input->output->data(), input->output->grad(), learning_rate, input->output->size(),
                                nzhip_default_stream()));
    }

    Adam::Adam(const Tensor::value_type learning_rate, const Tensor::value_type beta1, const Tensor::value_type beta2)
        : beta1(beta1), beta2(beta2) {
        this->learning_rate = learning_rate;
    }

    void Adam::skip(Node* input) {
        (void)input;
        it++;                                            // the reference counts every step() call (src/Optimizer.cu:87)
    }

    void Adam::step(Node* input) {
        it++;                                            // src/Optimizer.cu:87: one count per call, shared by all nodes
        for (auto* moments : {&m, &v}) {
            if (moments->find(input) == moments->end()) {
                Tensor zero(input->output->shape(), false);
                zero.clear();
                (*moments)[input] = std::move(zero);
            }
        }
        NZ_CHECK(nzhip_adam_step(input->output->data(), m[input].data(), v[input].data(), input->output->grad(),
                                 learning_rate, beta1, beta2, epsilon, it, input->output->size(), nzhip_default_stream()));
    }
}
