#include "NeuZephyr/Optimizer.cuh"

#include "NeuZephyr/NeuZephyrCudaErrorHandling.cuh"
#include "nzhip.h"

namespace nz::opt {
    SGD::SGD(const Tensor::value_type learning_rate) { this->learning_rate = learning_rate; }

    void SGD::begin() {
        collecting = true;
        pending.clear();
    }

    void SGD::end() {
        collecting = false;
        if (pending.empty()) return;
        std::vector<float*> data;
        std::vector<const float*> grad;
        std::vector<size_t> n;
        for (Node* node : pending) {
            data.push_back(node->output->data());
            grad.push_back(node->output->grad());
            n.push_back(node->output->size());
        }
        pending.clear();
        NZ_CHECK(nzhip_sgd_step_many(static_cast<int>(data.size()), data.data(), grad.data(), n.data(), learning_rate,
                                     nzhip_default_stream()));
    }

    void SGD::step(Node* input) {
        if (collecting) {
            pending.push_back(input);
            return;
        }
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
        if (collecting) {
            pending.emplace_back(input, it);
            return;
        }
        NZ_CHECK(nzhip_adam_step(input->output->data(), m[input].data(), v[input].data(), input->output->grad(),
                                 learning_rate, beta1, beta2, epsilon, it, input->output->size(), nzhip_default_stream()));
    }

    void Adam::begin() {
        collecting = true;
        pending.clear();
    }

    void Adam::end() {
        collecting = false;
        if (pending.empty()) return;
        std::vector<float*> data, m1, m2;
        std::vector<const float*> grad;
        std::vector<size_t> n;
        std::vector<int> t;
        for (auto& [node, count] : pending) {
            data.push_back(node->output->data());
            m1.push_back(m[node].data());
            m2.push_back(v[node].data());
            grad.push_back(node->output->grad());
            n.push_back(node->output->size());
            t.push_back(count);
        }
        pending.clear();
        NZ_CHECK(nzhip_adam_step_many(static_cast<int>(data.size()), data.data(), m1.data(), m2.data(), grad.data(), n.data(), t.data(),
                                      learning_rate, beta1, beta2, epsilon, nzhip_default_stream()));
    }
}
