// Optimizers that close a training iteration forward -> backward -> update (reference:
// include/NeuZephyr/Optimizer.cuh:125-306, 707-782; src/Optimizer.cu:9-19, 80-102). Only SGD and
// Adam exist here; both run one fused element-wise kernel per parameter tensor, or one for all the tensors
// of a ComputeGraph::update.
#ifndef NZ_OPTIMIZER_CUH
#define NZ_OPTIMIZER_CUH
#include <unordered_map>
#include <utility>
#include <vector>

#include "Nodes.cuh"
#include "dl_export.cuh"

namespace nz::opt {
    using namespace data;
    using namespace nodes;

    class DL_API Optimizer {
    protected:
        Tensor::value_type learning_rate = 0;

    public:
        explicit Optimizer() = default;
        virtual ~Optimizer() = default;
        virtual void step(Node* input) = 0;              // updates input->output from its gradient
        // Account for a step() the reference would make on `input` without touching its tensor:
        // ComputeGraph::update calls this for nodes whose output the next forward() overwrites, so that
        // whatever the optimizer counts per step() call advances exactly as in the reference.
        virtual void skip(Node* input) { (void)input; }
        // ComputeGraph::update brackets its step() calls with these: between them an optimizer may collect the steps
        // and launch them together in end() (same arithmetic per element; the reference launches one kernel per node).
        virtual void begin() {}
        virtual void end() {}
    };

    class DL_API SGD : public Optimizer {
    public:
        explicit SGD(Tensor::value_type learning_rate);
        void step(Node* input) override;                 // data -= lr * grad
        void begin() override;
        void end() override;

    private:
        bool collecting = false;
        std::vector<Node*> pending;
    };

    class DL_API Adam : public Optimizer {
    public:
        explicit Adam(Tensor::value_type learning_rate, Tensor::value_type beta1, Tensor::value_type beta2);
        void step(Node* input) override;
        void skip(Node* input) override;                 // advances the step count only
        void begin() override;
        void end() override;

    private:
        bool collecting = false;
        std::vector<std::pair<Node*, int>> pending;      // node and the step count it was called with
        Tensor::value_type beta1, beta2;
        int it = 0;                                      // counts step() calls, as the reference does
        Tensor::value_type epsilon = 1e-6f;
        std::unordered_map<Node*, Tensor> m, v;          // first and second moment per parameter node
    };
}
#endif
