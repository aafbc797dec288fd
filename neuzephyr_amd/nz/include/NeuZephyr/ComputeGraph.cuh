// Topological executor for the forward pass (reference: include/NeuZephyr/ComputeGraph.cuh,
// src/ComputeGraph.cu:258-296 Kahn sort, :405-412 forward). On top of the reference's
// node-by-node execution, chains of Model-internal nodes that form a Conv2d
// (Img2Col -> MatMul [-> Add] -> Col2Img [-> ReLU]) or a Linear (MatMul(W, x) [-> Add] [-> ReLU])
// are issued as ONE fused kernel; setFusion(false) restores plain node-by-node execution,
// which yields the same values up to fp32 summation order.
#ifndef NZ_COMPUTE_GRAPH_CUH
#define NZ_COMPUTE_GRAPH_CUH
#include <functional>
#include <memory>
#include <iosfwd>
#include <string>
#include <vector>

#include "Nodes.cuh"
#include "Optimizer.cuh"
#include "TensorOperations.cuh"
#include "dl_export.cuh"

namespace nz::graph {
    using namespace nodes;
    using namespace data;

    class DL_API ComputeGraph {
    public:
        ComputeGraph() = default;
        friend DL_API std::ostream& operator<<(std::ostream& os, ComputeGraph& graph);

        Node* addNode(Node* node);
        io::InputNode* addInput(io::InputNode* input);
        io::OutputNode* addOutput(io::OutputNode* node);
        [[nodiscard]] bool inGraph(Node* node) const;
        void topologicalSort();                          // throws std::runtime_error("Graph has cycle")
        [[nodiscard]] bool isSorted() const;
        void forward();
        // Reverse pass over the sorted nodes (reference: src/ComputeGraph.cu:414-432); throws
        // std::runtime_error if the graph is not sorted or does not have exactly one output node. If the
        // last forward() fused node chains, the skipped intermediates are recomputed first.
        void backward();
        void zeroGrad() const;                           // src/ComputeGraph.cu:434-438
        void update(opt::Optimizer* optimizer) const;    // step() per leaf that requires gradients, skip() per other node the reference would step (:541-547)
        [[nodiscard]] Tensor::value_type getLoss() const;      // of the first output node; throws std::runtime_error without one (:534-539)
        [[nodiscard]] io::OutputNode* getOutputNode() const;   // throws std::runtime_error without exactly one output
        void setFusion(bool enabled);
        [[nodiscard]] size_t fusedGroupCount() const { return fusedGroups; }
        // how often the fused layers have built the fp16 image of their weights so far (once per layer while the
        // weights stay untouched, again after every change)
        [[nodiscard]] unsigned long long weightImageBuilds() const;
        [[nodiscard]] const std::vector<Node*>& getNodes() const { return nodes; }

    private:
        void buildPlan();
        std::vector<Node*> nodes;
        std::vector<io::InputNode*> inputNodes;
        std::vector<io::OutputNode*> outputNodes;
        std::vector<Node*> sortedNodes;
        std::vector<std::function<void()>> plan;         // what forward() runs, in order
        std::vector<std::function<void()>> backPlan;     // what backward() runs, in order
        std::vector<Node*> fusedMembers;                 // nodes of fused chains whose outputs backward() needs, in sorted order
        bool intermediatesStale = false;                 // a fused forward() skipped their outputs
        bool fusion = true;
        bool planned = false;
        size_t fusedGroups = 0;
        std::vector<std::shared_ptr<PreparedOperand>> weightImages;   // one per fused layer of the current plan
    };
}
#endif
