// Declarative layer builders over ComputeGraph (reference: include/NeuZephyr/Model.cuh:188-1146,
// src/Model.cu:11-103, 223-263, 325-332). Only the builders on the GEMM path exist here:
// Add, Mul, Bias, Reshape, Linear, ReLU, Img2Col, Col2Img, Conv2d and defaultOutput.
// Parameter shapes and operand order are the reference's: Linear multiplies a weight
// [1,1,OUT,IN] by the input reshaped to [N,1,IN,1]; Conv2d multiplies the im2col matrix by a
// weight [N,1,C*Kh*Kw,O] (one copy per sample) and adds a bias [1,1,Ho*Wo,O].
#ifndef NZ_MODEL_CUH
#define NZ_MODEL_CUH
#include <vector>

#include "ComputeGraph.cuh"
#include "Nodes.cuh"
#include "dl_export.cuh"

using namespace nz::nodes;

namespace nz {
    class DL_API Model {
    public:
        Model();
        virtual ~Model();
        Model(const Model&) = delete;
        Model& operator=(const Model&) = delete;

        data::Tensor& forward();
        void backward();                                 // reverse pass of the graph (src/Model.cu:17-19)
        void update(opt::Optimizer* optimizer) const;    // graph update, then zeroGrad (src/Model.cu:20-23)
        [[nodiscard]] data::Tensor::value_type getLoss() const;   // loss of the last forward() (src/Model.cu:25-27)
        graph::ComputeGraph& graph() { return computeGraph; }
        // Parameters (weights, biases) in creation order, so that callers can inject values.
        [[nodiscard]] const std::vector<io::InputNode*>& parameters() const { return params; }

    private:
        std::vector<Node*> hiddenNodes;
        std::vector<io::InputNode*> params;
        Node* track(Node* node);

    protected:
        graph::ComputeGraph computeGraph;
        Node* Add(Node* lhs, Node* rhs);
        Node* Mul(Node* lhs, Node* rhs);
        Node* Bias(Node* input);
        Node* Reshape(Node* input, const data::Tensor::shape_type& shape);
        Node* Linear(Node* input, size_t outSize);
        Node* ReLU(Node* input);
        Node* Img2Col(Node* input, data::Tensor::size_type kernelHeight, data::Tensor::size_type kernelWidth,
                      data::Tensor::size_type stride, data::Tensor::size_type padding);
        Node* Col2Img(Node* input, data::Tensor::size_type outputHeight, data::Tensor::size_type outputWidth);
        Node* Conv2d(Node* input, data::Tensor::size_type outChannels, data::Tensor::size_type kernelHeight,
                     data::Tensor::size_type kernelWidth, data::Tensor::size_type stride,
                     data::Tensor::size_type padding, bool bias = true);
        // softmax over all of (c, h, w) per sample (the input is reshaped to [n, 1, c*h*w, 1] first; src/Model.cu:185-202)
        Node* Softmax(Node* input);
        // a batch-1 target repeated to `shape`'s batch; any other mismatch throws std::runtime_error (src/Model.cu:204-221)
        Node* TargetExpand(Node* input, const data::Tensor::shape_type& shape);
        Node* AvgPool2d(Node* input, data::Tensor::size_type poolSize, data::Tensor::size_type stride,
                        data::Tensor::size_type padding = 0);
        void MSELoss(Node* input, Node* target);         // terminates the graph (src/Model.cu:307-315)
        void BCELoss(Node* input, Node* target);         // terminates the graph (src/Model.cu:317-325)
        void defaultOutput(Node* input);
    };
}
#endif
