#include "NeuZephyr/Model.cuh"

#include <stdexcept>

namespace nz {
    Model::Model() = default;

    Model::~Model() {
        for (const auto* node : hiddenNodes) delete node;
    }

    data::Tensor& Model::forward() {
        computeGraph.forward();
        return *computeGraph.getOutputNode()->output;
    }

    void Model::backward() { computeGraph.backward(); }

    void Model::update(opt::Optimizer* optimizer) const {
        computeGraph.update(optimizer);
        computeGraph.zeroGrad();
    }

    Node* Model::track(Node* node) {
        node->internal = true;
        hiddenNodes.push_back(node);
        computeGraph.addNode(node);
        return node;
    }

    Node* Model::Add(Node* lhs, Node* rhs) {
        computeGraph.addNode(lhs);
        computeGraph.addNode(rhs);
        return track(new calc::AddNode(lhs, rhs));
    }

    Node* Model::Mul(Node* lhs, Node* rhs) {
        computeGraph.addNode(lhs);
        computeGraph.addNode(rhs);
        return track(new calc::MatMulNode(lhs, rhs));
    }

    Node* Model::Bias(Node* input) {
        const auto s = input->output->shape();
        auto* param = new io::InputNode({1, s[1], s[2], s[3]}, true);      // src/Model.cu:68-71
        param->output->randomize();
        hiddenNodes.push_back(param);
        params.push_back(param);
        computeGraph.addNode(param);
        return Add(input, param);
    }

    Node* Model::Reshape(Node* input, const data::Tensor::shape_type& shape) {
        computeGraph.addNode(input);
        return track(new calc::ReshapeNode(input, shape));
    }

    Node* Model::Linear(Node* input, const size_t outSize) {
        const auto s = input->output->shape();
        const size_t inputSize = s[1] * s[2] * s[3];
        Node* shaped = s[2] != inputSize ? Reshape(input, {s[0], 1, inputSize, 1}) : input;
        auto* weight = new io::InputNode({1, 1, outSize, inputSize}, true);
        weight->output->randomize();
        hiddenNodes.push_back(weight);
        params.push_back(weight);
        computeGraph.addNode(weight);
        return Bias(Mul(weight, shaped));
    }

    Node* Model::ReLU(Node* input) {
        computeGraph.addNode(input);
        return track(new calc::ReLUNode(input));
    }

    Node* Model::Img2Col(Node* input, const data::Tensor::size_type kernelHeight,
                         const data::Tensor::size_type kernelWidth, const data::Tensor::size_type stride,
                         const data::Tensor::size_type padding) {
        computeGraph.addNode(input);
        return track(new calc::Img2ColNode(input, kernelHeight, kernelWidth, stride, padding));
    }

    Node* Model::Col2Img(Node* input, const data::Tensor::size_type outputHeight,
                         const data::Tensor::size_type outputWidth) {
        computeGraph.addNode(input);
        return track(new calc::Col2ImgNode(input, outputHeight, outputWidth));
    }

    Node* Model::Conv2d(Node* input, const data::Tensor::size_type outChannels,
                        const data::Tensor::size_type kernelHeight, const data::Tensor::size_type kernelWidth,
                        const data::Tensor::size_type stride, const data::Tensor::size_type padding, const bool bias) {
        computeGraph.addNode(input);
        const auto s = input->output->shape();
        // one weight copy per sample, as the reference allocates it (src/Model.cu:248-252)
        auto* kernel = new io::InputNode(
            {s.N(), 1, static_cast<size_t>(s.C() * kernelHeight * kernelWidth), static_cast<size_t>(outChannels)}, true);
        kernel->output->randomize();
        hiddenNodes.push_back(kernel);
        params.push_back(kernel);
        computeGraph.addNode(kernel);
        Node* col = Img2Col(input, kernelHeight, kernelWidth, stride, padding);
        Node* result = Mul(col, kernel);
        if (bias) result = Bias(result);
        return Col2Img(result, (s.H() + 2 * padding - kernelHeight) / stride + 1,
                       (s.W() + 2 * padding - kernelWidth) / stride + 1);
    }

    Node* Model::Softmax(Node* input) {
        computeGraph.addNode(input);
        const auto s = input->output->shape();
        const size_t size = s[1] * s[2] * s[3];
        Node* shaped = s[2] != size ? Reshape(input, {s[0], 1, size, 1}) : input;
        return track(new calc::SoftmaxNode(shaped));
    }

    Node* Model::TargetExpand(Node* input, const data::Tensor::shape_type& shape) {
        computeGraph.addNode(input);
        const auto s = input->output->shape();
        if (s == shape) return input;
        if (s[0] != 1 || s[1] != shape[1] || s[2] != shape[2] || s[3] != shape[3])
            throw std::runtime_error("The input data cannot be expanded.");
        return track(new calc::ExpandNode(input, shape.N()));
    }

    Node* Model::AvgPool2d(Node* input, const data::Tensor::size_type poolSize, const data::Tensor::size_type stride,
                           const data::Tensor::size_type padding) {
        computeGraph.addNode(input);
        return track(new calc::AveragePoolingNode(input, poolSize, stride, padding));
    }

    void Model::MSELoss(Node* input, Node* target) {
        computeGraph.addNode(input);
        Node* expanded = TargetExpand(target, input->output->shape());
        auto* mse = new loss::MeanSquaredErrorNode(input, expanded);
        hiddenNodes.push_back(mse);
        computeGraph.addOutput(mse);
    }

    void Model::BCELoss(Node* input, Node* target) {
        computeGraph.addNode(input);
        Node* expanded = TargetExpand(target, input->output->shape());
        auto* bce = new loss::BinaryCrossEntropyNode(input, expanded);
        hiddenNodes.push_back(bce);
        computeGraph.addOutput(bce);
    }

    data::Tensor::value_type Model::getLoss() const { return computeGraph.getLoss(); }

    void Model::defaultOutput(Node* input) {
        auto* output = new io::OutputNode(input);
        hiddenNodes.push_back(output);
        computeGraph.addOutput(output);
        computeGraph.addNode(input);
    }
}
