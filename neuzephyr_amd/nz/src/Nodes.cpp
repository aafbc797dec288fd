#include "NeuZephyr/Nodes.cuh"

#include <algorithm>
#include <iostream>
#include <stdexcept>

#include "NeuZephyr/NeuZephyrCudaErrorHandling.cuh"
#include "NeuZephyr/TensorOperations.cuh"
#include "nzhip.h"

namespace nz::nodes {
    void Node::print(std::ostream& os) const {
        os << "Node(" << type << ")";
        if (output) os << " shape " << output->shape();
        os << std::endl;
    }

    void Node::dataInject(Tensor::value_type* data, const bool grad) const { output->dataInject(data, grad); }

    void Node::dataInject(const std::initializer_list<Tensor::value_type>& data, const bool grad) const {
        output->dataInject(data, grad);
    }

    namespace io {
        InputNode::InputNode(const Tensor::shape_type& shape, const bool requires_grad) {
            output = std::make_shared<Tensor>(shape, requires_grad);
            type = "Input";
        }

        InputNode::InputNode(const Tensor& tensor) {
            output = std::make_shared<Tensor>(tensor);
            type = "Input";
        }

        InputNode::InputNode(const Tensor::shape_type& shape, Tensor::value_type* data, const bool requires_grad,
                             const bool host) {
            output = std::make_shared<Tensor>(shape, data, requires_grad, host);
            type = "Input";
        }

        InputNode::InputNode(const Tensor::shape_type& shape, const std::initializer_list<Tensor::value_type>& data,
                             const bool requires_grad) {
            output = std::make_shared<Tensor>(shape, data, requires_grad);
            type = "Input";
        }

        OutputNode::OutputNode(Node* input) : loss(0) {
            inputs.push_back(input);
            type = "Output";
        }

        void OutputNode::forward() { output = inputs[0]->output; }

        void OutputNode::backward() {                                  // src/Nodes.cu:62-66
            if (inputs[0]->output->requiresGrad()) inputs[0]->output->fill(1, true);
        }
    }

    namespace calc {
        AddNode::AddNode(Node* input_left, Node* input_right) {
            const auto l = input_left->output->shape(), r = input_right->output->shape();
            if (!l.isBroadcastCompatible(r) || l.H() != r.H() || l.W() != r.W()) {
                throw std::invalid_argument("Shapes are not broadcast compatible.");
            }
            inputs.push_back(input_left);
            inputs.push_back(input_right);
            const bool requires_grad = input_left->output->requiresGrad() || input_right->output->requiresGrad();
            output = std::make_shared<Tensor>(l.Broadcast(r), requires_grad);
            type = "Add";
        }

        void AddNode::forward() { tensorMatrixAdd(*output, *inputs[0]->output, *inputs[1]->output); }
        void AddNode::backward() {                                     // src/Nodes.cu:99-146
            for (Node* in : inputs)
                if (in->output->requiresGrad()) {
                    // equal shapes: a plain copy of the gradient (every element written); broadcast inputs accumulate
                    const bool copies = in->output->shape() == output->shape();
                    iAddBackward(copies ? in->output->gradOverwrite() : in->output->grad(), output->grad(), in->output->shape(),
                                 output->shape());
                }
        }

        MatMulNode::MatMulNode(Node* input_left, Node* input_right) {
            const auto l = input_left->output->shape(), r = input_right->output->shape();
            if (!l.isBroadcastCompatible(r) || l.W() != r.H()) {
                throw std::invalid_argument("Shapes are not broadcast compatible.");
            }
            inputs.push_back(input_left);
            inputs.push_back(input_right);
            const bool requires_grad = input_left->output->requiresGrad() || input_right->output->requiresGrad();
            const Tensor::shape_type shape = {std::max(l[0], r[0]), std::max(l[1], r[1]), l[2], r[3]};
            output = std::make_shared<Tensor>(shape, requires_grad);
            type = "MatMul";
        }

        void MatMulNode::forward() { GEMMTensorCore(*output, *inputs[0]->output, *inputs[1]->output); }
        void MatMulNode::backward() {                                  // src/Nodes.cu:169-182: dA += dC*B^T, dB += A^T*dC
            Tensor& a = *inputs[0]->output;
            Tensor& b = *inputs[1]->output;
            if (!a.requiresGrad() && !b.requiresGrad()) return;
            iMatMulBackward(a.requiresGrad() ? a.grad() : nullptr, b.requiresGrad() ? b.grad() : nullptr, a.data(), b.data(),
                            output->grad(), a.shape(), b.shape(), output->shape());
        }

        ReLUNode::ReLUNode(Node* input) {
            inputs.push_back(input);
            output = std::make_shared<Tensor>(input->output->shape(), input->output->requiresGrad());
            type = "ReLU";
        }

        void ReLUNode::forward() { iRELU(output->data(), inputs[0]->output->data(), output->size()); }
        void ReLUNode::backward() {                                    // src/Nodes.cu:357-364
            if (inputs[0]->output->requiresGrad())
                iReLUBackward(inputs[0]->output->gradOverwrite(), inputs[0]->output->data(), output->grad(), output->size());
        }

        SoftmaxNode::SoftmaxNode(Node* input) {
            if (std::min(input->output->shape().H(), input->output->shape().W()) != 1) {
                throw std::invalid_argument("SoftmaxNode: input must be 1D");
            }
            inputs.push_back(input);
            output = std::make_shared<Tensor>(input->output->shape(), input->output->requiresGrad());
            type = "Softmax";
        }

        void SoftmaxNode::forward() { Softmax(*output, *inputs[0]->output); }

        void SoftmaxNode::backward() {                                 // src/Nodes.cu:538-548
            if (!inputs[0]->output->requiresGrad()) return;
            // Jacobian x gradient (J x dY for column vectors, dY x J for rows: the Jacobian is symmetric, so
            // both are the same sums) with fp16-rounded operands like the GEMM the reference calls, fused so
            // that the n x n Jacobian never reaches memory
            const auto& s = output->shape();
            iSoftmaxBackward(inputs[0]->output->gradOverwrite(), output->data(), output->grad(), s[2] * s[3], s[0] * s[1]);
        }

        ExpandNode::ExpandNode(Node* input, const Tensor::size_type newBatch) : newBatch(newBatch) {
            if (input->output->shape()[0] != 1) throw std::invalid_argument("ExpandNode: input must have batch size 1");
            inputs.push_back(input);
            const auto s = input->output->shape();
            output = std::make_shared<Tensor>(Tensor::shape_type{newBatch, s[1], s[2], s[3]}, input->output->requiresGrad());
            type = "Expand";
        }

        void ExpandNode::forward() { iExpand(output->data(), inputs[0]->output->data(), inputs[0]->output->size(), newBatch); }
        void ExpandNode::backward() {                                  // src/Nodes.cu:594-603
            if (inputs[0]->output->requiresGrad())
                iCompress(inputs[0]->output->grad(), output->grad(), inputs[0]->output->size(), newBatch);
        }

        AveragePoolingNode::AveragePoolingNode(Node* input, const Tensor::size_type poolSize, const Tensor::size_type stride,
                                               const Tensor::size_type padding)
            : poolSize(poolSize), stride(stride), padding(padding) {
            const auto s = input->output->shape();
            if (poolSize == 0 || stride == 0 || s[2] + 2 * padding < poolSize || s[3] + 2 * padding < poolSize)
                throw std::invalid_argument("AveragePoolingNode: window does not fit the padded input");
            inputs.push_back(input);
            output = std::make_shared<Tensor>(Tensor::shape_type{s[0], s[1], (s[2] + 2 * padding - poolSize) / stride + 1,
                                                                 (s[3] + 2 * padding - poolSize) / stride + 1},
                                              input->output->requiresGrad());
            type = "AveragePooling";
        }

        void AveragePoolingNode::forward() {
            const auto si = inputs[0]->output->shape(), so = output->shape();
            iAveragePooling(output->data(), inputs[0]->output->data(), poolSize, stride, padding, si[0], si[1], si[2], si[3],
                            so[2], so[3]);
        }

        void AveragePoolingNode::backward() {                          // src/Nodes.cu:684-690
            if (!inputs[0]->output->requiresGrad()) return;
            const auto si = inputs[0]->output->shape(), so = output->shape();
            // the first writer of a gradient that is still to be cleared overwrites it: no clear, no read of the zeros
            const bool fresh = inputs[0]->output->gradIsZero();
            iAveragePoolingBackward(fresh ? inputs[0]->output->gradOverwrite() : inputs[0]->output->grad(), output->grad(), poolSize,
                                    stride, padding, si[0], si[1], si[2], si[3], so[2], so[3], fresh);
        }

        ReshapeNode::ReshapeNode(Node* input, const Tensor::shape_type& newShape) : newShape(newShape) {
            if (input->output->shape().size() != newShape.size()) {
                throw std::invalid_argument("ReshapeNode: input and new shape must have the same number of dimensions");
            }
            inputs.push_back(input);
            output = std::make_shared<Tensor>(newShape, input->output->requiresGrad());
            type = "Reshape";
        }

        void ReshapeNode::forward() {
            NZ_CHECK(nzhip_memcpy_d2d(output->data(), inputs[0]->output->data(), output->size() * sizeof(Tensor::value_type)));
        }
        void ReshapeNode::backward() {                                 // src/Nodes.cu:565-571
            if (inputs[0]->output->requiresGrad())
                NZ_CHECK(nzhip_memcpy_d2d(inputs[0]->output->gradOverwrite(), output->grad(),
                                          output->size() * sizeof(Tensor::value_type)));
        }

        Img2ColNode::Img2ColNode(Node* input, const Tensor::size_type kernelHeight, const Tensor::size_type kernelWidth,
                                 const Tensor::size_type stride, const Tensor::size_type padding)
            : kernelHeight(kernelHeight), kernelWidth(kernelWidth), stride(stride), padding(padding),
              outputHeight((input->output->shape().H() + 2 * padding - kernelHeight) / stride + 1),
              outputWidth((input->output->shape().W() + 2 * padding - kernelWidth) / stride + 1) {
            inputs.push_back(input);
            const auto s = input->output->shape();
            output = std::make_shared<Tensor>(
                Tensor::shape_type{s[0], 1, static_cast<size_t>(outputHeight * outputWidth),
                                   static_cast<size_t>(kernelHeight * kernelWidth * s[1])},
                input->output->requiresGrad());
            type = "Img2Col";
        }

        void Img2ColNode::forward() {
            const auto s = inputs[0]->output->shape();
            iImg2col(output->data(), inputs[0]->output->data(), outputHeight, outputWidth, s[1], kernelHeight, kernelWidth,
                     stride, padding, s[2], s[3], s[0]);
        }
        void Img2ColNode::backward() {                                 // src/Nodes.cu:632-640
            if (!inputs[0]->output->requiresGrad()) return;
            const auto s = inputs[0]->output->shape();
            iImg2colBackward(inputs[0]->output->grad(), output->grad(), outputHeight, outputWidth, s[1], kernelHeight,
                             kernelWidth, stride, padding, s[2], s[3], s[0]);
        }

        Col2ImgNode::Col2ImgNode(Node* input, const Tensor::size_type outputHeight, const Tensor::size_type outputWidth)
            : outputHeight(outputHeight), outputWidth(outputWidth), outputChannels(input->output->shape()[3]) {
            inputs.push_back(input);
            output = std::make_shared<Tensor>(
                Tensor::shape_type(input->output->shape()[0], static_cast<size_t>(outputChannels),
                                   static_cast<size_t>(outputHeight), static_cast<size_t>(outputWidth)),
                input->output->requiresGrad());
            type = "Col2Img";
        }

        void Col2ImgNode::forward() {
            iCol2img(output->data(), inputs[0]->output->data(), outputHeight, outputWidth, outputChannels,
                     inputs[0]->output->shape()[0]);
        }
        void Col2ImgNode::backward() {                                 // src/Nodes.cu:660-665
            if (inputs[0]->output->requiresGrad())
                iCol2imgBackward(inputs[0]->output->gradOverwrite(), output->grad(), outputHeight, outputWidth, outputChannels,
                                 inputs[0]->output->shape()[0]);
        }
    }

    namespace loss {
        MeanSquaredErrorNode::MeanSquaredErrorNode(Node* input1, Node* input2) : OutputNode(input1) {
            if (input1->output->shape() != input2->output->shape())
                throw std::invalid_argument("input1 and input2 should have the same shape");
            inputs.push_back(input2);
            type = "MeanSquaredError";
        }

        void MeanSquaredErrorNode::forward() {                         // src/Nodes.cu:785-802
            OutputNode::forward();
            loss = iMeanSquaredError(inputs[0]->output->data(), inputs[1]->output->data(), output->size());
        }

        void MeanSquaredErrorNode::backward() {                        // src/Nodes.cu:804-811
            if (output->requiresGrad())
                iMSEBackward(output->gradOverwrite(), inputs[0]->output->data(), inputs[1]->output->data(), output->size());
        }

        BinaryCrossEntropyNode::BinaryCrossEntropyNode(Node* input1, Node* input2) : OutputNode(input1) {
            if (input1->output->shape() != input2->output->shape())
                throw std::invalid_argument("input1 and input2 should have the same shape");
            inputs.push_back(input2);
            type = "BinaryCrossEntropy";
        }

        void BinaryCrossEntropyNode::forward() {                       // src/Nodes.cu:822-840
            OutputNode::forward();
            loss = iBinaryCrossEntropy(inputs[0]->output->data(), inputs[1]->output->data(), output->size());
        }

        void BinaryCrossEntropyNode::backward() {                      // src/Nodes.cu:842-849
            if (output->requiresGrad())
                iBCEBackward(output->gradOverwrite(), inputs[0]->output->data(), inputs[1]->output->data(), output->size());
        }
    }
}
