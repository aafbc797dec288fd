#include "NeuZephyr/ComputeGraph.cuh"

#include <algorithm>
#include <iostream>
#include <queue>
#include <stdexcept>
#include <unordered_map>
#include <unordered_set>

#include "NeuZephyr/TensorOperations.cuh"

namespace nz::graph {
    Node* ComputeGraph::addNode(Node* node) {
        if (!inGraph(node)) {
            nodes.push_back(node);
            planned = false;
            sortedNodes.clear();
        }
        return node;
    }

    io::InputNode* ComputeGraph::addInput(io::InputNode* input) {
        addNode(input);
        inputNodes.push_back(input);
        return input;
    }

    io::OutputNode* ComputeGraph::addOutput(io::OutputNode* node) {
        addNode(node);
        outputNodes.push_back(node);
        return node;
    }

    bool ComputeGraph::inGraph(Node* node) const { return std::find(nodes.begin(), nodes.end(), node) != nodes.end(); }

    bool ComputeGraph::isSorted() const { return !nodes.empty() && sortedNodes.size() == nodes.size(); }

    void ComputeGraph::setFusion(const bool enabled) {
        fusion = enabled;
        planned = false;
    }

    // Kahn's algorithm, breadth first in insertion order (src/ComputeGraph.cu:258-296).
    void ComputeGraph::topologicalSort() {
        sortedNodes.clear();
        std::unordered_map<Node*, int> inDegree;
        std::unordered_map<Node*, std::vector<Node*>> consumers;
        for (Node* node : nodes) {
            inDegree.emplace(node, 0);
            for (Node* input : node->inputs) {
                consumers[input].push_back(node);
                inDegree[node]++;
            }
        }
        std::queue<Node*> ready;
        for (Node* node : nodes)
            if (inDegree[node] == 0) ready.push(node);
        while (!ready.empty()) {
            Node* node = ready.front();
            ready.pop();
            sortedNodes.push_back(node);
            for (Node* next : consumers[node])
                if (--inDegree[next] == 0) ready.push(next);
        }
        if (sortedNodes.size() != nodes.size()) throw std::runtime_error("Graph has cycle");
        planned = false;
    }

    namespace {
        template <typename T>
        T* as(Node* n, const char* type) {
            return (n && n->type == type) ? dynamic_cast<T*>(n) : nullptr;
        }
    }

    // Turns the sorted node list into the list of calls forward() makes. A chain is fused only if
    // every node whose output is skipped is Model-internal and has exactly one consumer.
    void ComputeGraph::buildPlan() {
        plan.clear();
        fusedGroups = 0;
        weightImages.clear();
        std::unordered_map<Node*, std::vector<Node*>> consumers;
        for (Node* node : nodes)
            for (Node* input : node->inputs) consumers[input].push_back(node);
        const auto soleConsumer = [&](Node* n) -> Node* {
            const auto it = consumers.find(n);
            return (it != consumers.end() && it->second.size() == 1) ? it->second[0] : nullptr;
        };
        const auto skippable = [&](Node* n) { return n->internal && soleConsumer(n) != nullptr; };
        struct Group {
            std::vector<Node*> members;          // nodes whose forward() the fused call replaces
            std::function<void()> call;
            std::function<void()> back;          // fused backward of the whole chain (empty: node by node)
        };
        std::vector<Group> groups;
        std::unordered_map<Node*, size_t> groupOf;
        const auto covered = [&](Node* n) { return groupOf.count(n) != 0; };
        const auto addGroup = [&](std::vector<Node*> members, std::function<void()> call,
                                  std::function<void()> back = {}) {
            for (Node* n : members) groupOf[n] = groups.size();
            groups.push_back({std::move(members), std::move(call), std::move(back)});
        };

        if (fusion) {
            for (Node* node : sortedNodes) {
                auto* mm = as<calc::MatMulNode>(node, "MatMul");
                if (!mm || covered(mm) || !skippable(mm)) continue;
                Node* lhs = mm->inputs[0];
                Node* rhs = mm->inputs[1];

                // ---- Conv2d: Img2Col -> MatMul [-> Add(bias [1,1,HW,O])] -> Col2Img [-> ReLU]
                if (auto* i2c = as<calc::Img2ColNode>(lhs, "Img2Col"); i2c && skippable(i2c) && !covered(i2c)) {
                    Node* cur = soleConsumer(mm);
                    calc::AddNode* add = as<calc::AddNode>(cur, "Add");
                    Node* biasNode = nullptr;
                    if (add) {
                        biasNode = add->inputs[0] == mm ? add->inputs[1] : add->inputs[0];
                        const auto bs = biasNode->output->shape(), ms = mm->output->shape();
                        if (!(skippable(add) && bs[0] == 1 && bs[1] == 1 && bs[2] == ms[2] && bs[3] == ms[3])) continue;
                        cur = soleConsumer(add);
                    }
                    auto* c2i = as<calc::Col2ImgNode>(cur, "Col2Img");
                    const auto xs = i2c->inputs[0]->output->shape(), ws = rhs->output->shape();
                    if (!c2i || c2i->outputHeight != i2c->outputHeight || c2i->outputWidth != i2c->outputWidth) continue;
                    if (ws[1] != 1 || (ws[0] != 1 && ws[0] != xs[0]) ||
                        ws[2] != xs[1] * i2c->kernelHeight * i2c->kernelWidth)
                        continue;
                    Node* last = c2i;
                    bool relu = false;
                    if (auto* r = as<calc::ReLUNode>(soleConsumer(c2i), "ReLU"); r && skippable(c2i)) {
                        last = r;
                        relu = true;
                    }
                    Node* x = i2c->inputs[0];
                    const size_t O = ws[3];
                    std::vector<Node*> members = {i2c, mm, c2i};
                    if (add) members.push_back(add);
                    if (relu) members.push_back(last);
                    // Backward of the whole chain without the column-matrix gradient: dZ = dY masked by the
                    // activation; bias and weight gradients from dZ in pixel-major form (Col2Img.backward,
                    // Add.backward, MatMul.backward for B with the column matrix recomputed); the data gradient
                    // as one convolution of dZ. Same accumulate / overwrite behaviour as the node chain.
                    std::function<void()> back;
                    // (the data gradient as one convolution needs a square kernel whose padding stays inside it and a stride up
                    // to 8; a chain whose input carries no gradient does not need it at all)
                    const bool dataGradientFused =
                        i2c->kernelHeight == i2c->kernelWidth && i2c->padding <= i2c->kernelHeight - 1 && i2c->stride >= 1 &&
                        i2c->stride <= 8;       // (strided: the call itself chooses between one convolution and the column-gradient chain)
                    {
                        Node* pre = add ? static_cast<Node*>(add) : static_cast<Node*>(mm);   // holds [N,1,HW,O] gradients
                        back = [=] {
                            if (!last->output->requiresGrad()) return;     // nothing in the chain carries a gradient
                            const bool needW = rhs->output->requiresGrad();
                            const bool needB = biasNode && biasNode->output->requiresGrad();
                            const size_t pixels = c2i->outputHeight * c2i->outputWidth;
                            // The Conv2d bias is [1, 1, pixels, O]: its gradient is the batch sum of the transposed
                            // output gradient and comes straight from the NCHW gradient in one kernel. (With one
                            // channel the gradient already has that layout and the plain batch sum reads it; with a
                            // batch of one Add.backward copies instead of adding: both stay on the node's own path.)
                            const auto bshape = biasNode ? biasNode->output->shape() : Tensor::shape_type{0, 0, 0, 0};
                            const bool fusedB = needB && O != 1 && xs[0] > 1 && bshape[0] == 1 && bshape[1] == 1 &&
                                                bshape[2] == pixels && bshape[3] == O;
                            float* dZ = last->output->grad();
                            bool biasDone = false;
                            if (relu) {
                                float* masked = c2i->output->gradOverwrite();     // every element written
                                if (fusedB) {                                     // mask and bias gradient in one pass
                                    iConv2dBackwardReluBias(masked, biasNode->output->grad(), last->output->data(), dZ, xs[0], O,
                                                            pixels);
                                    biasDone = true;
                                } else {
                                    iReLUBackward(masked, last->output->data(), dZ, last->output->size());
                                }
                                dZ = masked;
                            }
                            // weights straight from x and dZ where the geometry allows, else through the column matrix
                            const bool directW = needW && iConv2dBackwardWeights(rhs->output->grad(), x->output->data(), dZ, xs[0],
                                                                                 xs[1], xs[2], xs[3], O, i2c->kernelHeight,
                                                                                 i2c->kernelWidth, i2c->stride, i2c->padding, ws[0]);
                            // gradient in the layout of the matmul result, [n][pixel][channel]: with one output
                            // channel that is dZ itself, otherwise its per-image transpose
                            float* dPre = dZ;
                            if (O != 1 && ((needW && !directW) || (needB && !fusedB))) {
                                dPre = pre->output->gradOverwrite();
                                iCol2imgBackward(dPre, dZ, c2i->outputHeight, c2i->outputWidth, O, xs[0]);
                            }
                            if (fusedB && !biasDone)
                                iConv2dBackwardBias(biasNode->output->grad(), dZ, xs[0], O, pixels);
                            else if (needB && !fusedB)
                                iAddBackward(biasNode->output->grad(), dPre, biasNode->output->shape(), pre->output->shape());
                            if (needW && !directW) {
                                i2c->forward();                      // the column matrix the fused forward never wrote
                                iMatMulBackward(nullptr, rhs->output->grad(), i2c->output->data(), rhs->output->data(), dPre,
                                                i2c->output->shape(), rhs->output->shape(), mm->output->shape());
                            }
                            if (x->output->requiresGrad()) {
                                // the first writer of a gradient that is still to be cleared overwrites it: no clear, and the
                                // kernels neither read the zeros nor go through a temporary and an add pass
                                const bool fresh = dataGradientFused && x->output->gradIsZero();
                                float* dX = fresh ? x->output->gradOverwrite() : x->output->grad();
                                const bool asConvolution =
                                    dataGradientFused && iConv2dBackwardData(dX, dZ, const_cast<float*>(rhs->output->constData()),
                                                                             xs[0], xs[1], xs[2], xs[3], O, i2c->kernelHeight, i2c->kernelWidth,
                                                                             i2c->stride, i2c->padding, ws[0], !fresh);
                                if (!asConvolution) {
                                    // the reference's chain for this one gradient: dCol = dPre * W^T, then the gather into dx
                                    if (O != 1 && dPre == dZ) {
                                        dPre = pre->output->gradOverwrite();
                                        iCol2imgBackward(dPre, dZ, c2i->outputHeight, c2i->outputWidth, O, xs[0]);
                                    }
                                    i2c->output->zeroGrad();
                                    iMatMulBackward(i2c->output->grad(), nullptr, nullptr, const_cast<float*>(rhs->output->constData()), dPre, i2c->output->shape(),
                                                    rhs->output->shape(), mm->output->shape());
                                    iImg2colBackward(x->output->grad(), i2c->output->grad(), c2i->outputHeight, c2i->outputWidth, xs[1],
                                                     i2c->kernelHeight, i2c->kernelWidth, i2c->stride, i2c->padding, xs[2], xs[3], xs[0]);
                                }
                            }
                        };
                    }
                    // The fp16 image of the weights survives between forward passes while nobody has asked the
                    // weight tensor for a writable pointer (Tensor::version()).
                    auto image = std::make_shared<PreparedOperand>();
                    weightImages.push_back(image);
                    auto seen = std::make_shared<unsigned long long>(~0ull);
                    // The reference's bias is pixel-major, [1, 1, pixels, O]; the convolution kernels want channel planes,
                    // [O][pixels], and turn it into them on every call. Like the weight image, the planes survive between
                    // forward passes while the bias tensor stays untouched (16 x 64 x 128 x 128 -> 128: 7 of 65 us).
                    const size_t outPixels = c2i->outputHeight * c2i->outputWidth;
                    const auto bshapeF = biasNode ? biasNode->output->shape() : Tensor::shape_type{0, 0, 0, 0};
                    const bool keepPlanes = biasNode && bshapeF[0] == 1 && bshapeF[1] == 1 && bshapeF[2] == outPixels &&
                                            bshapeF[3] == O && O >= 8 && outPixels >= 64;
                    auto biasPlanes = std::make_shared<std::unique_ptr<Tensor>>();
                    auto seenBias = std::make_shared<unsigned long long>(~0ull);
                    addGroup(std::move(members), [=] {
                        const float* w = rhs->output->constData();
                        if (rhs->output->version() != *seen) {
                            image->invalidate();
                            *seen = rhs->output->version();
                        }
                        float* b = nullptr;
                        long long pixelStride = static_cast<long long>(O), channelStride = 1;
                        if (keepPlanes) {
                            if (!*biasPlanes)
                                *biasPlanes = std::make_unique<Tensor>(Tensor::shape_type{1, O, c2i->outputHeight, c2i->outputWidth});
                            if (biasNode->output->version() != *seenBias) {
                                iCol2img((*biasPlanes)->data(), const_cast<float*>(biasNode->output->constData()), c2i->outputHeight,
                                         c2i->outputWidth, O, 1);
                                *seenBias = biasNode->output->version();
                            }
                            b = const_cast<float*>((*biasPlanes)->constData());
                            pixelStride = 1;
                            channelStride = static_cast<long long>(outPixels);
                        } else if (biasNode) {
                            b = const_cast<float*>(biasNode->output->constData());
                        }
                        iConv2dForward(last->output->data(), x->output->data(), w, b, xs[0], xs[1], xs[2], xs[3], O,
                                       i2c->kernelHeight, i2c->kernelWidth, i2c->stride, i2c->padding, ws[0], pixelStride,
                                       channelStride, relu, image.get());
                    }, std::move(back));
                    continue;
                }

                // ---- Linear: MatMul(W[1,1,OUT,IN], x[N,1,IN,1]) -> Add(bias [1,1,OUT,1]) [-> ReLU]
                const auto ls = lhs->output->shape(), rs = rhs->output->shape();
                if (ls[0] == 1 && ls[1] == 1 && rs[1] == 1 && rs[3] == 1 && rs[2] == ls[3]) {
                    auto* add = as<calc::AddNode>(soleConsumer(mm), "Add");
                    if (!add) continue;                      // a bare MatMul already is a single kernel
                    Node* biasNode = add->inputs[0] == mm ? add->inputs[1] : add->inputs[0];
                    const auto bs = biasNode->output->shape();
                    if (bs[0] != 1 || bs[1] != 1 || bs[2] != ls[2] || bs[3] != 1) continue;
                    Node* last = add;
                    bool relu = false;
                    if (auto* r = as<calc::ReLUNode>(soleConsumer(add), "ReLU"); r && skippable(add)) {
                        last = r;
                        relu = true;
                    }
                    const size_t batch = rs[0], in = ls[3], out = ls[2];
                    std::vector<Node*> members = {mm, add};
                    if (relu) members.push_back(last);
                    // Backward of the whole chain from the fused output alone: the activation mask comes from y
                    // (y > 0 exactly where the ReLU's input was), the bias gradient is the batch sum of the masked
                    // gradient (Add.backward), and MatMul.backward takes it as dC directly. The node chain would
                    // first have to recompute the MatMul and Add outputs the fused forward never wrote.
                    std::function<void()> back = [=] {
                        if (!last->output->requiresGrad()) return;
                        float* dZ = last->output->grad();
                        if (relu) {
                            float* masked = add->output->gradOverwrite();     // every element written
                            iReLUBackward(masked, last->output->data(), dZ, last->output->size());
                            dZ = masked;
                        }
                        if (biasNode->output->requiresGrad())
                            iAddBackward(biasNode->output->grad(), dZ, biasNode->output->shape(), add->output->shape());
                        const bool needW = lhs->output->requiresGrad(), needX = rhs->output->requiresGrad();
                        if (needW || needX)
                            iMatMulBackward(needW ? lhs->output->grad() : nullptr, needX ? rhs->output->grad() : nullptr,
                                            lhs->output->data(), rhs->output->data(), dZ, lhs->output->shape(),
                                            rhs->output->shape(), mm->output->shape());
                    };
                    auto image = std::make_shared<PreparedOperand>();
                    weightImages.push_back(image);
                    auto seen = std::make_shared<unsigned long long>(~0ull);
                    addGroup(std::move(members), [=] {
                        const float* w = lhs->output->constData();
                        if (lhs->output->version() != *seen) {
                            image->invalidate();
                            *seen = lhs->output->version();
                        }
                        iLinearForward(last->output->data(), rhs->output->data(), w, biasNode->output->data(), batch, in, out,
                                       relu, image.get());
                    }, std::move(back));
                }
            }
        }

        // Emit in topological order. A fused call runs at the position of the LAST of its members,
        // where every external input of the chain (weights, bias) is guaranteed to be ready.
        std::unordered_map<Node*, size_t> position;
        for (size_t i = 0; i < sortedNodes.size(); ++i) position[sortedNodes[i]] = i;
        std::vector<size_t> emitAt(groups.size(), 0);
        for (size_t g = 0; g < groups.size(); ++g)
            for (Node* n : groups[g].members) emitAt[g] = std::max(emitAt[g], position[n]);
        for (size_t i = 0; i < sortedNodes.size(); ++i) {
            Node* node = sortedNodes[i];
            const auto it = groupOf.find(node);
            if (it == groupOf.end()) {
                plan.emplace_back([node] { node->forward(); });
            } else if (emitAt[it->second] == i) {
                plan.push_back(groups[it->second].call);
            }
        }
        // backward: reverse topological order; a chain with a fused backward runs it at the position of its
        // last member (by then every consumer has added its share to that member's gradient)
        backPlan.clear();
        for (size_t i = sortedNodes.size(); i-- > 0;) {
            Node* node = sortedNodes[i];
            const auto it = groupOf.find(node);
            if (it == groupOf.end() || !groups[it->second].back) {
                backPlan.emplace_back([node] { node->backward(); });
            } else if (emitAt[it->second] == i) {
                backPlan.push_back(groups[it->second].back);
            }
        }
        fusedGroups = groups.size();
        fusedMembers.clear();
        for (Node* node : sortedNodes)
            if (const auto it = groupOf.find(node); it != groupOf.end() && !groups[it->second].back)
                fusedMembers.push_back(node);
        planned = true;
    }

    void ComputeGraph::forward() {
        if (!isSorted()) topologicalSort();
        if (!planned) buildPlan();
        for (auto& step : plan) step();
        intermediatesStale = !fusedMembers.empty();
    }

    void ComputeGraph::backward() {
        if (!isSorted()) throw std::runtime_error("Graph is not sorted");
        if (outputNodes.empty()) throw std::runtime_error("No output node");
        if (outputNodes.size() > 1) throw std::runtime_error("Multiple output nodes");
        if (!planned) buildPlan();
        if (intermediatesStale) {
            // node-level gradients read the outputs a fused chain never wrote: produce them now
            for (Node* node : fusedMembers) node->forward();
            intermediatesStale = false;
        }
        // the leaves' gradients are added into: whatever zeroGrad() left to clear on them is cleared in one launch
        std::vector<const Tensor*> leaves;
        for (Node* node : nodes)
            if (node->inputs.empty() && node->output && node->output->requiresGrad()) leaves.push_back(node->output.get());
        Tensor::clearPendingGrads(leaves);
        for (auto& step : backPlan) step();
    }

    void ComputeGraph::update(opt::Optimizer* optimizer) const {
        // The reference steps every node whose output carries a gradient (:541-547), hidden activations
        // and the output node included. An activation is rewritten in full by the next forward(), so only
        // leaves (parameters and inputs that require gradients) are stepped here; the others are passed to
        // skip(), which keeps an optimizer's per-call state in step with the reference: Adam's bias
        // corrections use the number of step() calls so far (src/Optimizer.cu:86-101), so a leaf must see
        // the same count as it would there.
        optimizer->begin();                              // the steps of all leaves may go out as one launch
        for (Node* node : nodes) {
            if (!node->output || !node->output->requiresGrad()) continue;
            if (node->inputs.empty()) optimizer->step(node);
            else optimizer->skip(node);
        }
        optimizer->end();
    }

    unsigned long long ComputeGraph::weightImageBuilds() const {
        unsigned long long n = 0;
        for (const auto& image : weightImages) n += image->fills();
        return n;
    }

    void ComputeGraph::zeroGrad() const {
        for (Node* node : nodes)
            if (node->output && node->output->requiresGrad()) node->output->zeroGrad();
    }

    Tensor::value_type ComputeGraph::getLoss() const {
        if (outputNodes.empty()) throw std::runtime_error("No output node");
        return outputNodes[0]->getLoss();
    }

    io::OutputNode* ComputeGraph::getOutputNode() const {
        if (outputNodes.empty()) throw std::runtime_error("No output node");
        if (outputNodes.size() > 1) throw std::runtime_error("Multiple output nodes");
        return outputNodes[0];
    }

    std::ostream& operator<<(std::ostream& os, ComputeGraph& graph) {
        if (!graph.isSorted()) graph.topologicalSort();
        os << "ComputeGraph: " << graph.nodes.size() << " nodes" << std::endl;
        for (Node* node : graph.sortedNodes) node->print(os);
        return os;
    }
}
