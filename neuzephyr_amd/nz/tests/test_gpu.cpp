// GPU tests of the nz:: C++ API on the GEMM path. They restate, against this build, the
// reference's own tests for the path (test/Test.cpp:708-818 literal MatMul vectors,
// :820-903 MatMul backward vectors, :2880-3072 im2col loop nests, :3074-3177 col2im) and add
// Model::Linear / Model::Conv2d, which
// the reference never tests, against a host computation with the same semantics
// (fp16-rounded operands via the CPU's F16C converter, wide accumulation).
#include <immintrin.h>

#include <cmath>
#include <random>
#include <sstream>

#include "NeuZephyr/ComputeGraph.cuh"
#include "NeuZephyr/Model.cuh"
#include "NeuZephyr/Nodes.cuh"
#include "NeuZephyr/Optimizer.cuh"
#include "NeuZephyr/TensorOperations.cuh"
#include "mini_test.hpp"
#include "nzhip.h"

using namespace nz::data;
using namespace nz::nodes;
using namespace nz::nodes::io;
using namespace nz::nodes::calc;
using namespace nz::nodes::loss;

static float f16(float x) { return _cvtsh_ss(_cvtss_sh(x, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC)); }

static std::vector<float> randomVec(size_t n, unsigned seed, float lo, float hi) {
    std::mt19937 gen(seed);
    std::uniform_real_distribution<float> dist(lo, hi);
    std::vector<float> v(n);
    for (auto& x : v) x = dist(gen);
    return v;
}

static bool closeTo(const std::vector<float>& got, const std::vector<double>& want, double rel) {
    double rms = 0;
    for (double w : want) rms += w * w;
    rms = std::sqrt(rms / (want.empty() ? 1 : want.size()));
    for (size_t i = 0; i < want.size(); ++i) {
        const double d = std::fabs(got[i] - want[i]);
        if (!(d <= rel * std::max(std::fabs(want[i]), rms))) {
            std::printf("  mismatch at %zu: got %g want %g\n", i, got[i], want[i]);
            return false;
        }
    }
    return got.size() == want.size();
}

static const std::vector<float> kData1 = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12};
static const std::vector<float> kData2 = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18};
static const std::vector<float> kExpected = {22, 28, 49, 64, 58, 64, 139, 154, 94, 100, 229, 244,
                                             76, 100, 103, 136, 220, 244, 301, 334, 364, 388, 499, 532};

TEST(TensorCore, TensorCoreGEMMTest) {
    Tensor tensor1({2, 1, 2, 3}), tensor2({1, 3, 3, 2});
    tensor1.dataInject(kData1.begin(), kData1.end());
    tensor2.dataInject(kData2.begin(), kData2.end());
    Tensor result({2, 3, 2, 2});
    GEMMTensorCore(result, tensor1, tensor2);
    Tensor expected({2, 3, 2, 2});
    expected.dataInject(kExpected.begin(), kExpected.end());
    EXPECT_EQ(result, expected);
    EXPECT_TRUE(result.hostData() == kExpected);             // exact, not merely within 1e-5
}

// MappedTensor operands: the kernels of the path read and write page-locked host memory through the same
// pointers the host iterates over (reference: test/Test.cpp:2571-2598 computes its expectation this way).
TEST(MappedTensorPath, TensorCoreGEMMOnMappedOperands) {
    MappedTensor a({2, 1, 2, 3}), b({1, 3, 3, 2}), c({2, 3, 2, 2});
    a.dataInject(kData1.begin(), kData1.end());
    b.dataInject(kData2.begin(), kData2.end());
    GEMMTensorCore(c, a, b);
    std::vector<float> got(c.begin(), c.end());               // begin() waits for the kernel
    EXPECT_TRUE(got == kExpected);
    for (size_t i = 0; i < kExpected.size(); ++i) EXPECT_EQ(c[i], kExpected[i]);
    // the same through a device-resident Tensor
    Tensor ta({2, 1, 2, 3}), tb({1, 3, 3, 2}), tc({2, 3, 2, 2});
    ta.dataInject(a.begin(), a.end());
    tb.dataInject(b.begin(), b.end());
    GEMMTensorCore(tc, ta, tb);
    EXPECT_TRUE(tc.hostData() == got);
}

TEST(MappedTensorPath, MatMulReluAddChainEqualsTheNodeGraph) {
    // the chain of test/Test.cpp:2594-2597: GEMMTensorCore -> ReLU -> + on mapped tensors against the nodes
    MappedTensor x({2, 3, 4, 5}), w({1, 3, 5, 1}), bias({2, 3, 4, 1});
    const auto xv = randomVec(x.size(), 11, -10.f, 10.f), wv = randomVec(w.size(), 12, -10.f, 10.f),
               bv = randomVec(bias.size(), 13, -10.f, 10.f);
    x.dataInject(xv.begin(), xv.end());
    w.dataInject(wv.begin(), wv.end());
    bias.dataInject(bv.begin(), bv.end());
    MappedTensor product({2, 3, 4, 1});
    GEMMTensorCore(product, x, w);
    auto activated = ReLU(product);
    auto sum = activated + bias;

    InputNode in({2, 3, 4, 5}), wn({1, 3, 5, 1}), bn({2, 3, 4, 1});
    in.dataInject(xv.begin(), xv.end());
    wn.dataInject(wv.begin(), wv.end());
    bn.dataInject(bv.begin(), bv.end());
    MatMulNode mm(&in, &wn);
    ReLUNode relu(&mm);
    AddNode add(&relu, &bn);
    mm.forward();
    relu.forward();
    add.forward();
    EXPECT_TRUE(add.output->hostData() == std::vector<float>(sum.begin(), sum.end()));
    // and against the host: fp16-rounded operands, wide accumulation
    std::vector<double> want(sum.size());
    for (size_t n = 0; n < 2; ++n)
        for (size_t c = 0; c < 3; ++c)
            for (size_t h = 0; h < 4; ++h) {
                double acc = 0;
                for (size_t k = 0; k < 5; ++k) acc += double(f16(xv[((n * 3 + c) * 4 + h) * 5 + k])) * f16(wv[c * 5 + k]);
                want[(n * 3 + c) * 4 + h] = std::max(acc, 0.0) + bv[(n * 3 + c) * 4 + h];
            }
    EXPECT_TRUE(closeTo(std::vector<float>(sum.begin(), sum.end()), want, 1e-5));
}

TEST(MappedTensorPath, Img2colCol2imgAndHostMembers) {
    MappedTensor image({2, 3, 5, 4});
    const auto iv = randomVec(image.size(), 21, -1.f, 1.f);
    image.dataInject(iv.begin(), iv.end());
    auto cols = tensorImg2col(image, 3, 3, 1, 1);
    Tensor dimage({2, 3, 5, 4});
    dimage.dataInject(iv.begin(), iv.end());
    auto dcols = tensorImg2col(dimage, 3, 3, 1, 1);
    EXPECT_TRUE(dcols.hostData() == std::vector<float>(cols.begin(), cols.end()));
    auto back = tensorCol2img(cols, 5, 4);                    // [2,1,20,27] read as 5 x 4 pixels of 27 channels
    auto dback = tensorCol2img(dcols, 5, 4);
    EXPECT_TRUE(dback.hostData() == std::vector<float>(back.begin(), back.end()));

    // fp32-exact product and the host-side members
    MappedTensor p({1, 1, 2, 3}), q({1, 1, 3, 2});
    p.dataInject({1, 2, 3, 4, 5, 6});
    q.dataInject({1, 2, 3, 4, 5, 6});
    auto pq = p * q;
    EXPECT_TRUE(std::vector<float>(pq.begin(), pq.end()) == (std::vector<float>{22, 28, 49, 64}));
    MappedTensor pt(p);
    pt.transpose();
    EXPECT_TRUE(pt.shape() == Dimension(1, 1, 3, 2));
    EXPECT_TRUE(std::vector<float>(pt.begin(), pt.end()) == (std::vector<float>{1, 4, 2, 5, 3, 6}));
    EXPECT_EQ((p - p).sum(), 0.f);
    EXPECT_EQ(p.sum(), 21.f);
    EXPECT_EQ(p.sum(0, 0), 21.f);
    auto ratio = p / p;
    EXPECT_TRUE(std::vector<float>(ratio.begin(), ratio.end()) == std::vector<float>(6, 1.f));
    auto neg = -p;
    EXPECT_EQ(neg[5], -6.f);
    EXPECT_TRUE(p == MappedTensor(p));
    EXPECT_TRUE(p != neg);
    EXPECT_THROW(p[6], std::out_of_range);
    EXPECT_THROW(p.grad(), std::invalid_argument);
    EXPECT_THROW(p.clearGrad(), std::runtime_error);
    p.setRequiresGrad(true);
    p.fill(2.f, true);
    EXPECT_EQ(p.grad()[3], 2.f);
    p.fillMatrix(7.f, 0, 0);
    EXPECT_EQ(p[0], 7.f);
    p.reshape({1, 1, 2, 4});
    EXPECT_EQ(p[5], 7.f);
    EXPECT_EQ(p[7], 0.f);
    p.randomize(5);
    for (float v : p) EXPECT_TRUE(v > 0.f && v <= 1.f);
    std::istringstream text("1 2 3 4 5 6 7 8");
    text >> p;
    EXPECT_EQ(p[7], 8.f);
    std::ostringstream os;
    os << p;
    EXPECT_TRUE(os.str().find("Gradient: ") != std::string::npos);
    MappedTensor moved(std::move(p));
    EXPECT_EQ(p.size(), 0u);
    EXPECT_EQ(moved.size(), 8u);
    EXPECT_THROW(MappedTensor({1, 1, 2, 3}) + MappedTensor({1, 1, 3, 2}), std::invalid_argument);
}

TEST(NodeBasic, MatMulForward) {
    InputNode input1({2, 1, 2, 3}), input2({1, 3, 3, 2});
    input1.dataInject(kData1.begin(), kData1.end());
    input2.dataInject(kData2.begin(), kData2.end());
    MatMulNode mul(&input1, &input2);
    mul.forward();
    Tensor expected({2, 3, 2, 2});
    expected.dataInject(kExpected.begin(), kExpected.end());
    EXPECT_EQ(*mul.output, expected);
}

TEST(TensorBasic, InjectCompareCopyMove) {
    Tensor t({1, 2, 2, 2});
    std::vector<float> shortData(7, 1.f), data = {1, 2, 3, 4, 5, 6, 7, 8};
    EXPECT_THROW(t.dataInject(shortData.begin(), shortData.end()), std::runtime_error);
    t.dataInject(data.begin(), data.end());
    EXPECT_TRUE(t.hostData() == data);
    Tensor copy(t);
    EXPECT_EQ(copy, t);
    Tensor moved(std::move(copy));
    EXPECT_EQ(moved, t);
    EXPECT_EQ(copy.size(), 0u);
    Tensor other({1, 2, 2, 2}, {1, 2, 3, 4, 5, 6, 7, 8.001f});
    EXPECT_TRUE(other != t);
    Tensor withGrad({1, 2, 2, 2}, true);
    EXPECT_TRUE(withGrad != t);                               // requiresGrad flags differ
    EXPECT_THROW(Tensor({1, 1, 2, 2}, {1.f, 2.f}), std::invalid_argument);
    t.fill(3.5f);
    EXPECT_TRUE(t.hostData() == std::vector<float>(8, 3.5f));
    t.randomize(3);
    for (float v : t.hostData()) EXPECT_TRUE(v > 0.f && v <= 1.f);
}

TEST(NodeBasic, img2colForward) {
    const size_t n = 2, c = 3, h = 4, w = 5, k_h = 3, k_w = 3, stride = 1, pad = 1;
    const size_t H_out = (h + 2 * pad - k_h) / stride + 1, W_out = (w + 2 * pad - k_w) / stride + 1;
    std::vector<float> inputData = randomVec(n * c * h * w, 11, 0.1f, 0.9f);
    std::vector<float> expectedData(n * H_out * W_out * k_h * k_w * c);
    for (size_t b = 0; b < n; ++b)
        for (size_t i = 0; i < H_out; ++i)
            for (size_t j = 0; j < W_out; ++j)
                for (size_t r = 0; r < k_h; ++r)
                    for (size_t s = 0; s < k_w; ++s)
                        for (size_t c_in = 0; c_in < c; ++c_in) {
                            const int h_in = static_cast<int>(i * stride + r) - static_cast<int>(pad);
                            const int w_in = static_cast<int>(j * stride + s) - static_cast<int>(pad);
                            float val = 0.0f;
                            if (h_in >= 0 && h_in < static_cast<int>(h) && w_in >= 0 && w_in < static_cast<int>(w))
                                val = inputData[b * (c * h * w) + c_in * (h * w) + h_in * w + w_in];
                            expectedData[b * (H_out * W_out * k_h * k_w * c) + (i * W_out + j) * (k_h * k_w * c) +
                                         c_in * (k_h * k_w) + r * k_w + s] = val;
                        }
    InputNode input({n, c, h, w});
    input.dataInject(inputData.begin(), inputData.end());
    Img2ColNode result(&input, k_h, k_w, stride, pad);
    result.forward();
    Tensor expected({n, 1, H_out * W_out, k_h * k_w * c});
    expected.dataInject(expectedData.begin(), expectedData.end());
    EXPECT_EQ(expected, *result.output);
    EXPECT_EQ(expected, tensorImg2col(*input.output, k_h, k_w, stride, pad));
}

TEST(NodeBasic, col2imgForward) {
    const size_t n = 2, c = 3, h = 4, w = 5;
    std::vector<float> inputData = randomVec(n * c * h * w, 12, 0.1f, 0.9f), expectedData(n * c * h * w);
    for (size_t b = 0; b < n; ++b)
        for (size_t j = 0; j < c; ++j)
            for (size_t k = 0; k < h; ++k)
                for (size_t l = 0; l < w; ++l)
                    expectedData[b * (c * h * w) + j * (h * w) + k * w + l] = inputData[b * (c * h * w) + (k * w + l) * c + j];
    InputNode input({n, 1, h * w, c});
    input.dataInject(inputData.begin(), inputData.end());
    Col2ImgNode result(&input, h, w);
    result.forward();
    Tensor expected({n, c, h, w});
    expected.dataInject(expectedData.begin(), expectedData.end());
    EXPECT_EQ(expected, *result.output);
    EXPECT_EQ(expected, tensorCol2img(*input.output, h, w));
}

TEST(NodeBasic, AddBroadcastAndReLU) {
    InputNode a({2, 2, 1, 3}, {1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12});
    InputNode b({1, 1, 1, 3}, {0.5f, 0.5f, -20.f});
    AddNode add(&a, &b);
    add.forward();
    ReLUNode relu(&add);
    relu.forward();
    const std::vector<float> want = {1.5f, 0, 0, 0, 5.5f, 0, 7.5f, 0, 0, 0, 11.5f, 0};
    EXPECT_TRUE(relu.output->hostData() == want);
    Tensor out({2, 2, 1, 3});
    Tensor bad({1, 1, 2, 3});
    EXPECT_THROW(tensorMatrixAdd(out, *a.output, bad), std::invalid_argument);
}

// ---- Model::Linear ----------------------------------------------------------------------------
struct LinearModel : nz::Model {
    InputNode input;
    LinearModel(size_t batch, size_t features, size_t out, bool relu) : input({batch, 1, features, 1}) {
        Node* x = Linear(&input, out);
        if (relu) x = ReLU(x);
        defaultOutput(x);
    }
};

TEST(Model, LinearFusedEqualsUnfusedEqualsHost) {
    const size_t batch = 37, in = 200, out = 130;
    LinearModel m(batch, in, out, true);
    EXPECT_EQ(m.parameters().size(), 2u);
    EXPECT_TRUE(m.parameters()[0]->output->shape() == Dimension(1, 1, out, in));      // weight [1,1,OUT,IN]
    EXPECT_TRUE(m.parameters()[1]->output->shape() == Dimension(1, 1, out, 1));       // bias   [1,1,OUT,1]
    auto x = randomVec(batch * in, 1, -1.f, 1.f), W = randomVec(out * in, 2, -0.2f, 0.2f), b = randomVec(out, 3, -0.3f, 0.3f);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    std::vector<double> want(batch * out);
    for (size_t n = 0; n < batch; ++n)
        for (size_t o = 0; o < out; ++o) {
            double acc = 0;
            for (size_t k = 0; k < in; ++k) acc += static_cast<double>(f16(W[o * in + k])) * f16(x[n * in + k]);
            acc += b[o];
            want[n * out + o] = acc > 0 ? acc : 0;
        }
    const auto fused = m.forward().hostData();
    EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
    EXPECT_TRUE(m.forward().shape() == Dimension(batch, 1, out, 1));
    EXPECT_TRUE(closeTo(fused, want, 1e-5));
    m.graph().setFusion(false);
    const auto unfused = m.forward().hostData();
    EXPECT_EQ(m.graph().fusedGroupCount(), 0u);
    EXPECT_TRUE(closeTo(unfused, want, 1e-5));
}

// ---- Model::Conv2d ----------------------------------------------------------------------------
struct ConvModel : nz::Model {
    InputNode input;
    ConvModel(size_t n, size_t c, size_t h, size_t w, size_t o, size_t k, size_t stride, size_t pad, bool relu)
        : input({n, c, h, w}) {
        Node* x = Conv2d(&input, o, k, k, stride, pad);
        if (relu) x = ReLU(x);
        defaultOutput(x);
    }
};

static void convCase(size_t n, size_t c, size_t h, size_t w, size_t o, size_t k, size_t stride, size_t pad) {
    ConvModel m(n, c, h, w, o, k, stride, pad, true);
    const size_t Ho = (h + 2 * pad - k) / stride + 1, Wo = (w + 2 * pad - k) / stride + 1, ckk = c * k * k;
    EXPECT_TRUE(m.parameters()[0]->output->shape() == Dimension(n, 1, ckk, o));        // one weight copy per sample
    EXPECT_TRUE(m.parameters()[1]->output->shape() == Dimension(1, 1, Ho * Wo, o));    // per-pixel-per-channel bias
    auto x = randomVec(n * c * h * w, 5, -1.f, 1.f), W1 = randomVec(ckk * o, 6, -0.3f, 0.3f);
    auto b = randomVec(Ho * Wo * o, 7, -0.5f, 0.5f);
    std::vector<float> W(n * ckk * o);
    for (size_t i = 0; i < n; ++i) std::copy(W1.begin(), W1.end(), W.begin() + i * ckk * o);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    std::vector<double> want(n * o * Ho * Wo);
    for (size_t bi = 0; bi < n; ++bi)
        for (size_t oc = 0; oc < o; ++oc)
            for (size_t ho = 0; ho < Ho; ++ho)
                for (size_t wo = 0; wo < Wo; ++wo) {
                    double acc = 0;
                    for (size_t ci = 0; ci < c; ++ci)
                        for (size_t r = 0; r < k; ++r)
                            for (size_t s = 0; s < k; ++s) {
                                const long hi = static_cast<long>(ho * stride + r) - static_cast<long>(pad);
                                const long wi = static_cast<long>(wo * stride + s) - static_cast<long>(pad);
                                if (hi < 0 || hi >= static_cast<long>(h) || wi < 0 || wi >= static_cast<long>(w)) continue;
                                acc += static_cast<double>(f16(x[((bi * c + ci) * h + hi) * w + wi])) *
                                       f16(W1[(ci * k * k + r * k + s) * o + oc]);
                            }
                    acc += b[(ho * Wo + wo) * o + oc];
                    want[((bi * o + oc) * Ho + ho) * Wo + wo] = acc > 0 ? acc : 0;
                }
    size_t inUseBefore = 0, inUseFused = 0, cached = 0, allocs = 0;
    nzhip_allocator_stats(&inUseBefore, &cached, &allocs);
    const auto fused = m.forward().hostData();
    nzhip_allocator_stats(&inUseFused, &cached, &allocs);
    EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
    EXPECT_TRUE(m.forward().shape() == Dimension(n, o, Ho, Wo));
    EXPECT_TRUE(closeTo(fused, want, 1e-5));
    // fused: the column matrix [n,1,Ho*Wo,ckk] was never allocated
    EXPECT_TRUE(inUseFused - inUseBefore < n * Ho * Wo * ckk * sizeof(float) + n * o * Ho * Wo * sizeof(float) * 2);
    m.graph().setFusion(false);
    const auto unfused = m.forward().hostData();
    EXPECT_TRUE(closeTo(unfused, want, 1e-5));
}

TEST(Model, Conv2dFusedEqualsUnfusedEqualsHost) {
    convCase(2, 3, 9, 11, 4, 3, 1, 1);        // few channels: direct stencil route
    convCase(2, 16, 12, 40, 24, 3, 1, 1);     // implicit-GEMM route
    convCase(1, 5, 10, 9, 6, 3, 2, 0);        // stride 2: workspace route
}

struct TwoLayer : nz::Model {
    InputNode input{{4, 3, 16, 16}};
    TwoLayer() {
        Node* x = Conv2d(&input, 8, 3, 3, 1, 1);
        x = ReLU(x);
        x = Conv2d(x, 2, 3, 3, 1, 1);
        x = Linear(x, 10);
        defaultOutput(x);
    }
};

TEST(Model, ConvReluConvLinearRunsFusedAndUnfusedAlike) {
    TwoLayer m;
    auto x = randomVec(4 * 3 * 16 * 16, 9, 0.f, 1.f);
    m.input.dataInject(x.begin(), x.end());
    for (size_t i = 0; i < m.parameters().size(); ++i) {
        auto p = randomVec(m.parameters()[i]->output->size(), 20 + i, -0.1f, 0.1f);
        m.parameters()[i]->dataInject(p.begin(), p.end());
    }
    const auto fused = m.forward().hostData();
    EXPECT_EQ(m.graph().fusedGroupCount(), 3u);
    EXPECT_TRUE(m.forward().shape() == Dimension(4, 1, 10, 1));
    m.graph().setFusion(false);
    const auto unfused = m.forward().hostData();
    std::vector<double> want(unfused.begin(), unfused.end());
    EXPECT_TRUE(closeTo(fused, want, 1e-4));
    std::ostringstream os;
    os << m.graph();
    EXPECT_TRUE(os.str().find("Img2Col") != std::string::npos);
}

// ---- backward of the path (test/Test.cpp:820-903, 3011-3072, 3144-3177) ---------------------------
TEST(NodeBasic, MatMulBackwardSpecial) {
    const size_t n = 2, c = 3, m = 2, k = 3, p = 2;
    InputNode input1({n, 1, m, k}, true);
    InputNode input2({1, c, k, p}, true);
    input1.output->fill(1);
    input2.output->fill(1);
    MatMulNode mul(&input1, &input2);
    mul.output->fill(1, true);
    mul.backward();
    Tensor expected1({n, 1, m, k}, true);
    Tensor expected2({1, c, k, p}, true);
    expected1.fill(1);
    expected1.fill(2 * c, true);
    expected2.fill(1);
    expected2.fill(2 * n, true);
    EXPECT_EQ(expected1, *input1.output);
    EXPECT_EQ(expected2, *input2.output);
}

TEST(NodeBasic, MatMulBackwardNormal) {
    const size_t n = 2, c = 3, m = 2, k = 3, p = 2;
    std::vector<float> Adata = {1, 2, 3, 4, 5, 6, 2, 3, 4, 5, 6, 7, 3, 4, 5, 6, 7, 8,
                                1, 2, 3, 4, 5, 6, 2, 3, 4, 5, 6, 7, 3, 4, 5, 6, 7, 8};
    std::vector<float> Bdata = {1, 4, 2, 5, 3, 6, 2, 5, 3, 6, 4, 7, 3, 6, 4, 7, 5, 8};
    std::vector<float> Cgrad(n * c * m * p, 1.f);
    std::vector<float> Agrad = {5, 7, 9, 5, 7, 9, 7, 9, 11, 7, 9, 11, 9, 11, 13, 9, 11, 13,
                                5, 7, 9, 5, 7, 9, 7, 9, 11, 7, 9, 11, 9, 11, 13, 9, 11, 13};
    std::vector<float> Bgrad = {10, 10, 14, 14, 18, 18, 14, 14, 18, 18, 22, 22, 18, 18, 22, 22, 26, 26};
    InputNode input1({n, c, m, k}, true);
    InputNode input2({1, c, k, p}, true);
    input1.dataInject(Adata.begin(), Adata.end());
    input2.dataInject(Bdata.begin(), Bdata.end());
    MatMulNode mul(&input1, &input2);
    mul.output->dataInject(Cgrad.begin(), Cgrad.end(), true);
    mul.backward();
    Tensor expected1({n, c, m, k}, true);
    Tensor expected2({1, c, k, p}, true);
    expected1.dataInject(Adata.begin(), Adata.end());
    expected1.dataInject(Agrad.begin(), Agrad.end(), true);
    expected2.dataInject(Bdata.begin(), Bdata.end());
    expected2.dataInject(Bgrad.begin(), Bgrad.end(), true);
    EXPECT_EQ(expected1, *input1.output);
    EXPECT_EQ(expected2, *input2.output);
    // the materialised-transpose form of the reference (Nodes.cu:171-181) through iGEMMBackward
    Tensor dB({1, c, k, p}, true);
    std::vector<float> At(n * c * k * m);
    for (size_t b = 0; b < n * c; ++b)
        for (size_t r = 0; r < m; ++r)
            for (size_t q = 0; q < k; ++q) At[b * m * k + q * m + r] = Adata[b * m * k + r * k + q];
    Tensor AT({n, c, k, m});
    AT.dataInject(At.begin(), At.end());
    iGEMMBackward(AT.data(), mul.output->grad(), dB.grad(), AT.shape(), mul.output->shape(), dB.shape());
    dB.dataInject(Bdata.begin(), Bdata.end());
    EXPECT_EQ(expected2, dB);
}

TEST(NodeBasic, img2colBackward) {
    const size_t n = 2, c = 3, h = 4, w = 5, k_h = 3, k_w = 3, stride = 1, pad = 1;
    const size_t H_out = (h + 2 * pad - k_h) / stride + 1, W_out = (w + 2 * pad - k_w) / stride + 1;
    std::vector<float> gradData(n * H_out * W_out * k_h * k_w * c), expectedGradData(n * c * h * w, 0.f);
    std::mt19937 gen(4);
    std::uniform_int_distribution<int> dist(1, 9);                // integers: the sum is exact in any order
    for (auto& g : gradData) g = static_cast<float>(dist(gen));
    for (size_t b = 0; b < n; ++b)
        for (size_t i = 0; i < H_out; ++i)
            for (size_t j = 0; j < W_out; ++j)
                for (size_t r = 0; r < k_h; ++r)
                    for (size_t s = 0; s < k_w; ++s)
                        for (size_t c_in = 0; c_in < c; ++c_in) {
                            const int h_in = static_cast<int>(i * stride) - static_cast<int>(pad) + static_cast<int>(r);
                            const int w_in = static_cast<int>(j * stride) - static_cast<int>(pad) + static_cast<int>(s);
                            if (h_in >= 0 && h_in < static_cast<int>(h) && w_in >= 0 && w_in < static_cast<int>(w))
                                expectedGradData[b * (c * h * w) + c_in * (h * w) + h_in * w + w_in] +=
                                    gradData[b * (H_out * W_out * k_h * k_w * c) + (i * W_out + j) * (k_h * k_w * c) +
                                             c_in * (k_h * k_w) + r * k_w + s];
                        }
    InputNode input({n, c, h, w}, true);
    input.output->clear();
    Img2ColNode result(&input, k_h, k_w, stride, pad);
    result.dataInject(gradData.begin(), gradData.end(), true);
    result.backward();
    EXPECT_TRUE(input.output->hostGrad() == expectedGradData);
}

TEST(NodeBasic, Col2imgBackward) {
    const size_t n = 2, c = 3, h = 4, w = 5;
    auto inputData = randomVec(n * c * h * w, 8, 0.1f, 0.9f);
    std::vector<float> expectedData(n * c * h * w);
    for (size_t i = 0; i < n; i++)
        for (size_t j = 0; j < c; j++)
            for (size_t k = 0; k < h; k++)
                for (size_t l = 0; l < w; l++)
                    expectedData[i * (c * h * w) + j * (h * w) + k * w + l] = inputData[i * (c * h * w) + (k * w + l) * c + j];
    InputNode input({n, 1, h * w, c}, true);
    Col2ImgNode result(&input, h, w);
    result.dataInject(expectedData.begin(), expectedData.end(), true);
    result.backward();
    EXPECT_TRUE(input.output->hostGrad() == inputData);
}

TEST(NodeBasic, AddReluOutputBackward) {
    InputNode a({2, 2, 1, 3}, true), b({1, 2, 1, 3}, true);
    a.dataInject({-1, 2, 0, 4, -5, 6, 7, -8, 9, -1, 2, 3});
    b.dataInject({1, 1, 1, 1, 1, 1});
    AddNode add(&a, &b);
    ReLUNode relu(&add);
    OutputNode out(&relu);
    add.forward();
    relu.forward();
    out.forward();
    out.backward();                                            // seeds d(relu) = 1
    relu.backward();
    add.backward();
    // a + b = {0,3,1, 5,-4,7, 8,-7,10, 0,3,4}: gradient 1 where positive
    const std::vector<float> dSum = {0, 1, 1, 1, 0, 1, 1, 0, 1, 0, 1, 1};
    EXPECT_TRUE(add.output->hostGrad() == dSum);
    EXPECT_TRUE(a.output->hostGrad() == dSum);                  // same shape: copied
    EXPECT_TRUE(b.output->hostGrad() == (std::vector<float>{1, 1, 2, 1, 1, 2}));   // summed over n
}

TEST(Model, LinearBackwardAfterFusedForward) {
    const size_t batch = 23, in = 70, out = 45;
    LinearModel m(batch, in, out, true);
    auto x = randomVec(batch * in, 31, -1.f, 1.f), W = randomVec(out * in, 32, -0.2f, 0.2f), b = randomVec(out, 33, -0.3f, 0.3f);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    m.forward();
    EXPECT_EQ(m.graph().fusedGroupCount(), 1u);                 // the MatMul / Add outputs were skipped ...
    m.backward();                                               // ... and are recomputed before the reverse pass
    std::vector<double> dW(out * in, 0.0), db(out, 0.0);
    for (size_t n = 0; n < batch; ++n)
        for (size_t o = 0; o < out; ++o) {
            double z = b[o];
            for (size_t k = 0; k < in; ++k) z += static_cast<double>(f16(W[o * in + k])) * f16(x[n * in + k]);
            if (z > 0) {                                        // d(loss)/dz = 1 where the ReLU is open
                db[o] += 1;
                for (size_t k = 0; k < in; ++k) dW[o * in + k] += f16(x[n * in + k]);
            }
        }
    EXPECT_TRUE(closeTo(m.parameters()[0]->output->hostGrad(), dW, 1e-5));
    EXPECT_TRUE(closeTo(m.parameters()[1]->output->hostGrad(), db, 1e-6));
    // a second pass accumulates onto the weight gradient (MatMul "+="), zeroGrad() resets
    m.forward();
    m.backward();
    for (auto& v : dW) v *= 2;
    EXPECT_TRUE(closeTo(m.parameters()[0]->output->hostGrad(), dW, 1e-5));
    m.graph().zeroGrad();
    for (float v : m.parameters()[0]->output->hostGrad()) EXPECT_TRUE(v == 0.f);
}

TEST(Model, Conv2dBackwardMatchesFiniteStructure) {
    // dW of a 1-output-channel 3x3 convolution with an open ReLU everywhere (positive data and
    // weights): dW[q] = sum over pixels of the column matrix entry, db[pixel] = 1.
    const size_t n = 2, c = 2, h = 5, w = 6, o = 1, k = 3;
    ConvModel m(n, c, h, w, o, k, 1, 1, true);
    auto x = randomVec(n * c * h * w, 41, 0.5f, 1.f);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->output->fill(0.25f);
    m.parameters()[1]->output->fill(0.125f);
    m.forward();
    m.backward();
    std::vector<double> dW(n * c * k * k, 0.0);
    for (size_t b = 0; b < n; ++b)
        for (size_t ci = 0; ci < c; ++ci)
            for (size_t r = 0; r < k; ++r)
                for (size_t s = 0; s < k; ++s)
                    for (size_t ho = 0; ho < h; ++ho)
                        for (size_t wo = 0; wo < w; ++wo) {
                            const long hi = static_cast<long>(ho + r) - 1, wi = static_cast<long>(wo + s) - 1;
                            if (hi < 0 || hi >= static_cast<long>(h) || wi < 0 || wi >= static_cast<long>(w)) continue;
                            dW[b * c * k * k + ci * k * k + r * k + s] += f16(x[((b * c + ci) * h + hi) * w + wi]);
                        }
    EXPECT_TRUE(closeTo(m.parameters()[0]->output->hostGrad(), dW, 1e-5));        // weights are per sample
    for (float v : m.parameters()[1]->output->hostGrad()) EXPECT_TRUE(v == static_cast<float>(n));
}

struct ConvGradModel : nz::Model {
    InputNode input;
    ConvGradModel(size_t n, size_t c, size_t h, size_t w, size_t o, size_t k, size_t stride, size_t pad, bool relu)
        : input({n, c, h, w}, true) {                               // the input wants its gradient too
        Node* x = Conv2d(&input, o, k, k, stride, pad);
        if (relu) x = ReLU(x);
        defaultOutput(x);
    }
};

static void convBackwardFusedEqualsChain(size_t n, size_t c, size_t h, size_t w, size_t o, size_t k, size_t stride,
                                         size_t pad, bool relu) {
    // integer-valued data: every gradient is exact, so the fused chain backward (one convolution for dx,
    // no column-matrix gradient) must equal the node-by-node backward bit for bit
    ConvGradModel m(n, c, h, w, o, k, stride, pad, relu);
    auto ints = [](size_t count, unsigned seed, int lo, int hi) {
        auto v = randomVec(count, seed, static_cast<float>(lo), static_cast<float>(hi) + 0.999f);
        for (auto& e : v) e = std::floor(e);
        return v;
    };
    const size_t Ho = (h + 2 * pad - k) / stride + 1, Wo = (w + 2 * pad - k) / stride + 1, ckk = c * k * k;
    auto x = ints(n * c * h * w, 61, -3, 3), W = ints(n * ckk * o, 62, -2, 2), b = ints(Ho * Wo * o, 63, -4, 4);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    m.graph().zeroGrad();
    m.forward();
    EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
    m.backward();
    const auto dx = m.input.output->hostGrad(), dW = m.parameters()[0]->output->hostGrad(),
               db = m.parameters()[1]->output->hostGrad();
    m.graph().setFusion(false);
    m.graph().zeroGrad();
    m.forward();
    m.backward();
    EXPECT_TRUE(m.input.output->hostGrad() == dx);
    EXPECT_TRUE(m.parameters()[0]->output->hostGrad() == dW);
    EXPECT_TRUE(m.parameters()[1]->output->hostGrad() == db);
    bool anyX = false;
    for (float v : dx) anyX = anyX || v != 0.f;
    EXPECT_TRUE(anyX);
}

TEST(Model, Conv2dFusedBackwardEqualsNodeChain) {
    convBackwardFusedEqualsChain(2, 3, 7, 9, 5, 3, 1, 1, true);
    convBackwardFusedEqualsChain(1, 16, 12, 40, 24, 3, 1, 1, true);   // implicit-GEMM kernels
    convBackwardFusedEqualsChain(2, 4, 6, 6, 3, 1, 1, 0, false);      // 1x1, no activation
    convBackwardFusedEqualsChain(3, 20, 8, 10, 33, 1, 1, 0, true);    // 1x1: the weight gradient is one batched product of x and the gradient
    convBackwardFusedEqualsChain(2, 3, 9, 8, 4, 3, 2, 1, true);       // stride 2: weights by the gather kernel, the data gradient from the spread-out output gradient
    convBackwardFusedEqualsChain(2, 5, 14, 12, 6, 5, 3, 2, true);     // stride 3, 5x5, rows and columns no window reaches
    convBackwardFusedEqualsChain(1, 16, 20, 24, 8, 3, 2, 0, false);   // stride 2, no padding, no activation
    convBackwardFusedEqualsChain(2, 128, 12, 12, 256, 3, 2, 1, true); // stride 2 with many channels on small images: the data gradient through the column-matrix gradient inside the fused backward
    convBackwardFusedEqualsChain(2, 6, 14, 20, 10, 5, 1, 2, true);    // 5x5: weights by the gather kernel
    convBackwardFusedEqualsChain(2, 40, 10, 136, 36, 3, 1, 1, true);  // W a multiple of 8: weights without the column matrix
}

struct RectConvGradModel : nz::Model {
    InputNode input;
    RectConvGradModel(size_t n, size_t c, size_t h, size_t w, size_t o, size_t kh, size_t kw, size_t stride, size_t pad)
        : input({n, c, h, w}, true) {
        defaultOutput(ReLU(Conv2d(&input, o, kh, kw, stride, pad)));
    }
};

TEST(Model, Conv2dFusedBackwardWithAKernelThatIsNotSquare) {
    // 2 x 3 kernel, stride 2: weights by the gather kernel, bias in one pass, the data gradient through the column-matrix
    // gradient inside the fused backward; all equal to the node chain on integers
    const size_t n = 2, c = 5, h = 10, w = 12, o = 6, kh = 2, kw = 3, stride = 2, pad = 1;
    RectConvGradModel m(n, c, h, w, o, kh, kw, stride, pad);
    auto ints = [](size_t count, unsigned seed, int lo, int hi) {
        auto v = randomVec(count, seed, static_cast<float>(lo), static_cast<float>(hi) + 0.999f);
        for (auto& e : v) e = std::floor(e);
        return v;
    };
    const size_t Ho = (h + 2 * pad - kh) / stride + 1, Wo = (w + 2 * pad - kw) / stride + 1;
    auto x = ints(n * c * h * w, 81, -3, 3), W = ints(n * c * kh * kw * o, 82, -2, 2), b = ints(Ho * Wo * o, 83, -4, 4);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    m.graph().zeroGrad();
    m.forward();
    EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
    m.backward();
    const auto dx = m.input.output->hostGrad(), dW = m.parameters()[0]->output->hostGrad(), db = m.parameters()[1]->output->hostGrad();
    m.graph().setFusion(false);
    m.graph().zeroGrad();
    m.forward();
    m.backward();
    EXPECT_TRUE(m.input.output->hostGrad() == dx);
    EXPECT_TRUE(m.parameters()[0]->output->hostGrad() == dW);
    EXPECT_TRUE(m.parameters()[1]->output->hostGrad() == db);
    bool anyX = false;
    for (float v : dx) anyX = anyX || v != 0.f;
    EXPECT_TRUE(anyX);
}

struct LinearGradModel : nz::Model {
    InputNode input;
    LinearGradModel(size_t batch, size_t features, size_t out, bool relu) : input({batch, 1, features, 1}, true) {
        Node* x = Linear(&input, out);
        if (relu) x = ReLU(x);
        defaultOutput(x);
    }
};

TEST(Model, LinearFusedBackwardEqualsNodeChain) {
    // integer-valued data: every gradient is exact, so the fused backward (mask from y, bias gradient and
    // MatMul.backward straight from the masked gradient) must equal the node-by-node backward bit for bit,
    // twice in a row (gradients are cleared in between)
    for (const bool relu : {true, false}) {
        const size_t batch = 9, in = 40, out = 24;
        LinearGradModel m(batch, in, out, relu);
        auto ints = [](size_t count, unsigned seed, int lo, int hi) {
            auto v = randomVec(count, seed, static_cast<float>(lo), static_cast<float>(hi) + 0.999f);
            for (auto& e : v) e = std::floor(e);
            return v;
        };
        auto x = ints(batch * in, 71, -3, 3), W = ints(out * in, 72, -2, 2), b = ints(out, 73, -4, 4);
        m.input.dataInject(x.begin(), x.end());
        m.parameters()[0]->dataInject(W.begin(), W.end());
        m.parameters()[1]->dataInject(b.begin(), b.end());
        std::vector<float> dx, dW, db;
        for (int pass = 0; pass < 2; ++pass) {
            m.graph().zeroGrad();
            m.forward();
            EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
            m.backward();
            dx = m.input.output->hostGrad();
            dW = m.parameters()[0]->output->hostGrad();
            db = m.parameters()[1]->output->hostGrad();
        }
        m.graph().setFusion(false);
        m.graph().zeroGrad();
        m.forward();
        m.backward();
        EXPECT_TRUE(m.input.output->hostGrad() == dx);
        EXPECT_TRUE(m.parameters()[0]->output->hostGrad() == dW);
        EXPECT_TRUE(m.parameters()[1]->output->hostGrad() == db);
        bool any = false;
        for (float v : dW) any = any || v != 0.f;
        EXPECT_TRUE(any);
    }
}

// ---- weight images kept between forward passes ------------------------------------------------------------
TEST(Model, WeightImagesAreKeptWhileWeightsStayUntouchedAndRebuiltAfterAChange) {
    // Linear at a size that takes the two-pass route (the fp16 image of W is its B operand), and a Conv2d on the
    // implicit-GEMM kernels: three forward passes build each image once and give the same values; new weights
    // (dataInject, an optimizer step) are seen by the very next forward pass, which must equal the unfused graph.
    {
        const size_t batch = 4096, in = 1024, out = 4096;
        LinearModel m(batch, in, out, true);
        auto x = randomVec(batch * in, 11, -1.f, 1.f), W = randomVec(out * in, 12, -0.08f, 0.08f), b = randomVec(out, 13, -0.03f, 0.03f);
        m.input.dataInject(x.begin(), x.end());
        m.parameters()[0]->dataInject(W.begin(), W.end());
        m.parameters()[1]->dataInject(b.begin(), b.end());
        const auto first = m.forward().hostData();
        EXPECT_EQ(m.graph().weightImageBuilds(), 1ull);
        EXPECT_TRUE(m.forward().hostData() == first);
        EXPECT_TRUE(m.forward().hostData() == first);
        EXPECT_EQ(m.graph().weightImageBuilds(), 1ull);
        auto W2 = randomVec(out * in, 14, -0.08f, 0.08f);
        m.parameters()[0]->dataInject(W2.begin(), W2.end());
        const auto second = m.forward().hostData();
        EXPECT_EQ(m.graph().weightImageBuilds(), 2ull);
        EXPECT_TRUE(second != first);
        m.graph().setFusion(false);
        EXPECT_TRUE(closeTo(m.forward().hostData(), std::vector<double>(second.begin(), second.end()), 1e-5));
    }
    {
        ConvModel m(8, 16, 64, 64, 32, 3, 1, 1, true);           // enough patches for the implicit-GEMM kernel
        auto x = randomVec(8 * 16 * 64 * 64, 21, -1.f, 1.f);
        m.input.dataInject(x.begin(), x.end());
        auto W = randomVec(8 * 16 * 9 * 32, 22, -0.2f, 0.2f), b = randomVec(64 * 64 * 32, 23, -0.1f, 0.3f);
        m.parameters()[0]->dataInject(W.begin(), W.end());
        m.parameters()[1]->dataInject(b.begin(), b.end());
        const auto first = m.forward().hostData();
        EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
        EXPECT_EQ(m.graph().weightImageBuilds(), 1ull);
        EXPECT_TRUE(m.forward().hostData() == first);
        EXPECT_EQ(m.graph().weightImageBuilds(), 1ull);
        m.backward();
        nz::opt::SGD optimizer(0.05f);
        m.update(&optimizer);
        const auto second = m.forward().hostData();
        EXPECT_EQ(m.graph().weightImageBuilds(), 2ull);
        EXPECT_TRUE(second != first);
        m.graph().setFusion(false);
        EXPECT_TRUE(closeTo(m.forward().hostData(), std::vector<double>(second.begin(), second.end()), 1e-5));
    }
}

// ---- fp32 matmul and optimizers (test/Test.cpp:119-184, 2230-2265, 2398-2452, 2816-2878) ------------
TEST(TensorBasic, TensorMultiplicationTest) {
    Tensor tensor1({2, 1, 2, 3});
    Tensor tensor2({1, 3, 3, 2});
    tensor1.dataInject(kData1.begin(), kData1.end());
    tensor2.dataInject(kData2.begin(), kData2.end());
    Tensor result = tensor1 * tensor2;
    Tensor expected({2, 3, 2, 2});
    expected.dataInject(kExpected.begin(), kExpected.end());
    EXPECT_TRUE(result == expected);
    // the tensor-core path agrees with it on integers (test/Test.cpp:708-751)
    Tensor tc({2, 3, 2, 2});
    GEMMTensorCore(tc, tensor1, tensor2);
    EXPECT_EQ(tc, result);
    // no fp16 rounding on this path: 1 + 2^-12 survives
    Tensor a({1, 1, 1, 1}), b({1, 1, 1, 1});
    a.fill(1.f + 1.f / 4096.f);
    b.fill(1.f);
    EXPECT_TRUE((a * b).hostData()[0] == 1.f + 1.f / 4096.f);
    Tensor bad({1, 1, 4, 2});
    EXPECT_THROW(tensor1 * bad, std::invalid_argument);
}

TEST(OptimizerBasic, SGDTest) {
    const size_t n = 2, c = 3, h = 3, w = 4;
    const float learningRate = 0.01f;
    auto data = randomVec(n * c * h * w, 51, -10.f, 10.f), grad = randomVec(n * c * h * w, 52, -10.f, 10.f);
    std::vector<float> expectedData(data.size());
    for (size_t i = 0; i < data.size(); i++) expectedData[i] = data[i] - learningRate * grad[i];
    InputNode input({n, c, h, w}, true);
    input.dataInject(data.begin(), data.end());
    input.dataInject(grad.begin(), grad.end(), true);
    nz::opt::SGD optimizer(learningRate);
    optimizer.step(&input);
    Tensor expected({n, c, h, w}, true);
    expected.dataInject(expectedData.begin(), expectedData.end());
    expected.dataInject(grad.begin(), grad.end(), true);
    EXPECT_EQ(*input.output, expected);
}

TEST(OptimizerBasic, AdamTest) {
    const size_t n = 2, c = 3, h = 3, w = 4;
    const float learningRate = 0.01f, beta1 = 0.9f, beta2 = 0.999f, epsilon = 1e-6f;
    auto data = randomVec(n * c * h * w, 53, -10.f, 10.f), grad = randomVec(n * c * h * w, 54, -10.f, 10.f);
    std::vector<float> expectedData(data), m(data.size(), 0.f), v(data.size(), 0.f);
    for (int it = 1; it <= 2; it++)
        for (size_t i = 0; i < data.size(); i++) {
            m[i] = beta1 * m[i] + (1 - beta1) * grad[i];
            v[i] = beta2 * v[i] + (1 - beta2) * grad[i] * grad[i];
            const float modified_m = m[i] / (1 - std::pow(beta1, it));
            const float modified_v = v[i] / (1 - std::pow(beta2, it));
            expectedData[i] = expectedData[i] - (learningRate / (std::sqrt(modified_v) + epsilon)) * modified_m;
        }
    InputNode input({n, c, h, w}, true);
    input.dataInject(data.begin(), data.end());
    input.dataInject(grad.begin(), grad.end(), true);
    nz::opt::Adam optimizer(learningRate, beta1, beta2);
    optimizer.step(&input);
    optimizer.step(&input);
    Tensor expected({n, c, h, w}, true);
    expected.dataInject(expectedData.begin(), expectedData.end());
    expected.dataInject(grad.begin(), grad.end(), true);
    EXPECT_EQ(*input.output, expected);
}

struct SGDTestModel : nz::Model {                               // test/Test.cpp:2816-2835
    InputNode input1{{5, 3, 12, 1}, true};
    InputNode input2{{5, 3, 12, 1}, false};
    SGDTestModel() {
        auto x = Add(&input1, &input2);
        defaultOutput(x);
    }
};

TEST(Model, SGDOptimize) {
    const size_t count = 5 * 3 * 12;
    const float lr = 0.01f;
    auto d1 = randomVec(count, 61, 0.1f, 0.9f), d2 = randomVec(count, 62, 0.1f, 0.9f), g1 = randomVec(count, 63, 0.1f, 0.9f);
    std::vector<float> expectedData(count);
    for (size_t i = 0; i < count; i++) expectedData[i] = d1[i] - lr * g1[i];
    SGDTestModel model{};
    model.input1.dataInject(d1.begin(), d1.end());
    model.input2.dataInject(d2.begin(), d2.end());
    model.input1.dataInject(g1.begin(), g1.end(), true);
    nz::opt::SGD optimizer(lr);
    model.update(&optimizer);
    Tensor expected({5, 3, 12, 1}, true);
    expected.dataInject(expectedData.begin(), expectedData.end());
    EXPECT_EQ(expected, *model.input1.output);                   // gradient was reset by update()
}

TEST(Model, AdamThroughUpdateCountsStepsLikeTheReference) {
    // ComputeGraph::update of the reference calls Adam::step for EVERY node whose output carries a gradient
    // (src/ComputeGraph.cu:541-547), and Adam counts calls, not updates (src/Optimizer.cu:86-101): the t of
    // a parameter's bias corrections is its position among those nodes, plus their number per earlier update.
    // Restated here on the host for the two parameters of a Linear layer over two updates.
    const size_t batch = 6, in = 20, out = 12;
    LinearModel m(batch, in, out, true);
    auto x = randomVec(batch * in, 301, -1.f, 1.f), W = randomVec(out * in, 302, -0.5f, 0.5f), b = randomVec(out, 303, -0.3f, 0.3f);
    m.input.dataInject(x.begin(), x.end());
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    const float lr = 0.01f, beta1 = 0.9f, beta2 = 0.999f, eps = 1e-6f;
    nz::opt::Adam optimizer(lr, beta1, beta2);
    const auto& nodes = m.graph().getNodes();
    size_t per_update = 0;
    std::vector<std::vector<float>> data = {W, b}, mo = {std::vector<float>(W.size(), 0.f), std::vector<float>(b.size(), 0.f)}, ve = mo;
    for (int update = 0; update < 2; ++update) {
        m.forward();
        m.backward();
        if (update == 0) {                                       // counted once the graph has run: every node has its output
            for (Node* n : nodes) per_update += n->output && n->output->requiresGrad();
            EXPECT_TRUE(per_update > 2);                         // hidden activations and the output node count too
        }
        std::vector<std::vector<float>> grads;
        for (int k = 0; k < 2; ++k) grads.push_back(m.parameters()[k]->output->hostGrad());
        int t = update * (int)per_update;
        for (Node* n : nodes) {                                   // the reference's loop
            if (!(n->output && n->output->requiresGrad())) continue;
            ++t;
            for (int k = 0; k < 2; ++k) {
                if (n != m.parameters()[k]) continue;
                const float c1 = 1.0f - std::pow(beta1, (float)t), c2 = 1.0f - std::pow(beta2, (float)t);
                for (size_t i = 0; i < data[k].size(); ++i) {
                    const float g = grads[k][i];
                    mo[k][i] = mo[k][i] * beta1 + g * (1 - beta1);
                    ve[k][i] = ve[k][i] * beta2 + g * g * (1 - beta2);
                    data[k][i] -= lr * (mo[k][i] / c1) / (std::sqrt(ve[k][i] / c2) + eps);
                }
            }
        }
        m.update(&optimizer);
    }
    for (int k = 0; k < 2; ++k) {
        const auto got = m.parameters()[k]->output->hostData();
        double worst = 0;
        for (size_t i = 0; i < got.size(); ++i) worst = std::max(worst, (double)std::fabs(got[i] - data[k][i]));
        // counting only the stepped leaves instead (t = 2 where the reference has 3) moves entries by about 4e-3
        EXPECT_TRUE(worst < 2e-5);
    }
}

TEST(Model, LinearTrainingStepLowersTheOutputSum) {
    // forward -> backward (d(sum of outputs)) -> SGD: the sum of the outputs must go down
    LinearModel m(16, 40, 24, false);
    auto x = randomVec(16 * 40, 71, -1.f, 1.f);
    m.input.dataInject(x.begin(), x.end());
    auto total = [&] {
        double s = 0;
        for (float v : m.forward().hostData()) s += v;
        return s;
    };
    const double before = total();
    m.backward();
    nz::opt::SGD optimizer(0.01f);
    m.update(&optimizer);
    EXPECT_TRUE(total() < before);
}

TEST(Model, ConvTrainingStepsLowerTheOutputSum) {
    // Conv2d + ReLU: forward -> fused backward (weights straight from x and dy, data gradient as one convolution)
    // -> Adam, three times; the sum of the outputs goes down every step
    ConvModel m(2, 16, 12, 24, 20, 3, 1, 1, true);
    auto x = randomVec(2 * 16 * 12 * 24, 91, -1.f, 1.f);
    m.input.dataInject(x.begin(), x.end());
    auto W = randomVec(2 * 16 * 9 * 20, 92, 0.0f, 0.2f), b = randomVec(12 * 24 * 20, 93, 0.1f, 0.3f);
    m.parameters()[0]->dataInject(W.begin(), W.end());
    m.parameters()[1]->dataInject(b.begin(), b.end());
    auto total = [&] {
        double s = 0;
        for (float v : m.forward().hostData()) s += v;
        return s;
    };
    nz::opt::Adam optimizer(0.01f, 0.9f, 0.999f);
    double before = total();
    EXPECT_EQ(m.graph().fusedGroupCount(), 1u);
    for (int step = 0; step < 3; ++step) {
        m.backward();
        m.update(&optimizer);
        const double after = total();
        EXPECT_TRUE(after < before);
        before = after;
    }
}

// ---- softmax (test/Test.cpp:1733-1870) -------------------------------------------------------------
TEST(NodeBasic, SoftmaxForwardJacobianBackward) {
    const size_t n = 2, c = 3, h = 12, w = 1;
    auto inputData = randomVec(n * c * h * w, 81, -10.f, 10.f), grad = randomVec(n * c * h * w, 82, -10.f, 10.f);
    std::vector<float> outputData(inputData.size()), jacobianData(n * c * h * h);
    for (size_t i = 0; i < n * c; i++) {
        float sum = 0.0f;
        for (size_t k = 0; k < h; k++) sum += std::exp(inputData[i * h + k]);
        for (size_t k = 0; k < h; k++) outputData[i * h + k] = std::exp(inputData[i * h + k]) / sum;
        for (size_t x = 0; x < h; x++)
            for (size_t y = 0; y < h; y++)
                jacobianData[i * h * h + x * h + y] = x == y ? outputData[i * h + x] * (1 - outputData[i * h + x])
                                                             : -outputData[i * h + x] * outputData[i * h + y];
    }
    InputNode input({n, c, h, w}, true);
    input.dataInject(inputData.begin(), inputData.end());
    SoftmaxNode softmax(&input);
    softmax.forward();
    Tensor expectedOut({n, c, h, w}, true);
    expectedOut.dataInject(outputData.begin(), outputData.end());
    EXPECT_EQ(expectedOut, *softmax.output);
    Tensor probs({n, c, h, w});
    probs.dataInject(outputData.begin(), outputData.end());
    Tensor expectedJ({n, c, h, h});
    expectedJ.dataInject(jacobianData.begin(), jacobianData.end());
    EXPECT_EQ(softmaxJacobian(probs), expectedJ);
    // backward: Jacobian x gradient through the fp16 GEMM, exactly what the reference's test builds
    Tensor outputGrad({n, c, h, w}), inputGrad({n, c, h, w});
    outputGrad.dataInject(grad.begin(), grad.end());
    GEMMTensorCore(inputGrad, expectedJ, outputGrad);
    const auto want = inputGrad.hostData();
    softmax.output->dataInject(grad.begin(), grad.end(), true);
    softmax.backward();
    std::vector<double> wantD(want.begin(), want.end());
    EXPECT_TRUE(closeTo(input.output->hostGrad(), wantD, 1e-4));
    InputNode notVector({1, 1, 2, 2});
    EXPECT_THROW(SoftmaxNode bad(&notVector), std::invalid_argument);
}

// ---- pooling, loss, expand: the loop nests of the reference's tests (test/Test.cpp:3179-3385, 1937-1999, 2663-2730) ----
TEST(NodeBasic, AveragePoolingForwardBackward) {
    const size_t n = 2, c = 3, h = 9, w = 7, pool = 3, stride = 2, pad = 1;
    const size_t Ho = (h + 2 * pad - pool) / stride + 1, Wo = (w + 2 * pad - pool) / stride + 1;
    auto x = randomVec(n * c * h * w, 101, 0.1f, 0.9f), g = randomVec(n * c * Ho * Wo, 102, 0.1f, 0.9f);
    std::vector<float> want(n * c * Ho * Wo, 0.f);
    std::vector<double> wantGrad(n * c * h * w, 0.0);
    for (size_t pl = 0; pl < n * c; pl++)
        for (size_t k = 0; k < Ho; k++)
            for (size_t l = 0; l < Wo; l++) {
                const long long h0 = (long long)(k * stride) - (long long)pad, w0 = (long long)(l * stride) - (long long)pad;
                size_t count = 0;
                float sum = 0.f;
                for (size_t r = 0; r < pool; r++)
                    for (size_t q = 0; q < pool; q++) {
                        const long long hi = h0 + (long long)r, wi = w0 + (long long)q;
                        if (hi >= 0 && hi < (long long)h && wi >= 0 && wi < (long long)w) {
                            sum += x[pl * h * w + hi * w + wi];
                            count++;
                        }
                    }
                want[pl * Ho * Wo + k * Wo + l] = count ? sum / static_cast<float>(count) : 0.f;
                for (size_t r = 0; r < pool; r++)
                    for (size_t q = 0; q < pool; q++) {
                        const long long hi = h0 + (long long)r, wi = w0 + (long long)q;
                        if (hi >= 0 && hi < (long long)h && wi >= 0 && wi < (long long)w)
                            wantGrad[pl * h * w + hi * w + wi] += g[pl * Ho * Wo + k * Wo + l] / static_cast<float>(count);
                    }
            }
    InputNode input({n, c, h, w}, true);
    input.dataInject(x.begin(), x.end());
    AveragePoolingNode poolNode(&input, pool, stride, pad);
    poolNode.forward();
    EXPECT_TRUE(poolNode.output->hostData() == want);
    input.output->zeroGrad();
    poolNode.output->dataInject(g.begin(), g.end(), true);
    poolNode.backward();
    EXPECT_TRUE(closeTo(input.output->hostGrad(), wantGrad, 1e-6));
    Tensor t({n, c, h, w});
    t.dataInject(x.begin(), x.end());
    EXPECT_TRUE(tensorAveragePooling(t, pool, stride, pad).hostData() == want);
    EXPECT_THROW(AveragePoolingNode bad(&input, 12, 1, 0), std::invalid_argument);
}

TEST(NodeLoss, BCEForwardBackward) {
    const size_t n = 2, c = 3, h = 12, w = 5, total = n * c * h * w;
    auto predict = randomVec(total, 103, 0.1f, 0.9f), target = randomVec(total, 104, 0.1f, 0.9f);
    double lossWant = 0;
    std::vector<double> gradWant(total);
    for (size_t i = 0; i < total; i++) {
        lossWant += -target[i] * std::log((double)predict[i]) - (1 - target[i]) * std::log(1.0 - predict[i]);
        gradWant[i] = ((predict[i] - target[i]) / ((double)predict[i] * (1 - predict[i]))) / total;
    }
    lossWant /= total;
    InputNode input1({n, c, h, w}, true), input2({n, c, h, w});
    input1.dataInject(predict.begin(), predict.end());
    input2.dataInject(target.begin(), target.end());
    BinaryCrossEntropyNode bce(&input1, &input2);
    bce.forward();
    EXPECT_TRUE(std::fabs(bce.getLoss() - lossWant) < 1e-5 * lossWant);
    bce.forward();                                            // the loss of a pass, not a running total
    EXPECT_TRUE(std::fabs(bce.getLoss() - lossWant) < 1e-5 * lossWant);
    bce.backward();
    EXPECT_TRUE(closeTo(input1.output->hostGrad(), gradWant, 1e-6));
    InputNode other({n, c, h, w + 1});
    EXPECT_THROW(BinaryCrossEntropyNode bad(&input1, &other), std::invalid_argument);
}

TEST(NodeLoss, MSEForwardBackward) {                       // test/Test.cpp:1872-1935
    const size_t n = 2, c = 3, h = 12, w = 5, total = n * c * h * w;
    auto predict = randomVec(total, 107, 0.1f, 0.9f), target = randomVec(total, 108, 0.1f, 0.9f);
    double lossWant = 0;
    std::vector<double> gradWant(total);
    for (size_t i = 0; i < total; i++) {
        lossWant += ((double)predict[i] - target[i]) * ((double)predict[i] - target[i]);
        gradWant[i] = 2 * ((double)predict[i] - target[i]) / total;
    }
    lossWant /= total;
    InputNode input1({n, c, h, w}, true), input2({n, c, h, w});
    input1.dataInject(predict.begin(), predict.end());
    input2.dataInject(target.begin(), target.end());
    MeanSquaredErrorNode mse(&input1, &input2);
    mse.forward();
    EXPECT_TRUE(std::fabs(mse.getLoss() - lossWant) < 1e-5 * lossWant);
    mse.backward();
    EXPECT_TRUE(closeTo(input1.output->hostGrad(), gradWant, 1e-6));
}

// Linear -> ReLU -> Linear with an MSE loss against a target given once for the whole batch
struct RegressionModel : nz::Model {
    InputNode input, target;
    RegressionModel() : input({8, 1, 64, 1}), target({1, 1, 4, 1}) {
        Node* x = Linear(&input, 32);
        x = ReLU(x);
        x = Linear(x, 4);
        MSELoss(x, &target);
    }
};

TEST(Model, MSELossTrainingLowersTheLoss) {
    RegressionModel m;
    auto x = randomVec(8 * 64, 131, -1.f, 1.f);
    m.input.dataInject(x.begin(), x.end());
    m.target.dataInject({0.5f, -0.25f, 1.0f, 0.0f});
    unsigned seed = 140;
    for (auto* p : m.parameters()) {
        auto v = randomVec(p->output->size(), seed++, -0.2f, 0.2f);
        p->dataInject(v.begin(), v.end());
    }
    nz::opt::SGD optimizer(0.05f);
    m.forward();
    float before = m.getLoss();
    EXPECT_TRUE(before > 0.f);
    for (int step = 0; step < 10; ++step) {
        m.backward();
        m.update(&optimizer);
        m.forward();
        EXPECT_TRUE(m.getLoss() < before);
        before = m.getLoss();
    }
}

TEST(NodeBasic, ExpandForwardBackward) {
    const size_t c = 2, h = 3, w = 4, batch = 5, per = c * h * w;
    auto x = randomVec(per, 105, -1.f, 1.f), g = randomVec(per * batch, 106, -1.f, 1.f);
    InputNode input({1, c, h, w}, true);
    input.dataInject(x.begin(), x.end());
    ExpandNode expand(&input, batch);
    expand.forward();
    const auto out = expand.output->hostData();
    for (size_t i = 0; i < per * batch; i++) EXPECT_TRUE(out[i] == x[i % per]);
    input.output->zeroGrad();
    expand.output->dataInject(g.begin(), g.end(), true);
    expand.backward();
    std::vector<double> want(per, 0.0);
    for (size_t i = 0; i < per * batch; i++) want[i % per] += g[i];
    EXPECT_TRUE(closeTo(input.output->hostGrad(), want, 1e-6));
    InputNode batched({2, c, h, w});
    EXPECT_THROW(ExpandNode bad(&batched, 3), std::invalid_argument);
}

// The network of the reference's README (README.md:62-90) at a reduced image size: Conv2d -> ReLU -> Conv2d ->
// AvgPool2d -> Linear -> Softmax -> BCELoss, trained with Adam. The labels are given once and expanded to the batch.
struct ReadmeModel : nz::Model {
    InputNode input, target;
    ReadmeModel(size_t n, size_t h, size_t w) : input({n, 3, h, w}), target({1, 1, 16, 1}) {
        Node* x = Conv2d(&input, 1, 3, 3, 1, 1);
        x = ReLU(x);
        x = Conv2d(x, 1, 3, 3, 1, 1);
        x = AvgPool2d(x, 5, 2);
        x = Linear(x, 16);
        x = Softmax(x);
        BCELoss(x, &target);
    }
    Node* checkExpand(Node* t) { return TargetExpand(t, Tensor::shape_type{4, 1, 16, 1}); }
};

TEST(Model, ReadmeExampleTrains) {
    const size_t n = 4, h = 40, w = 48;
    ReadmeModel m(n, h, w);
    auto x = randomVec(n * 3 * h * w, 111, 0.f, 1.f);
    m.input.dataInject(x.begin(), x.end());
    std::vector<float> labels(16, 0.02f);
    labels[3] = 0.7f;
    m.target.dataInject(labels.begin(), labels.end());
    // small positive parameters keep the ReLU alive and the softmax away from saturation
    unsigned seed = 120;
    for (auto* p : m.parameters()) {
        auto v = randomVec(p->output->size(), seed++, 0.0f, 0.05f);
        p->dataInject(v.begin(), v.end());
    }
    nz::opt::Adam optimizer(0.01f, 0.9f, 0.999f);
    m.forward();
    const float first = m.getLoss();
    EXPECT_TRUE(std::isfinite(first) && first > 0.f);
    float last = first;
    for (int epoch = 0; epoch < 8; ++epoch) {
        m.backward();
        m.update(&optimizer);
        m.forward();
        last = m.getLoss();
        EXPECT_TRUE(std::isfinite(last));
    }
    EXPECT_TRUE(last < first);
    // the same steps without the fused chains reach the same loss
    ReadmeModel r(n, h, w);
    r.graph().setFusion(false);
    r.input.dataInject(x.begin(), x.end());
    r.target.dataInject(labels.begin(), labels.end());
    seed = 120;
    for (auto* p : r.parameters()) {
        auto v = randomVec(p->output->size(), seed++, 0.0f, 0.05f);
        p->dataInject(v.begin(), v.end());
    }
    nz::opt::Adam optimizer2(0.01f, 0.9f, 0.999f);
    r.forward();
    EXPECT_TRUE(std::fabs(r.getLoss() - first) <= 1e-5f * first);
    for (int epoch = 0; epoch < 8; ++epoch) {
        r.backward();
        r.update(&optimizer2);
        r.forward();
    }
    EXPECT_TRUE(std::fabs(r.getLoss() - last) <= 2e-3f * std::fabs(last));
    InputNode wrong({2, 1, 16, 1});
    EXPECT_THROW(m.checkExpand(&wrong), std::runtime_error);
}

TEST(TensorBasic, ZeroGradIsLazyButObservable) {
    // zeroGrad() defers the clear; every reader still sees zeros, and a full overwrite replaces it
    Tensor t({1, 1, 2, 3}, true);
    std::vector<float> g = {1, 2, 3, 4, 5, 6};
    t.dataInject(g.begin(), g.end(), true);
    EXPECT_TRUE(t.hostGrad() == g);
    t.zeroGrad();
    EXPECT_TRUE(t.hostGrad() == std::vector<float>(6, 0.f));
    t.dataInject(g.begin(), g.end(), true);
    t.zeroGrad();
    std::vector<float> h = {6, 5, 4, 3, 2, 1};
    EXPECT_EQ(nzhip_memcpy_h2d(t.gradOverwrite(), h.data(), 6 * sizeof(float)), 0);
    EXPECT_TRUE(t.hostGrad() == h);                           // the pending clear did not run over the new values
    t.zeroGrad();
    Tensor copy(t);                                           // a copy of a cleared gradient is cleared
    EXPECT_TRUE(copy.hostGrad() == std::vector<float>(6, 0.f));
    // accumulation after zeroGrad starts from zero: d(relu)/dx of ones through a node that adds (MatMul)
    InputNode a({1, 1, 2, 2}, true), b({1, 1, 2, 2}, true);
    a.dataInject({1, 2, 3, 4});
    b.dataInject({1, 0, 0, 1});
    MatMulNode mm(&a, &b);
    mm.forward();
    for (int pass = 0; pass < 2; ++pass) {
        a.output->zeroGrad();
        b.output->zeroGrad();
        mm.output->dataInject({1, 1, 1, 1}, true);
        mm.backward();
        EXPECT_TRUE(a.output->hostGrad() == (std::vector<float>{1, 1, 1, 1}));   // dC * B^T, not twice that on pass 2
    }
}

TEST(Runtime, AllocatorCachesAndErrorsSurfaceAsExceptions) {
    size_t inUse0 = 0, cached0 = 0, allocs0 = 0, inUse1 = 0, cached1 = 0, allocs1 = 0;
    {
        Tensor t({1, 1, 256, 256});
        t.clear();
    }
    nzhip_allocator_stats(&inUse0, &cached0, &allocs0);
    {
        Tensor t({1, 1, 256, 256});
        t.clear();                                            // served from the cache: no new device allocation
    }
    nzhip_allocator_stats(&inUse1, &cached1, &allocs1);
    EXPECT_EQ(allocs0, allocs1);
    EXPECT_EQ(inUse0, inUse1);
    float* out = nullptr;
    EXPECT_THROW(iRELU(out, out, 16), std::invalid_argument);  // C-ABI status -> exception, nothing launched
}

int main(int argc, char** argv) { return mini::run_all(argc > 1 ? argv[1] : nullptr); }
