// GPU-free tests of the nz:: host layer: Dimension semantics, the shape checks node
// constructors perform (tensors allocate lazily, so no device is touched), graph ordering and
// fusion planning, and the caching allocator's bookkeeping against a fake backend from several
// threads. The error behaviours are the reference's (src/Dimension.cu:40-45, 67-134;
// src/Nodes.cu:80-86, 149-152, 555-558; src/Tensor.cu:445-450).
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <set>
#include <thread>

#include "../../csrc/nz_pool_allocator.hpp"
#include "NeuZephyr/ComputeGraph.cuh"
#include "NeuZephyr/Model.cuh"
#include "NeuZephyr/Nodes.cuh"
#include "mini_test.hpp"

using namespace nz::data;
using namespace nz::nodes;
using namespace nz::nodes::io;
using namespace nz::nodes::calc;

TEST(Dimension, StridesSizeAndIndexing) {
    Dimension d(2, 3, 4, 5);
    EXPECT_EQ(d.size(), 120u);
    EXPECT_EQ(d.getStride(0), 60u);
    EXPECT_EQ(d.getStride(1), 20u);
    EXPECT_EQ(d.getStride(2), 5u);
    EXPECT_EQ(d.getStride(3), 1u);
    EXPECT_THROW(d.getStride(4), std::out_of_range);
    EXPECT_THROW(d[4], std::out_of_range);
    d[2] = 8;
    EXPECT_EQ(d.H(), 8u);
    EXPECT_EQ(d.getStride(1), 40u);
    EXPECT_TRUE(Dimension() == Dimension(1, 1, 1, 1));
    EXPECT_TRUE(Dimension(std::vector<size_t>{1, 2, 3, 4}) == Dimension(1, 2, 3, 4));
}

TEST(Dimension, BroadcastLooksAtNAndCOnly) {
    EXPECT_TRUE(Dimension(2, 1, 4, 5).isBroadcastCompatible(Dimension(1, 3, 9, 9)));   // h, w ignored
    EXPECT_TRUE(!Dimension(2, 1, 4, 5).isBroadcastCompatible(Dimension(3, 1, 4, 5)));
    EXPECT_TRUE(Dimension(2, 1, 4, 5).Broadcast(Dimension(1, 3, 4, 5)) == Dimension(2, 3, 4, 5));
    EXPECT_THROW(Dimension(2, 1, 4, 5).Broadcast(Dimension(3, 1, 4, 5)), std::invalid_argument);
    Dimension r(2, 3, 4, 5);
    EXPECT_TRUE(r.reshape(Dimension(6, 1, 20, 1)));
    EXPECT_TRUE(!r.reshape(Dimension(6, 1, 21, 1)));
}

TEST(Nodes, ShapeErrorsMatchTheReference) {
    InputNode a({2, 1, 2, 3}), b({1, 3, 3, 2}), bad_k({1, 3, 4, 2}), bad_n({3, 1, 3, 2});
    MatMulNode ok(&a, &b);
    EXPECT_TRUE(ok.output->shape() == Dimension(2, 3, 2, 2));
    EXPECT_TRUE(ok.type == "MatMul");
    EXPECT_THROW(MatMulNode(&a, &bad_k), std::invalid_argument);
    EXPECT_THROW(MatMulNode(&a, &bad_n), std::invalid_argument);
    try {
        MatMulNode m(&a, &bad_k);
    } catch (const std::invalid_argument& e) {
        EXPECT_TRUE(std::string(e.what()) == "Shapes are not broadcast compatible.");
    }
    InputNode p({2, 3, 4, 4}), q({1, 1, 4, 4}), q_bad({1, 1, 4, 5});
    AddNode add(&p, &q);
    EXPECT_TRUE(add.output->shape() == Dimension(2, 3, 4, 4));
    EXPECT_THROW(AddNode(&p, &q_bad), std::invalid_argument);
    EXPECT_THROW(ReshapeNode(&p, Dimension(2, 3, 4, 5)), std::invalid_argument);
    Img2ColNode col(&p, 3, 3, 1, 1);
    EXPECT_TRUE(col.output->shape() == Dimension(2, 1, 16, 27));
    Img2ColNode col2(&p, 2, 2, 2, 0);
    EXPECT_TRUE(col2.output->shape() == Dimension(2, 1, 4, 12));
    InputNode colres({2, 1, 16, 7});
    Col2ImgNode c2i(&colres, 4, 4);
    EXPECT_TRUE(c2i.output->shape() == Dimension(2, 7, 4, 4));
    Tensor t({1, 1, 2, 2});
    EXPECT_THROW(t.grad(), std::runtime_error);
    ok.backward();                          // no operand wants a gradient: nothing is launched
}

TEST(Graph, TopologicalOrderCyclesAndOutputs) {
    nz::graph::ComputeGraph g;
    InputNode a({1, 1, 2, 3}), b({1, 1, 3, 2});
    MatMulNode mm(&a, &b);
    ReLUNode relu(&mm);
    OutputNode out(&relu);
    g.addNode(&relu);                       // inserted out of order on purpose
    g.addNode(&mm);
    g.addInput(&a);
    g.addInput(&b);
    EXPECT_THROW(g.getOutputNode(), std::runtime_error);
    g.addOutput(&out);
    g.topologicalSort();
    EXPECT_TRUE(g.isSorted());
    EXPECT_TRUE(g.getOutputNode() == &out);
    EXPECT_TRUE(g.inGraph(&mm) && g.getNodes().size() == 5);
    // a cycle is reported
    nz::graph::ComputeGraph cyc;
    InputNode x({1, 1, 2, 2});
    ReLUNode r1(&x);
    ReLUNode r2(&r1);
    r1.inputs[0] = &r2;
    cyc.addNode(&r1);
    cyc.addNode(&r2);
    EXPECT_THROW(cyc.topologicalSort(), std::runtime_error);
    g.backward();                           // sorted, one output, no gradients wanted: a no-op
    EXPECT_THROW(cyc.backward(), std::runtime_error);       // "Graph is not sorted"
    nz::graph::ComputeGraph none;
    none.addNode(&mm);
    none.addInput(&a);
    none.addInput(&b);
    none.topologicalSort();
    EXPECT_THROW(none.backward(), std::runtime_error);      // "No output node"
}

// ---- caching allocator against a fake backend ------------------------------------------------
struct FakeBackend {
    std::atomic<size_t>* live;
    std::atomic<size_t>* allocs;
    size_t budget;
    int raw_alloc(void** p, size_t bytes) {
        if (live->load() + bytes > budget) {
            *p = nullptr;
            return 2;   // "out of memory"
        }
        *p = std::malloc(64);   // bookkeeping only: holds the size tag, never the payload
        std::memcpy(*p, &bytes, sizeof(bytes));
        live->fetch_add(bytes);
        allocs->fetch_add(1);
        return 0;
    }
    int raw_free(void* p) {
        size_t bytes;
        std::memcpy(&bytes, p, sizeof(bytes));
        live->fetch_sub(bytes);
        std::free(p);
        return 0;
    }
};

TEST(Pool, SizeClassesReuseAndPerStreamCaching) {
    std::atomic<size_t> live{0}, allocs{0};
    {
        nzhip::PoolAllocator<FakeBackend> pool(FakeBackend{&live, &allocs, size_t(1) << 40});
        EXPECT_EQ(nzhip::pool_round_size(1), 512u);
        EXPECT_EQ(nzhip::pool_round_size(513), 1024u);
        EXPECT_EQ(nzhip::pool_round_size((size_t(1) << 20) + 1), size_t(2) << 20);
        void *a = nullptr, *b = nullptr, *c = nullptr;
        EXPECT_EQ(pool.allocate(&a, 1000, 7), 0);
        EXPECT_EQ(pool.free_async(a, 7), 0);
        EXPECT_EQ(pool.allocate(&b, 900, 7), 0);          // same class, same stream: reused
        EXPECT_TRUE(a == b);
        EXPECT_EQ(pool.free_async(b, 7), 0);
        EXPECT_EQ(pool.allocate(&c, 900, 8), 0);          // other stream: cached block must not migrate
        EXPECT_TRUE(c != b);
        EXPECT_EQ(pool.free_async(c, 8), 0);
        EXPECT_EQ(pool.free_async(c, 8), -1);             // double free is reported, not absorbed
        int dummy;
        EXPECT_EQ(pool.free_async(&dummy, 8), -1);        // foreign pointer
        const auto st = pool.stats();
        EXPECT_EQ(st.bytes_in_use, 0u);
        EXPECT_EQ(st.device_allocs, 2u);
        EXPECT_EQ(st.cache_hits, 1u);
        EXPECT_EQ(st.bytes_cached, 2048u);
        // a much larger cached block does not serve a small request (25 % slack rule)
        void* big = nullptr;
        EXPECT_EQ(pool.allocate(&big, 64 << 10, 7), 0);
        EXPECT_EQ(pool.free_async(big, 7), 0);
        void* small = nullptr;
        EXPECT_EQ(pool.allocate(&small, 1 << 10, 7), 0);
        EXPECT_TRUE(small != big);
        EXPECT_EQ(pool.free_now(small), 0);
        pool.trim();
        EXPECT_EQ(pool.stats().bytes_cached, 0u);
    }
    EXPECT_EQ(live.load(), 0u);                           // everything went back to the backend
}

TEST(Pool, OutOfMemoryTrimsCacheAndRetries) {
    std::atomic<size_t> live{0}, allocs{0};
    nzhip::PoolAllocator<FakeBackend> pool(FakeBackend{&live, &allocs, size_t(8) << 20});
    void *a = nullptr, *b = nullptr;
    EXPECT_EQ(pool.allocate(&a, size_t(6) << 20), 0);
    EXPECT_EQ(pool.free_async(a), 0);                     // 6 MiB cached
    EXPECT_EQ(pool.allocate(&b, size_t(4) << 20), 0);     // does not fit beside the cache: cache is dropped
    EXPECT_EQ(live.load(), size_t(4) << 20);
    void* c = nullptr;
    EXPECT_TRUE(pool.allocate(&c, size_t(6) << 20) != 0); // genuinely out of memory
    EXPECT_TRUE(c == nullptr);
    EXPECT_EQ(pool.free_async(b), 0);
}

TEST(Pool, ConcurrentAllocateFreeKeepsBooksConsistent) {
    std::atomic<size_t> live{0}, allocs{0};
    nzhip::PoolAllocator<FakeBackend> pool(FakeBackend{&live, &allocs, size_t(1) << 40});
    std::vector<std::thread> threads;
    std::atomic<int> errors{0};
    for (int t = 0; t < 8; ++t) {
        threads.emplace_back([&, t] {
            std::vector<void*> mine;
            unsigned s = 1234u + t;
            for (int i = 0; i < 4000; ++i) {
                s = s * 1664525u + 1013904223u;
                if (mine.size() < 16 && (s >> 16) % 3 != 0) {
                    void* p = nullptr;
                    if (pool.allocate(&p, 256 + (s >> 8) % 100000, t % 2) != 0 || !p) errors++;
                    mine.push_back(p);
                } else if (!mine.empty()) {
                    if (pool.free_async(mine.back(), t % 2) != 0) errors++;
                    mine.pop_back();
                }
            }
            for (void* p : mine)
                if (pool.free_async(p, t % 2) != 0) errors++;
        });
    }
    for (auto& th : threads) th.join();
    EXPECT_EQ(errors.load(), 0);
    EXPECT_EQ(pool.stats().bytes_in_use, 0u);
    EXPECT_TRUE(pool.stats().cache_hits > 0);
    pool.trim();
    EXPECT_EQ(live.load(), 0u);
}

int main(int argc, char** argv) { return mini::run_all(argc > 1 ? argv[1] : nullptr); }
