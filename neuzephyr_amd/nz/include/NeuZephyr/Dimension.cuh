// 4-D NCHW shape with contiguous strides (reference: include/NeuZephyr/Dimension.cuh,
// src/Dimension.cu:5-141). The 4-argument constructor is deliberately non-explicit so that
// braced shapes `Tensor t({n, c, h, w})` compile, as the reference's tests rely on.
#ifndef NZ_DIMENSION_CUH
#define NZ_DIMENSION_CUH
#include <cstddef>
#include <iosfwd>
#include <vector>

#include "dl_export.cuh"

namespace nz::data {
    class DL_API Dimension {
    public:
        friend DL_API std::ostream& operator<<(std::ostream& os, const Dimension& dim);
        friend DL_API std::istream& operator>>(std::istream& is, Dimension& dim);

        Dimension(size_t n, size_t c, size_t h, size_t w);
        Dimension();
        explicit Dimension(const std::vector<size_t>& dims);
        Dimension(const Dimension& other) = default;
        Dimension& operator=(const Dimension& other) = default;

        [[nodiscard]] size_t size() const;
        [[nodiscard]] size_t getStride(size_t i) const;          // throws std::out_of_range
        [[nodiscard]] std::vector<size_t> getDims() const;
        [[nodiscard]] size_t N() const { return dims_[0]; }
        [[nodiscard]] size_t C() const { return dims_[1]; }
        [[nodiscard]] size_t H() const { return dims_[2]; }
        [[nodiscard]] size_t W() const { return dims_[3]; }
        size_t& operator[](size_t i);                             // throws std::out_of_range
        const size_t& operator[](size_t i) const;
        bool operator==(const Dimension& other) const;
        bool operator!=(const Dimension& other) const { return !(*this == other); }
        // Only n and c take part (src/Dimension.cu:101-108): h and w are checked by the callers.
        [[nodiscard]] bool isBroadcastCompatible(const Dimension& other) const;
        bool reshape(const Dimension& newShape);
        [[nodiscard]] Dimension Broadcast(const Dimension& other) const;   // element-wise max; throws std::invalid_argument
        void updateStride() {}                                     // strides are derived on demand

    private:
        size_t dims_[4];
    };
}
#endif
