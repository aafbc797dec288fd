#include "NeuZephyr/Dimension.cuh"

#include <algorithm>
#include <iostream>
#include <stdexcept>

namespace nz::data {
    Dimension::Dimension(const size_t n, const size_t c, const size_t h, const size_t w) : dims_{n, c, h, w} {}

    Dimension::Dimension() : Dimension(1, 1, 1, 1) {}

    Dimension::Dimension(const std::vector<size_t>& dims) : dims_{0, 0, 0, 0} {
        if (dims.size() < 4) throw std::out_of_range("Dimension needs four extents");
        for (int i = 0; i < 4; ++i) dims_[i] = dims[i];
    }

    size_t Dimension::size() const { return dims_[0] * dims_[1] * dims_[2] * dims_[3]; }

    size_t Dimension::getStride(const size_t i) const {
        // contiguous NCHW: stride of axis i is the product of the extents after it
        if (i > 3) throw std::out_of_range("Index out of range");
        size_t s = 1;
        for (size_t k = 3; k > i; --k) s *= dims_[k];
        return s;
    }

    std::vector<size_t> Dimension::getDims() const { return {dims_[0], dims_[1], dims_[2], dims_[3]}; }

    size_t& Dimension::operator[](const size_t i) {
        if (i > 3) throw std::out_of_range("Index out of range");
        return dims_[i];
    }

    const size_t& Dimension::operator[](const size_t i) const {
        if (i > 3) throw std::out_of_range("Index out of range");
        return dims_[i];
    }

    bool Dimension::operator==(const Dimension& other) const {
        return std::equal(dims_, dims_ + 4, other.dims_);
    }

    bool Dimension::isBroadcastCompatible(const Dimension& other) const {
        for (int i = 0; i < 2; ++i) {
            if (dims_[i] != other.dims_[i] && dims_[i] != 1 && other.dims_[i] != 1) return false;
        }
        return true;
    }

    bool Dimension::reshape(const Dimension& newShape) {
        if (newShape.size() != size()) return false;
        *this = newShape;
        return true;
    }

    Dimension Dimension::Broadcast(const Dimension& other) const {
        if (!isBroadcastCompatible(other)) throw std::invalid_argument("Dimensions are not broadcast compatible");
        return {std::max(dims_[0], other.dims_[0]), std::max(dims_[1], other.dims_[1]),
                std::max(dims_[2], other.dims_[2]), std::max(dims_[3], other.dims_[3])};
    }

    std::ostream& operator<<(std::ostream& os, const Dimension& dim) {
        return os << dim.dims_[0] << " " << dim.dims_[1] << " " << dim.dims_[2] << " " << dim.dims_[3];
    }

    std::istream& operator>>(std::istream& is, Dimension& dim) {
        return is >> dim.dims_[0] >> dim.dims_[1] >> dim.dims_[2] >> dim.dims_[3];
    }
}
