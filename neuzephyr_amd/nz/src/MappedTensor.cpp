#include "NeuZephyr/MappedTensor.cuh"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <iostream>
#include <iterator>
#include <vector>

#include <exception>

#include "NeuZephyr/NeuZephyrCudaErrorHandling.cuh"
#include "NeuZephyr/TensorOperations.cuh"
#include "nzhip.h"

namespace nz::data {
    namespace {
        float* hostAlloc(const unsigned long long elements) {
            void* p = nullptr;
            NZ_CHECK(nzhip_host_malloc(&p, static_cast<size_t>(elements) * sizeof(float)));
            return static_cast<float*>(p);
        }

        void wait() { NZ_CHECK(nzhip_sync_ptr(nullptr)); }

        bool close(const float a, const float b) {
            const float diff = std::abs(a - b);
            return !(diff > std::max(1e-5f * std::max(std::abs(a), std::abs(b)), 1e-6f));
        }

        std::ostream& printPlanes(std::ostream& os, const float* base, const Dimension& shape) {
            const std::ostream_iterator<float> oit(os, " ");
            for (size_t n = 0; n < shape.N(); ++n) {
                os << "n=" << n << " [\n";
                for (size_t c = 0; c < shape.C(); ++c) {
                    os << "  c=" << c << " [\n";
                    for (size_t h = 0; h < shape.H(); ++h) {
                        const float* row = base + n * shape.getStride(0) + c * shape.getStride(1) + h * shape.getStride(2);
                        os << "    [";
                        std::copy(row, row + shape.W(), oit);
                        os << "]\n";
                    }
                    os << "  ]\n";
                }
                os << "]\n\n";
            }
            return os;
        }

        // out(n, c, i) = f(a(n or 0, c or 0, i), b(n or 0, c or 0, i)) over h*w elements per plane
        template <typename F>
        void planewise(const MappedTensor& out, const MappedTensor& a, const MappedTensor& b, F f) {
            const Dimension so = out.shape(), sa = a.shape(), sb = b.shape();
            if (!sa.isBroadcastCompatible(sb) || sa.H() != sb.H() || sa.W() != sb.W()) {
                throw std::invalid_argument("Shapes are not broadcast compatible.");
            }
            wait();
            const size_t plane = so.H() * so.W();
            for (size_t n = 0; n < so.N(); ++n) {
                for (size_t c = 0; c < so.C(); ++c) {
                    float* o = out.data() + n * so.getStride(0) + c * so.getStride(1);
                    const float* x = a.data() + (sa.N() == 1 ? 0 : n) * sa.getStride(0) + (sa.C() == 1 ? 0 : c) * sa.getStride(1);
                    const float* y = b.data() + (sb.N() == 1 ? 0 : n) * sb.getStride(0) + (sb.C() == 1 ? 0 : c) * sb.getStride(1);
                    for (size_t i = 0; i < plane; ++i) o[i] = f(x[i], y[i]);
                }
            }
        }
    }

    std::ostream& operator<<(std::ostream& os, const MappedTensor& tensor) {
        tensor.print(os);
        if (tensor._requires_grad) {
            os << "Gradient: " << std::endl;
            tensor.printGrad(os);
        }
        return os;
    }

    std::istream& operator>>(std::istream& is, MappedTensor& tensor) {
        wait();
        for (MappedTensor::size_type i = 0; i < tensor._size; ++i) {
            if (!(is >> tensor._data[i])) break;
        }
        return is;
    }

    MappedTensor::MappedTensor() : _size(0), _shape(0, 0, 0, 0), _data(nullptr), _grad(nullptr), _requires_grad(false) {}

    MappedTensor::MappedTensor(const shape_type& shape, const bool requires_grad)
        : _size(shape.size()), _shape(shape), _data(nullptr), _grad(nullptr), _requires_grad(requires_grad) {
        _data = hostAlloc(_size);
        if (_requires_grad) _grad = hostAlloc(_size);
    }

    MappedTensor::MappedTensor(const MappedTensor& other) : MappedTensor(other._shape, other._requires_grad) {
        wait();
        if (_size) std::memcpy(_data, other._data, _size * sizeof(value_type));
        if (_requires_grad && _size) std::memcpy(_grad, other._grad, _size * sizeof(value_type));
    }

    MappedTensor::MappedTensor(MappedTensor&& other) noexcept
        : _size(other._size), _shape(other._shape), _data(other._data), _grad(other._grad),
          _requires_grad(other._requires_grad) {
        other._data = nullptr;
        other._grad = nullptr;
        other._size = 0;
        other._requires_grad = false;
        other._shape = Dimension(0, 0, 0, 0);
    }

    MappedTensor& MappedTensor::operator=(const MappedTensor& other) {
        if (this == &other) return *this;
        MappedTensor copy(other);
        *this = std::move(copy);
        return *this;
    }

    MappedTensor& MappedTensor::operator=(MappedTensor&& other) noexcept(false) {
        if (this == &other) return *this;
        release();
        _size = other._size;
        _shape = other._shape;
        _data = other._data;
        _grad = other._grad;
        _requires_grad = other._requires_grad;
        other._data = nullptr;
        other._grad = nullptr;
        other._size = 0;
        other._requires_grad = false;
        other._shape = Dimension(0, 0, 0, 0);
        return *this;
    }

    MappedTensor::~MappedTensor() noexcept(false) {
        try {
            release();
        } catch (...) {
            // a second exception during stack unwinding would end the process: report only when nothing else is in flight
            if (std::uncaught_exceptions() == 0) throw;
        }
    }

    void MappedTensor::release() {
        // nzhip_host_free waits for the compute stream: a kernel may still be using the memory
        if (_grad) NZ_CHECK(nzhip_host_free(_grad));
        if (_data) NZ_CHECK(nzhip_host_free(_data));
        _grad = nullptr;
        _data = nullptr;
    }

    MappedTensor::iterator MappedTensor::begin() const {
        sync();
        return _data;
    }

    MappedTensor::iterator MappedTensor::end() const {
        sync();
        return _data + _size;
    }

    MappedTensor::value_type* MappedTensor::grad() const {
        if (!_requires_grad) {
            throw std::invalid_argument("Gradient access is not allowed for tensors that do not require gradients.");
        }
        return _grad;
    }

    void MappedTensor::setRequiresGrad(const bool requires_grad) {
        if (_requires_grad && !requires_grad) {
            NZ_CHECK(nzhip_host_free(_grad));
            _grad = nullptr;
        } else if (!_requires_grad && requires_grad) {
            _grad = hostAlloc(_size);
        }
        _requires_grad = requires_grad;
    }

    void MappedTensor::setShape(const shape_type& shape) { _shape.reshape(shape); }

    MappedTensor::value_type* MappedTensor::target(const bool isGrad, const char* complaint) const {
        if (isGrad && !_requires_grad) throw std::invalid_argument(complaint);
        wait();
        return isGrad ? _grad : _data;
    }

    void MappedTensor::dataInject(float* data, const size_type size, const bool isGrad) const {
        value_type* dst = target(isGrad, "Gradient injection is not allowed for tensors that do not require gradients.");
        const size_type count = size < _size ? size : _size;
        if (count) std::memcpy(dst, data, count * sizeof(value_type));
    }

    void MappedTensor::dataInject(const std::initializer_list<value_type>& data, const bool isGrad) const {
        value_type* dst = target(isGrad, "Gradient injection is not allowed for tensors that do not require gradients.");
        const size_type count = data.size() < _size ? data.size() : _size;
        std::copy_n(data.begin(), count, dst);
    }

    auto MappedTensor::operator[](const size_type index) const -> value_type& {
        syncData();
        if (index >= _size) throw std::out_of_range("Index out of range.");
        return _data[index];
    }

    std::ostream& MappedTensor::print(std::ostream& os) const {
        syncData();
        return printPlanes(os, _data, _shape);
    }

    std::ostream& MappedTensor::printGrad(std::ostream& os) const {
        if (!_requires_grad) {
            throw std::invalid_argument("Gradient printing is not allowed for tensors that do not require gradients.");
        }
        syncGrad();
        return printPlanes(os, _grad, _shape);
    }

    void MappedTensor::clear() const {
        wait();
        if (_size) std::memset(_data, 0, _size * sizeof(value_type));
    }

    void MappedTensor::clearGrad() const {
        if (!_requires_grad) {
            throw std::runtime_error("Gradient clearing is not allowed for tensors that do not require gradients.");
        }
        wait();
        if (_size) std::memset(_grad, 0, _size * sizeof(value_type));
    }

    void MappedTensor::reshape(const shape_type& shape) {
        const size_type newSize = shape.size();
        if (newSize != _size) std::cerr << "[WARN] Reshaping to a different size will cause data loss" << std::endl;
        wait();
        auto move = [&](value_type*& buffer) {
            value_type* fresh = hostAlloc(newSize);
            const size_type keep = _size < newSize ? _size : newSize;
            if (keep) std::memcpy(fresh, buffer, keep * sizeof(value_type));
            if (newSize > keep) std::memset(fresh + keep, 0, (newSize - keep) * sizeof(value_type));
            NZ_CHECK(nzhip_host_free(buffer));
            buffer = fresh;
        };
        move(_data);
        if (_requires_grad) move(_grad);
        _shape = shape;
        _size = newSize;
    }

    void MappedTensor::randomize(size_type seed, const bool isGrad) const {
        value_type* dst = target(isGrad, "Gradient randomization is not allowed for tensors that do not require gradients.");
        if (!seed) seed = static_cast<size_type>(std::chrono::system_clock::now().time_since_epoch().count());
        // splitmix64 stream -> uniform (0, 1], the range cuRAND's uniform generator produces
        unsigned long long s = seed * 0x9e3779b97f4a7c15ull + 0x2545f4914f6cdd1dull;
        for (size_type i = 0; i < _size; ++i) {
            unsigned long long z = (s += 0x9e3779b97f4a7c15ull);
            z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
            z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
            z ^= z >> 31;
            dst[i] = static_cast<value_type>(((z >> 40) + 1) * (1.0 / 16777216.0));
        }
    }

    void MappedTensor::fill(const value_type value, const bool isGrad) const {
        value_type* dst = target(isGrad, "Gradient filling is not allowed for tensors that do not require gradients.");
        std::fill_n(dst, _size, value);
    }

    void MappedTensor::fillMatrix(const value_type value, const size_type batch, const size_type channels, const bool isGrad) {
        if (batch >= _shape[0] || channels >= _shape[1]) throw std::invalid_argument("Invalid batch or channels");
        value_type* dst = target(isGrad, "Gradient filling is not allowed for tensors that do not require gradients.");
        std::fill_n(dst + batch * _shape.getStride(0) + channels * _shape.getStride(1), _shape[2] * _shape[3], value);
    }

    void MappedTensor::transpose() {
        wait();
        const size_t H = _shape.H(), W = _shape.W(), planes = _shape.N() * _shape.C();
        auto flip = [&](value_type*& buffer) {
            value_type* fresh = hostAlloc(_size);
            for (size_t p = 0; p < planes; ++p) {
                const value_type* src = buffer + p * H * W;
                value_type* dst = fresh + p * H * W;
                for (size_t h = 0; h < H; ++h)
                    for (size_t w = 0; w < W; ++w) dst[w * H + h] = src[h * W + w];
            }
            NZ_CHECK(nzhip_host_free(buffer));
            buffer = fresh;
        };
        flip(_data);
        if (_requires_grad) flip(_grad);
        _shape = Dimension(_shape.N(), _shape.C(), W, H);
    }

    MappedTensor MappedTensor::operator+(const MappedTensor& other) const {
        MappedTensor result(_shape.Broadcast(other._shape), _requires_grad || other._requires_grad);
        tensorMatrixAdd(result, *this, other);
        return result;
    }

    MappedTensor MappedTensor::operator-(const MappedTensor& other) const {
        MappedTensor result(_shape.Broadcast(other._shape), _requires_grad || other._requires_grad);
        planewise(result, *this, other, [](const float a, const float b) { return a - b; });
        return result;
    }

    MappedTensor MappedTensor::operator*(const MappedTensor& other) const {
        MappedTensor result({std::max(_shape.N(), other._shape.N()), std::max(_shape.C(), other._shape.C()), _shape.H(),
                             other._shape.W()},
                            _requires_grad || other._requires_grad);
        tensorGeneralMatrixMul(result, *this, other);
        return result;
    }

    MappedTensor MappedTensor::operator/(const MappedTensor& other) const {
        MappedTensor result(_shape.Broadcast(other._shape), _requires_grad || other._requires_grad);
        planewise(result, *this, other, [](const float a, const float b) { return a / b; });
        return result;
    }

    MappedTensor MappedTensor::operator-() const {
        MappedTensor result(_shape, _requires_grad);
        wait();
        for (size_type i = 0; i < _size; ++i) result._data[i] = -_data[i];
        return result;
    }

    bool MappedTensor::operator==(const MappedTensor& other) const {
        if (_requires_grad != other._requires_grad || _shape != other._shape) return false;
        wait();
        for (size_type i = 0; i < _size; ++i)
            if (!close(_data[i], other._data[i])) return false;
        if (_requires_grad)
            for (size_type i = 0; i < _size; ++i)
                if (!close(_grad[i], other._grad[i])) return false;
        return true;
    }

    void MappedTensor::recip() {
        wait();
        for (size_type i = 0; i < _size; ++i) _data[i] = 1.0f / _data[i];
    }

    namespace {
        // sums of 256 consecutive elements, added in ascending order: the grouping of the reference's
        // block-wise reduction (src/MappedTensor.cu:521-537); the order inside a block is not pinned by it
        template <typename F>
        float blockedSum(const float* x, const size_t n, F f) {
            float total = 0.0f;
            for (size_t b = 0; b < n; b += 256) {
                float part = 0.0f;
                for (size_t i = b; i < std::min(n, b + 256); ++i) part += f(x[i]);
                total += part;
            }
            return total;
        }
    }

    MappedTensor::value_type MappedTensor::sum() const {
        syncData();
        return blockedSum(_data, _size, [](const float v) { return v; });
    }

    MappedTensor::value_type MappedTensor::sum(const size_t batch, const size_t channel) const {
        if (batch >= _shape[0] || channel >= _shape[1]) throw std::invalid_argument("Invalid position");
        syncData();
        return blockedSum(_data + batch * _shape.getStride(0) + channel * _shape.getStride(1), _shape[2] * _shape[3],
                          [](const float v) { return v; });
    }

    MappedTensor::value_type MappedTensor::expSum() const {
        syncData();
        return blockedSum(_data, _size, [](const float v) { return std::exp(v); });
    }

    MappedTensor::value_type MappedTensor::expSum(const size_t batch, const size_t channel) const {
        if (batch >= _shape[0] || channel >= _shape[1]) throw std::invalid_argument("Invalid position");
        syncData();
        return blockedSum(_data + batch * _shape.getStride(0) + channel * _shape.getStride(1), _shape[2] * _shape[3],
                          [](const float v) { return std::exp(v); });
    }

    void MappedTensor::syncGrad() const {
        if (_requires_grad) NZ_CHECK(nzhip_sync_ptr(_grad));
    }

    void MappedTensor::syncData() const { NZ_CHECK(nzhip_sync_ptr(_data)); }

    void MappedTensor::sync() const {
        syncData();
        syncGrad();
    }
}
