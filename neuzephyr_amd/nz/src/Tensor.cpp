#include "NeuZephyr/Tensor.cuh"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <iostream>

#include "NeuZephyr/NeuZephyrCudaErrorHandling.cuh"
#include "nzhip.h"

namespace nz::detail {
    void throwStatus(const int status, const char* file, const int line, const char* expr) {
        const char* text = nzhip_last_error();
        if (status == NZHIP_E_SHAPE) throw std::invalid_argument(text && *text ? text : "Shapes are not broadcast compatible.");
        if (status == NZHIP_E_INVALID || status == NZHIP_E_UNSUPPORTED) throw std::invalid_argument(text ? text : "invalid argument");
        if (status == NZHIP_E_NOMEM) throw std::bad_alloc();
        if (status == NZHIP_E_TIMEOUT) throw std::runtime_error(text && *text ? text : "a GEMM's bounded waits ran out");
        throw nz::CudaException(file, line, status, expr, text);
    }
}

namespace nz::data {
    namespace {
        float* deviceAlloc(const unsigned long long elements) {
            void* p = nullptr;
            NZ_CHECK(nzhip_malloc(&p, static_cast<size_t>(elements) * sizeof(float)));
            return static_cast<float*>(p);
        }
    }

    Tensor::Tensor() : _size(0), _shape(0, 0, 0, 0), _data(nullptr), _grad(nullptr), _requires_grad(false) {}

    Tensor::Tensor(const shape_type& shape, const bool requires_grad)
        : _size(shape.size()), _shape(shape), _data(nullptr), _grad(nullptr), _requires_grad(requires_grad) {}

    Tensor::Tensor(const shape_type& shape, value_type* data, const bool requires_grad, const bool host)
        : Tensor(shape, requires_grad) {
        if (_size == 0) return;
        if (host) {
            NZ_CHECK(nzhip_memcpy_h2d(this->data(), data, _size * sizeof(value_type)));
        } else {
            NZ_CHECK(nzhip_memcpy_d2d(this->data(), data, _size * sizeof(value_type)));
        }
    }

    Tensor::Tensor(const shape_type& shape, const std::initializer_list<value_type>& data, const bool requires_grad)
        : Tensor(shape, requires_grad) {
        if (static_cast<size_type>(data.size()) < _size) {
            throw std::invalid_argument("Initializer list size is less than the tensor size.");
        }
        dataInject(data);
    }

    Tensor::Tensor(const Tensor& other) : Tensor(other._shape, other._requires_grad) {
        if (other._data) NZ_CHECK(nzhip_memcpy_d2d(data(), other._data, _size * sizeof(value_type)));
        if (_requires_grad && other._grad) NZ_CHECK(nzhip_memcpy_d2d(gradOverwrite(), other.grad(), _size * sizeof(value_type)));
    }

    Tensor::Tensor(Tensor&& other) noexcept
        : _size(other._size), _shape(other._shape), _data(other._data), _grad(other._grad),
          _requires_grad(other._requires_grad) {
        _gradZeroPending = other._gradZeroPending;
        other._gradZeroPending = false;
        other._data = nullptr;
        other._grad = nullptr;
        other._size = 0;
        other._shape = Dimension(0, 0, 0, 0);
        other._requires_grad = false;
    }

    Tensor& Tensor::operator=(const Tensor& other) {
        if (this == &other) return *this;
        Tensor copy(other);
        *this = std::move(copy);
        return *this;
    }

    Tensor& Tensor::operator=(Tensor&& other) noexcept {
        if (this == &other) return *this;
        release();
        _size = other._size;
        _shape = other._shape;
        _data = other._data;
        _grad = other._grad;
        _requires_grad = other._requires_grad;
        _gradZeroPending = other._gradZeroPending;
        other._gradZeroPending = false;
        other._data = nullptr;
        other._grad = nullptr;
        other._size = 0;
        other._shape = Dimension(0, 0, 0, 0);
        other._requires_grad = false;
        ++_version;   // new contents, possibly at an address this tensor held before
        return *this;
    }

    void Tensor::release() noexcept {
        // stream-ordered: the blocks go back to the pool behind everything already enqueued
        if (_data) nzhip_free_async(_data);
        if (_grad) nzhip_free_async(_grad);
        _data = nullptr;
        _grad = nullptr;
    }

    Tensor::~Tensor() { release(); }

    void Tensor::setRequiresGrad(const bool requires_grad) {
        if (!requires_grad && _grad) {
            nzhip_free_async(_grad);
            _grad = nullptr;
            _gradZeroPending = false;
        }
        _requires_grad = requires_grad;
    }

    Tensor::value_type* Tensor::data() const {
        if (!_data && _size) _data = deviceAlloc(_size);
        ++_version;
        return _data;
    }

    const Tensor::value_type* Tensor::constData() const {
        if (!_data && _size) _data = deviceAlloc(_size);
        return _data;
    }

    Tensor::value_type* Tensor::grad() const {
        if (!_requires_grad) throw std::runtime_error("Tensor does not require gradients");
        if (!_grad && _size) {
            _grad = deviceAlloc(_size);
            _gradZeroPending = true;
        }
        if (_gradZeroPending) {
            _gradZeroPending = false;
            NZ_CHECK(nzhip_memset(_grad, 0, _size * sizeof(value_type)));
        }
        return _grad;
    }

    Tensor::value_type* Tensor::gradOverwrite() const {
        if (!_requires_grad) throw std::runtime_error("Tensor does not require gradients");
        if (!_grad && _size) _grad = deviceAlloc(_size);
        _gradZeroPending = false;
        return _grad;
    }

    std::vector<Tensor::value_type> Tensor::hostData() const {
        std::vector<value_type> result(_size);
        if (_size) NZ_CHECK(nzhip_memcpy_d2h(result.data(), data(), _size * sizeof(value_type)));
        return result;
    }

    std::vector<Tensor::value_type> Tensor::hostGrad() const {
        std::vector<value_type> result(_size);
        if (_size) NZ_CHECK(nzhip_memcpy_d2h(result.data(), grad(), _size * sizeof(value_type)));
        return result;
    }

    void Tensor::dataInject(value_type* src, const bool isGrad) const {
        if (_size == 0) return;
        NZ_CHECK(nzhip_memcpy_h2d(isGrad ? grad() : data(), src, _size * sizeof(value_type)));
    }

    void Tensor::dataInject(const std::initializer_list<value_type>& src, const bool isGrad) const {
        dataInject(src.begin(), src.end(), isGrad);
    }

    void Tensor::zeroGrad() const {
        // a gradient nobody has asked for yet is not allocated, and is cleared when it is (grad())
        if (_requires_grad && _size && _grad) _gradZeroPending = true;
    }

    void Tensor::clearPendingGrads(const std::vector<const Tensor*>& tensors) {
        std::vector<value_type*> ptrs;
        std::vector<size_t> counts;
        for (const Tensor* t : tensors) {
            if (!t || !t->_requires_grad || !t->_grad || !t->_gradZeroPending || t->_size == 0) continue;
            ptrs.push_back(t->_grad);
            counts.push_back(t->_size);
            t->_gradZeroPending = false;
        }
        if (!ptrs.empty())
            NZ_CHECK(nzhip_fill_many(static_cast<int>(ptrs.size()), ptrs.data(), counts.data(), 0.f, nzhip_default_stream()));
    }

    void Tensor::clear() const {
        if (_size) NZ_CHECK(nzhip_memset(data(), 0, _size * sizeof(value_type)));
    }

    void Tensor::fill(const value_type value, const bool isGrad) const {
        if (_size == 0) return;
        // on the device, like the reference's Fill kernel: OutputNode::backward fills the whole output gradient on every pass
        NZ_CHECK(nzhip_fill(isGrad ? gradOverwrite() : data(), value, _size, nzhip_default_stream()));
    }

    void Tensor::randomize(const unsigned long long seed) const {
        if (_size == 0) return;
        // splitmix64 stream -> uniform (0,1], the range cuRAND's uniform generator produces
        std::vector<value_type> host(_size);
        unsigned long long s = seed * 0x9e3779b97f4a7c15ull + 0x2545f4914f6cdd1dull;
        for (auto& v : host) {
            unsigned long long z = (s += 0x9e3779b97f4a7c15ull);
            z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
            z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
            z ^= z >> 31;
            v = static_cast<value_type>(((z >> 40) + 1) * (1.0 / 16777216.0));
        }
        NZ_CHECK(nzhip_memcpy_h2d(data(), host.data(), _size * sizeof(value_type)));
    }

    void Tensor::reshape(const shape_type& shape) {
        if (shape.size() != _size) throw std::invalid_argument("Tensor::reshape: element count must not change");
        _shape = shape;
    }

    Tensor Tensor::operator*(const Tensor& other) const {
        if (!_shape.isBroadcastCompatible(other._shape) || _shape.W() != other._shape.H()) {
            throw std::invalid_argument("Shapes are not broadcast compatible.");
        }
        Tensor result({std::max(_shape.N(), other._shape.N()), std::max(_shape.C(), other._shape.C()), _shape.H(),
                       other._shape.W()},
                      _requires_grad || other._requires_grad);
        size_t sa[4], sb[4], sc[4];
        for (size_t i = 0; i < 4; ++i) {
            sa[i] = _shape[i];
            sb[i] = other._shape[i];
            sc[i] = result._shape[i];
        }
        NZ_CHECK(nzhip_matmul_f32(data(), other.data(), result.data(), sa, sb, sc, nzhip_default_stream()));
        return result;
    }

    bool Tensor::operator==(const Tensor& other) const {
        if (_requires_grad != other._requires_grad || _shape != other._shape) return false;
        constexpr value_type abs_epsilon = 1e-6f, rel_epsilon = 1e-5f;   // src/Tensor.cu:513-514
        const auto close = [&](const std::vector<value_type>& a, const std::vector<value_type>& b) {
            for (size_type i = 0; i < _size; ++i) {
                const value_type diff = std::fabs(a[i] - b[i]);
                if (!(diff <= std::max(rel_epsilon * std::max(std::fabs(a[i]), std::fabs(b[i])), abs_epsilon))) return false;
            }
            return true;
        };
        if (!close(hostData(), other.hostData())) return false;
        return !_requires_grad || close(hostGrad(), other.hostGrad());
    }

    void Tensor::syncData() const { NZ_CHECK(nzhip_sync_ptr(_data)); }
    void Tensor::syncGrad() const { NZ_CHECK(nzhip_sync_ptr(_grad)); }
    void Tensor::sync() const { NZ_CHECK(nzhip_sync_ptr(_data)); }

    std::ostream& operator<<(std::ostream& os, const Tensor& tensor) {
        const auto host = tensor.hostData();
        const auto s = tensor.shape();
        size_t idx = 0;
        for (size_t n = 0; n < s.N(); ++n)
            for (size_t c = 0; c < s.C(); ++c) {
                os << "n=" << n << " c=" << c << "\n";
                for (size_t h = 0; h < s.H(); ++h) {
                    os << "[";
                    for (size_t w = 0; w < s.W(); ++w) os << host[idx++] << (w + 1 < s.W() ? ", " : "");
                    os << "]\n";
                }
            }
        return os;
    }
}
