// Device tensor: RAII owner of contiguous NCHW fp32 storage (and an optional gradient buffer)
// in HBM (reference: include/NeuZephyr/Tensor.cuh:131-1630, src/Tensor.cu). Storage comes from
// the caching pool behind nzhip_malloc / nzhip_free_async; every operation is enqueued on the
// library's ordered compute stream and returns immediately -- hostData(), operator==,
// operator<< and the sync*() members are the only blocking calls.
//
// Differences from the reference, all invisible through the API:
//   * buffers are allocated lazily, on first use, so a node whose output is fused away
//     (e.g. the im2col matrix of Conv2d) never costs memory;
//   * sizes passed to the allocator are bytes (the reference multiplies by sizeof(T) twice).
#ifndef NZ_TENSOR_CUH
#define NZ_TENSOR_CUH
#include <initializer_list>
#include <iosfwd>
#include <iterator>
#include <stdexcept>
#include <vector>

#include "Dimension.cuh"
#include "dl_export.cuh"

namespace nz::data {
    class DL_API Tensor {
    public:
        using size_type = unsigned long long;
        using value_type = float;
        using shape_type = Dimension;

        friend DL_API std::ostream& operator<<(std::ostream& os, const Tensor& tensor);

        Tensor();
        explicit Tensor(const shape_type& shape, bool requires_grad = false);
        explicit Tensor(const shape_type& shape, value_type* data, bool requires_grad = false, bool host = true);
        explicit Tensor(const shape_type& shape, const std::initializer_list<value_type>& data,
                        bool requires_grad = false);
        Tensor(const Tensor& other);
        Tensor(Tensor&& other) noexcept;
        Tensor& operator=(const Tensor& other);
        Tensor& operator=(Tensor&& other) noexcept;
        ~Tensor();

        [[nodiscard]] bool requiresGrad() const noexcept { return _requires_grad; }
        [[nodiscard]] shape_type shape() const noexcept { return _shape; }
        [[nodiscard]] size_type size() const noexcept { return _size; }
        void setRequiresGrad(bool requires_grad);

        [[nodiscard]] value_type* data() const;                    // device pointer (allocates on first use)
        // The same pointer for a caller that only reads. data() hands out a writable pointer and therefore counts
        // as a possible write: version() goes up with every data() call (and so with every member that writes),
        // never with constData(). Whoever keeps something derived from the contents (the fused layers keep the
        // fp16 image of their weights between forward passes) compares version() to know whether it is still good.
        [[nodiscard]] const value_type* constData() const;
        [[nodiscard]] unsigned long long version() const noexcept { return _version; }
        [[nodiscard]] value_type* grad() const;                    // throws std::runtime_error without gradients
        // the same buffer for a caller that is about to write EVERY element of it (contents undefined on return)
        [[nodiscard]] value_type* gradOverwrite() const;
        // True when the next grad() call would hand out zeros (a clear is pending or the buffer does not exist yet): a writer
        // that can overwrite instead of add may then take gradOverwrite() and skip both the clear and its own read of the zeros.
        [[nodiscard]] bool gradIsZero() const noexcept { return _requires_grad && _size != 0 && (_gradZeroPending || !_grad); }
        [[nodiscard]] std::vector<value_type> hostData() const;    // blocks
        [[nodiscard]] std::vector<value_type> hostGrad() const;    // blocks

        void dataInject(value_type* data, bool grad = false) const;
        template <typename Iterator>
        void dataInject(Iterator begin, Iterator end, const bool grad = false) const {
            if (static_cast<size_type>(std::distance(begin, end)) < _size) {
                throw std::runtime_error("Tensor::dataInject: not enough elements");
            }
            std::vector<value_type> staging(_size);
            auto it = begin;
            for (size_type i = 0; i < _size; ++i, ++it) staging[i] = static_cast<value_type>(*it);
            dataInject(staging.data(), grad);
        }
        void dataInject(const std::initializer_list<value_type>& data, bool grad = false) const;

        void zeroGrad() const;
        // Runs the clears that zeroGrad() left pending on these tensors in one launch (a backward pass that will add
        // into a dozen small parameter gradients would otherwise start a dozen clears, one per first touch).
        static void clearPendingGrads(const std::vector<const Tensor*>& tensors);
        void clear() const;
        void fill(value_type value, bool isGrad = false) const;
        // Deterministic uniform (0,1] fill. The reference draws from cuRAND's XORWOW stream
        // (src/Tensor.cu:298-300), which is not reproduced; the distribution is the same.
        void randomize(unsigned long long seed = 0) const;
        void reshape(const shape_type& shape);

        // fp32-exact batched matrix product with (n, c) broadcast (reference: src/Tensor.cu:343-350)
        Tensor operator*(const Tensor& other) const;
        bool operator==(const Tensor& other) const;               // rel 1e-5 / abs 1e-6, also compares gradients
        bool operator!=(const Tensor& other) const { return !(*this == other); }

        void syncData() const;
        void syncGrad() const;
        void sync() const;

    private:
        void release() noexcept;
        size_type _size;
        shape_type _shape;
        mutable value_type* _data;
        mutable value_type* _grad;
        // zeroGrad() only notes that the gradient is zero; the clear runs when somebody reads or adds to it
        // (grad()) and is skipped when the next user overwrites every element (gradOverwrite())
        mutable bool _gradZeroPending = false;
        mutable unsigned long long _version = 0;
        bool _requires_grad;
    };
}
#endif
