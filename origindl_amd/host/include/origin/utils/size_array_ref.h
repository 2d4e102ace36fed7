// A non-owning view of a run of size_t values, as include/origin/utils/size_array_ref.h: lets one parameter accept a
// C array, a pointer and length, a vector or a braced list without copying. The viewed storage must outlive the view
// (a braced list lives until the end of the full expression of the call).
#pragma once
#include <cstddef>
#include <initializer_list>
#include <vector>

namespace origin
{
class SizeArrayRef
{
public:
    constexpr SizeArrayRef() noexcept : data_(nullptr), size_(0) {}
    template <size_t N>
    constexpr SizeArrayRef(const size_t (&arr)[N]) noexcept : data_(arr), size_(N)
    {}
    constexpr SizeArrayRef(const size_t *data, size_t size) noexcept : data_(data), size_(size) {}
    SizeArrayRef(const std::vector<size_t> &v) noexcept : data_(v.data()), size_(v.size()) {}
    SizeArrayRef(std::initializer_list<size_t> l) noexcept : data_(l.begin()), size_(l.size()) {}

    constexpr const size_t *data() const noexcept { return data_; }
    constexpr size_t size() const noexcept { return size_; }
    constexpr bool empty() const noexcept { return size_ == 0; }
    constexpr const size_t &operator[](size_t i) const noexcept { return data_[i]; }
    constexpr const size_t *begin() const noexcept { return data_; }
    constexpr const size_t *end() const noexcept { return data_ + size_; }
    std::vector<size_t> to_vector() const { return std::vector<size_t>(data_, data_ + size_); }

private:
    const size_t *data_;
    size_t size_;
};
}  // namespace origin
