// dlprim::Shape: up to 8 dimensions, the subset of include/dlprim/shape.hpp:25-171
// that the convolution path and its callers use.
#pragma once
#include <array>
#include <initializer_list>
#include <ostream>

#include "definitions.hpp"

namespace dlprim {

constexpr int max_tensor_dim = 8;

class Shape {
public:
    Shape() : n_(0) { dims_.fill(0); }
    template <typename... Dims>
    Shape(size_t d0, Dims... rest) : n_(1 + sizeof...(rest))
    {
        static_assert(1 + sizeof...(rest) <= max_tensor_dim, "at most 8 dimensions");
        dims_.fill(0);
        size_t v[] = {d0, static_cast<size_t>(rest)...};
        for (int i = 0; i < n_; i++)
            dims_[i] = v[i];
    }
    // the dimensions [begin, end) (include/dlprim/shape.hpp:47-58 of the reference)
    template <typename It>
    static Shape from_range(It begin, It end)
    {
        Shape s;
        for (It p = begin; p != end; ++p) {
            DLPRIM_CHECK(s.n_ < max_tensor_dim);
            s.dims_[s.n_++] = size_t(*p);
        }
        return s;
    }
    int size() const { return n_; }
    size_t &operator[](int i) { return dims_[index(i)]; }
    size_t operator[](int i) const { return dims_[index(i)]; }
    size_t total_size() const
    {
        if (n_ == 0)
            return 0;
        size_t r = 1;
        for (int i = 0; i < n_; i++)
            r *= dims_[i];
        return r;
    }
    // product of all dimensions but the first
    size_t size_no_batch() const
    {
        if (n_ <= 0)
            return 0;
        size_t r = 1;
        for (int i = 1; i < n_; i++)
            r *= dims_[i];
        return r;
    }
    bool operator==(Shape const &o) const
    {
        if (n_ != o.n_)
            return false;
        for (int i = 0; i < n_; i++)
            if (dims_[i] != o.dims_[i])
                return false;
        return true;
    }
    bool operator!=(Shape const &o) const { return !(*this == o); }

private:
    int index(int i) const
    {
        if (i < 0)
            i += n_;
        DLPRIM_CHECK(i >= 0 && i < n_);
        return i;
    }
    std::array<size_t, max_tensor_dim> dims_;
    int n_;
};

inline std::ostream &operator<<(std::ostream &o, Shape const &s)
{
    o << '(';
    for (int i = 0; i < s.size(); i++)
        o << (i ? "," : "") << s[i];
    return o << ')';
}

} // namespace dlprim
