// dlprim::Tensor over HIP device memory for the convolution path.
//
// As in dlprimitives (include/dlprim/tensor.hpp:106-294, src/tensor.cpp:104-133) a
// Tensor is a cheap shared handle: device buffer + ELEMENT offset + shape + dtype,
// with a lazily allocated host mirror that to_device()/to_host() copy from/to.
// sub_tensor() shares the memory.  Kernels receive device_ptr(), i.e. the buffer
// already advanced by the offset.
#pragma once
#include <cstring>
#include <memory>
#include <vector>

#include "context.hpp"
#include "shape.hpp"

namespace dlprim {

class Tensor {
public:
    Tensor() {}
    Tensor(Context &ctx, Shape const &s, DataType d = float_data) : shape_(s), dtype_(d), cpu_(ctx.is_cpu_context())
    {
        mem_ = std::make_shared<Memory>();
        mem_->bytes = s.total_size() * size_of_data_type(d);
        if (!cpu_) {
            ctx.select();
            details::check_status(dlp_malloc(&mem_->dev, mem_->bytes));
        }
    }
    // wrap device memory owned by somebody else
    Tensor(void *device_memory, size_t element_offset, Shape const &s, DataType d = float_data) : shape_(s), dtype_(d), offset_(element_offset)
    {
        mem_ = std::make_shared<Memory>();
        mem_->dev = device_memory;
        mem_->owned = false;
        mem_->bytes = (element_offset + s.total_size()) * size_of_data_type(d);
    }

    Shape const &shape() const { return shape_; }
    DataType dtype() const { return dtype_; }
    size_t memory_size() const { return shape_.total_size() * size_of_data_type(dtype_); }
    size_t device_offset() const { return offset_; }
    void reshape(Shape const &s)
    {
        DLPRIM_CHECK(s.total_size() <= capacity_elements());
        shape_ = s;
    }

    // device address of element 0 of this (sub)tensor
    void *device_ptr() const
    {
        DLPRIM_CHECK(mem_ && !cpu_);
        return static_cast<char *>(mem_->dev) + offset_ * size_of_data_type(dtype_);
    }
    void *host_data()
    {
        DLPRIM_CHECK(mem_);
        if (mem_->host.size() < mem_->bytes)
            mem_->host.resize(mem_->bytes);
        return mem_->host.data() + offset_ * size_of_data_type(dtype_);
    }
    template <typename T>
    T *data()
    {
        return static_cast<T *>(host_data());
    }

    void to_device(ExecutionContext const &e, bool /*sync*/ = true)
    {
        if (cpu_)
            return;
        details::check_status(dlp_memcpy_h2d(device_ptr(), host_data(), memory_size(), e.stream()));
    }
    void to_host(ExecutionContext const &e, bool /*sync*/ = true)
    {
        if (cpu_)
            return;
        details::check_status(dlp_memcpy_d2h(host_data(), device_ptr(), memory_size(), e.stream()));
    }

    // offset is in elements of THIS tensor's dtype
    Tensor sub_tensor(size_t offset, Shape const &s, DataType d = float_data) const
    {
        const size_t byte_off = (offset_ + offset) * size_of_data_type(dtype_);
        DLPRIM_CHECK(byte_off % size_of_data_type(d) == 0);
        DLPRIM_CHECK(byte_off + s.total_size() * size_of_data_type(d) <= mem_->bytes);
        Tensor r(*this);
        r.shape_ = s;
        r.dtype_ = d;
        r.offset_ = byte_off / size_of_data_type(d);
        return r;
    }
    Tensor workspace_as_type(DataType d = float_data) const
    {
        return sub_tensor(0, Shape(memory_size() / size_of_data_type(d)), d);
    }
    Tensor alias() const { return *this; }

private:
    struct Memory {
        void *dev = nullptr;
        bool owned = true;
        size_t bytes = 0;
        std::vector<char> host;
        ~Memory()
        {
            if (dev && owned)
                dlp_free(dev);
        }
    };
    size_t capacity_elements() const { return mem_ ? mem_->bytes / size_of_data_type(dtype_) - offset_ : 0; }
    std::shared_ptr<Memory> mem_;
    Shape shape_;
    DataType dtype_ = float_data;
    size_t offset_ = 0;
    bool cpu_ = false;
};

} // namespace dlprim
