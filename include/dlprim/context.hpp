// dlprim::Context / ExecutionContext over HIP for the convolution path.
//
// In dlprimitives a Context names an OpenCL platform:device and an
// ExecutionContext wraps an in-order cl::CommandQueue plus optional events
// (include/dlprim/context.hpp:128-299,309-431).  Here a Context names a HIP
// device and an ExecutionContext wraps a hipStream_t (kept as void* so that
// this header needs no HIP headers).  Work enqueued on one ExecutionContext runs
// in order; finish() is the only host synchronisation.
#pragma once
#include <memory>
#include <string>

#include "definitions.hpp"

namespace dlprim {

class ExecutionContext {
public:
    ExecutionContext() {}
    // adopt an existing hipStream_t (not owned)
    explicit ExecutionContext(void *hip_stream) : raw_(hip_stream), has_(true) {}
    bool is_cpu_context() const { return !has_; }
    void *stream() const { return owned_ ? owned_->s : raw_; }
    void finish() const
    {
        if (has_)
            details::check_status(dlp_stream_sync(stream()));
    }

private:
    friend class Context;
    struct Owned {
        void *s = nullptr;
        ~Owned()
        {
            if (s)
                dlp_stream_destroy(s);
        }
    };
    std::shared_ptr<Owned> owned_;
    void *raw_ = nullptr;
    bool has_ = false;
};

class Context {
public:
    enum ContextType { cpu = 0, hip = 1 };

    // "cpu" or a device index ("0", also accepted as "P:D" with the platform ignored)
    explicit Context(std::string const &dev_id)
    {
        if (dev_id == "cpu") {
            type_ = cpu;
            device_ = -1;
            return;
        }
        std::string d = dev_id;
        size_t colon = d.find(':');
        if (colon != std::string::npos)
            d = d.substr(colon + 1);
        type_ = hip;
        device_ = std::stoi(d);
        select();
    }
    explicit Context(ContextType t = cpu, int /*platform*/ = 0, int device = 0) : type_(t), device_(t == cpu ? -1 : device)
    {
        if (type_ == hip)
            select();
    }
    bool is_cpu_context() const { return type_ == cpu; }
    bool is_hip_context() const { return type_ == hip; }
    int device_id() const { return device_; }
    std::string name() const
    {
        if (is_cpu_context())
            return "CPU";
        char buf[256];
        details::check_status(dlp_device_name(device_, buf, sizeof(buf)));
        return buf;
    }
    // a new in-order queue on this device
    ExecutionContext make_execution_context() const
    {
        ExecutionContext e;
        if (is_cpu_context())
            return e;
        select();
        e.owned_ = std::make_shared<ExecutionContext::Owned>();
        details::check_status(dlp_stream_create(&e.owned_->s));
        e.has_ = true;
        return e;
    }
    void select() const
    {
        if (type_ == hip)
            details::check_status(dlp_set_device(device_));
    }

private:
    ContextType type_;
    int device_;
};

} // namespace dlprim
