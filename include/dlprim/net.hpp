// dlprim::Net, forward (predict) part, over the HIP operators of this library.
//
// Mirrors what dlprimitives' Net does for inference (include/dlprim/net.hpp:21-294, src/net.cpp):
// it loads a network in the JSON format of docs/network_json_format.md (inputs / outputs / operators
// with name, type, inputs, outputs, params, options), loads parameters from a DLPW file
// (src/net.cpp:63-101 writer, :204-305 reader: "DLPW", big-endian header length, JSON header
// {"tensors": {name: {dtype, shape, size, start}}}, raw data), infers shapes, plans tensor memory by
// liveness (src/net.cpp:585-654: intermediate tensors share chunks unless keep_intermediate_tensors),
// and runs the operators in order on one ExecutionContext with one shared workspace
// (src/net.cpp:836-851).  Operator types: Convolution2D, BatchNorm, Activation, Pooling2D,
// GlobalPooling, Elementwise, InnerProduct -- what docs/nets_for_benchmark/*.js use -- plus Softmax, Flatten, Concat, Slice, Reshape, Squeeze, Threshold, Abs, Hardtanh and
// TransposedConvolution2D, with the option names of the reference's *Config::from_json functions.
//
// In predict mode two graph rewrites are applied at setup (fuse(true), the default):
//  * a BatchNorm that is the only consumer of a Convolution2D / InnerProduct output is folded into its
//    weights and bias: W' = W * gamma / sqrt(var + eps) per output channel, b' = beta + (b - mean) * scale
//    (closed form of src/ops/batch_normalization.cpp:210-232);
//  * an Activation that is the next user of the output of an operator with a fused activation slot
//    (Convolution2D, InnerProduct, Elementwise, BatchNorm) whose activation is identity moves into that
//    slot (the reference's ONNX importer does the same merge, src/importers/onnx.cpp:531-580);
//  * a residual sum moves into the epilogue of the 1x1 convolution that produces its later branch;
//  * a depthwise 3x3 convolution and the 1x1 convolution that is its only reader run as one kernel where the library serves
//    the pair (core::DepthwisePointwiseForward: float tensors, images 20 to 56 wide), so the tensor between them is never written.
// Training, gradients and the other operator types are not part of this library.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "core/conv.hpp"
#include "core/ip.hpp"
#include "core/pool.hpp"
#include "json.hpp"

namespace dlprim {

enum class CalculationsMode { train, predict };

class Net {
public:
    explicit Net(Context &ctx) : ctx_(ctx) {}
    Net(Net const &) = delete;
    Net &operator=(Net const &) = delete;

    void load_from_json_file(std::string const &name)
    {
        std::ifstream f(name);
        if (!f)
            throw ValidationError("Failed to open file " + name);
        load_from_json(json::value::load(f));
    }
    void load_from_json(json::value const &v)
    {
        for (auto const &in : v["inputs"].array()) {
            std::string dt = in.get("dtype", "float");
            DataType input_type = float_data; // float: stored as the network's storage type
            if (dt == "int" || dt == "int32")
                input_type = int32_data; // class labels of a loss
            else if (dt != "float" && dt != "float32")
                throw NotImplementedError("input dtype " + dt);
            std::vector<int> dims = in.get<std::vector<int>>("shape");
            add_input_tensor(in.get("name", "data"), shape_of(dims), input_type);
        }
        for (auto const &op : v["operators"].array()) {
            Node n;
            n.name = op.get<std::string>("name");
            n.type = op.get<std::string>("type");
            n.inputs = op.get("inputs", std::vector<std::string>());
            n.outputs = op.get("outputs", std::vector<std::string>());
            if (!op.find("params").is_undefined())
                n.param_names = op.get<std::vector<std::string>>("params");
            n.options = op.find("options");
            nodes_.push_back(std::move(n));
        }
        for (auto const &out : v["outputs"].array())
            mark_output_tensor(out.type() == json::is_string ? out.str() : out.get<std::string>("name"));
    }
    // float_data: an input in the network's storage type; int32_data: labels of a loss operator
    void add_input_tensor(std::string const &name, Shape const &s, DataType dt = float_data)
    {
        if (dt != float_data && dt != int32_data)
            throw NotImplementedError("input tensors are float or int32");
        input_names_.push_back(name);
        specs_[name] = s;
        if (dt == int32_data)
            int_inputs_.insert(name);
    }
    void mark_output_tensor(std::string const &name) { output_names_.push_back(name); }

    void mode(CalculationsMode m)
    {
        if (m != CalculationsMode::predict)
            throw NotImplementedError("only CalculationsMode::predict is implemented");
    }
    CalculationsMode mode() const { return CalculationsMode::predict; }
    // keep every tensor in memory of its own (no sharing between intermediate tensors)
    void keep_intermediate_tensors(bool keep) { keep_intermediate_ = keep; }
    bool keep_intermediate_tensors() const { return keep_intermediate_; }
    // fold BatchNorm into the preceding convolution / inner product and merge activations (default on)
    void fuse(bool on) { fuse_ = on; }
    // Storage type of the tensors between operators (inputs and outputs included) and of the convolution /
    // inner-product weights on the device: float_data (as the reference) or bfloat16_data (16-bit elements,
    // arithmetic in fp32, biases and BatchNorm coefficients stay fp32).  Set before setup().  Parameters on
    // the host and in DLPW files are float either way; set_input / get_output convert.
    void storage_type(DataType dt)
    {
        DLPRIM_CHECK(!ready_);
        if (dt != float_data && dt != bfloat16_data)
            throw NotImplementedError("Net storage types: float_data and bfloat16_data");
        dtype_ = dt;
    }
    DataType storage_type() const { return dtype_; }
    // float values into input `id` (converted to the storage type, copied to the device) / output `id` as floats
    void set_input(unsigned id, float const *values, ExecutionContext const &e)
    {
        Tensor &t = input(id);
        const size_t n = t.shape().total_size();
        if (t.dtype() == int32_data)
            for (size_t i = 0; i < n; i++)
                t.data<int32_t>()[i] = int32_t(values[i]);
        else if (dtype_ == float_data)
            std::copy(values, values + n, t.data<float>());
        else
            for (size_t i = 0; i < n; i++)
                t.data<uint16_t>()[i] = to_bf16_bits(values[i]);
        t.to_device(e);
    }
    void get_output(unsigned id, float *values, ExecutionContext const &e)
    {
        Tensor &t = output(id);
        t.to_host(e);
        e.finish();
        const size_t n = t.shape().total_size();
        if (dtype_ == float_data)
            std::copy(t.data<float>(), t.data<float>() + n, values);
        else
            for (size_t i = 0; i < n; i++) {
                const uint32_t bits = uint32_t(t.data<uint16_t>()[i]) << 16;
                std::memcpy(values + i, &bits, 4);
            }
    }
    // round to nearest even, NaN stays NaN
    static uint16_t to_bf16_bits(float f)
    {
        uint32_t u;
        std::memcpy(&u, &f, 4);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u)
            return uint16_t((u >> 16) | 0x40);
        return uint16_t((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    }

    // transform the convolution weights once, when the parameters go to the device (default on);
    // off: every forward pass transforms them again, as the reference's operators do
    void prepack(bool on) { prepack_ = on; }
    // Tensors between bfloat16 convolutions are kept as [image][row][column][channel] wherever every operator that touches them can
    // take that layout and a reader is faster on it (plan_layouts; default on; network inputs, outputs and parameters keep the
    // reference's layout, and nothing changes with float_data or keep_intermediate_tensors)
    void channels_last(bool on) { channels_last_ = on; }
    // A max pooling that is the only reader of a bfloat16 convolution runs inside that convolution where the device code has such a
    // kernel (the 7x7 stride-2 stem of a ResNet with its 3x3 stride-2 pooling; default on, part of the graph rewrites).  The pair stays
    // one operator for the life of the network: reshape() to an image size that the kernel does not serve (rows off the multiples of
    // 8 pixels) throws NotImplementedError, so a network that will see such sizes switches this off before setup()
    void fuse_max_pooling(bool on) { fuse_max_pool_ = on; }

    // shapes, rewrites, operators, memory; parameters are allocated (zero on the host) and wait for load_parameters
    void setup()
    {
        infer_and_create_params();
        if (fuse_)
            rewrite_graph();
        plan_layouts();
        try {
            create_operators();
        } catch (NotImplementedError const &) {
            if (cl_groups_.empty())
                throw;
            cl_groups_.clear(); // an operator refused its layout: the reference's layout throughout
            create_operators();
        }
        allocate_tensors();
        ready_ = true;
    }

    // After the inputs were given other shapes (net.input(i).reshape(...)): every tensor takes the shape that follows.
    // As in the reference (include/dlprim/net.hpp: "reshape all tensors in network after reshaping the input data"),
    // tensors keep their memory, so shapes may shrink (a smaller batch, a smaller image) but not grow beyond what
    // setup() allocated.  Convolutions whose image size changed are planned again (and their weights packed again).
    void reshape()
    {
        DLPRIM_CHECK(ready_);
        release_graph();
        for (auto const &name : input_names_)
            specs_[name] = tensors_.at(name).shape();
        ExecutionContext e = ctx_.is_cpu_context() ? ExecutionContext() : ctx_.make_execution_context();
        for (auto &n : nodes_) {
            if (n.skipped)
                continue;
            Shape const in = n.inputs.empty() ? spec(n.outputs[0]) : spec(n.inputs[0]);
            Shape out;
            switch (n.kind) {
            case k_interp: out = interpolation_shape(n, in); break;
            case k_reduce: out = reduction_shape(n, in); break;
            case k_mse_loss:
                if (spec(n.inputs[1]) != in)
                    throw ValidationError("MSELoss inputs of different shapes after reshape (" + n.name + ")");
                out = n.loss_reduce == DLP_LOSS_REDUCE_NONE ? in : Shape(size_t(1));
                break;
            case k_nll_loss:
                check_labels(n);
                out = Shape(n.loss_reduce == DLP_LOSS_REDUCE_NONE ? in[0] : size_t(1));
                break;
            case k_softmax_loss:
                check_labels(n);
                out = Shape(size_t(1));
                break;
            case k_conv: {
                DLPRIM_CHECK(in.size() == 4 && int(in[1]) == n.conv.channels_in);
                if (n.dw_node >= 0) { // `in` is the input of the depthwise convolution that this node runs as well
                    out = core::Conv2DBase::get_output_shape(n.conv, core::Conv2DBase::get_output_shape(nodes_[size_t(n.dw_node)].conv, in));
                    if (n.dwpw_op && (n.planned_in[2] != in[2] || n.planned_in[3] != in[3]))
                        create_conv_operator(n, in); // NotImplementedError if the pair is not served at the new size: set up again, or fuse(false)
                    break;
                }
                out = core::Conv2DBase::get_output_shape(n.conv, in);
                if (n.pool_node >= 0) { // the node writes the pooled tensor
                    Node const &pl = nodes_[size_t(n.pool_node)];
                    out = Shape(out[0], out[1], size_t(core::calc_pooling_output_size(int(out[2]), pl.kernel[0], pl.pad[0], pl.stride[0], pl.ceil_mode)),
                                size_t(core::calc_pooling_output_size(int(out[3]), pl.kernel[1], pl.pad[1], pl.stride[1], pl.ceil_mode)));
                }
                Shape const &old = n.planned_in;
                if (n.conv_op && (old[2] != in[2] || old[3] != in[3])) {
                    create_conv_operator(n, in);
                    if (workspace_bytes_ > workspace_.memory_size())
                        workspace_ = Tensor(ctx_, Shape(workspace_bytes_), uint8_data);
                    if (n.is_packed) {
                        n.is_packed = false;
                        pack_conv_weights(n, e);
                    }
                }
                break;
            }
            case k_tconv: {
                DLPRIM_CHECK(in.size() == 4 && int(in[1]) == n.conv.channels_in);
                out = core::Conv2DBase::get_output_shape_transposed(n.conv, in, n.output_pad);
                Shape const &old = n.planned_in;
                if (n.tconv_op && (old[2] != in[2] || old[3] != in[3] || in[0] > old[0])) {
                    create_tconv_operator(n, in);
                    if (workspace_bytes_ > workspace_.memory_size())
                        workspace_ = Tensor(ctx_, Shape(workspace_bytes_), uint8_data);
                }
                break;
            }
            case k_ip:
                DLPRIM_CHECK(in.size_no_batch() == size_t(n.ip_inputs));
                out = Shape(in[0], size_t(n.ip_outputs));
                break;
            case k_pool:
                DLPRIM_CHECK(in.size() == 4);
                out = Shape(in[0], in[1], size_t(core::calc_pooling_output_size(int(in[2]), n.kernel[0], n.pad[0], n.stride[0], n.ceil_mode)),
                            size_t(core::calc_pooling_output_size(int(in[3]), n.kernel[1], n.pad[1], n.stride[1], n.ceil_mode)));
                break;
            case k_gpool: out = Shape(in[0], in[1], 1, 1); break;
            case k_flatten: out = Shape(in[0], in.size_no_batch()); break;
            case k_concat: out = concat_shape(n); break;
            case k_slice: out = slice_shape(n, in); break;
            case k_view: out = view_shape(n, in); break;
            case k_eltwise:
                if (n.broadcast)
                    out = broadcast_shape(in, spec(n.inputs[1]), n.name);
                else {
                    if (spec(n.inputs[1]) != in)
                        throw ValidationError("Elementwise inputs of different shapes after reshape (" + n.name + ")");
                    out = in;
                }
                break;
            default: out = in; break;
            }
            specs_[n.outputs[0]] = out;
            tensors_.at(n.outputs[0]).reshape(out);
            if (!ctx_.is_cpu_context()) {
                workspace_bytes_ = std::max(workspace_bytes_, node_workspace(n));
                if (workspace_bytes_ > workspace_.memory_size())
                    workspace_ = Tensor(ctx_, Shape(workspace_bytes_), uint8_data);
            }
        }
        if (!ctx_.is_cpu_context())
            e.finish();
    }

    void load_parameters(std::string const &file, bool allow_missing = false)
    {
        std::ifstream f(file, std::ios::binary);
        if (!f)
            throw ValidationError("Failed to open file " + file);
        load_parameters(f, allow_missing);
    }
    void load_parameters(std::istream &f, bool allow_missing = false)
    {
        DLPRIM_CHECK(ready_);
        char magic[4] = {0, 0, 0, 0};
        unsigned char len_bytes[4] = {0, 0, 0, 0};
        f.read(magic, 4);
        f.read(reinterpret_cast<char *>(len_bytes), 4);
        if (!f || std::string(magic, 4) != "DLPW")
            throw ValidationError("Not a DLPW parameters file");
        size_t len = (size_t(len_bytes[0]) << 24) | (size_t(len_bytes[1]) << 16) | (size_t(len_bytes[2]) << 8) | size_t(len_bytes[3]);
        std::string header(len, '\0');
        f.read(&header[0], (std::streamsize)len);
        if (!f)
            throw ValidationError("Truncated DLPW header");
        json::value h = json::value::parse(header);
        std::streamoff data_start = f.tellg();
        std::set<std::string> loaded;
        for (auto const &kv : h["tensors"].object()) {
            auto p = params_.find(kv.first);
            if (p == params_.end())
                continue; // the file may hold more than this network uses
            json::value const &ts = kv.second;
            if (ts.get("dtype", "float") != "float")
                throw NotImplementedError("parameter dtype of " + kv.first);
            std::vector<int> dims = ts.get<std::vector<int>>("shape");
            if (shape_of(dims).total_size() != p->second.shape().total_size())
                throw ValidationError("Parameter " + kv.first + " has a different size in the file");
            size_t bytes = ts.get<size_t>("size");
            DLPRIM_CHECK(bytes == p->second.memory_size());
            f.seekg(data_start + (std::streamoff)ts.get<size_t>("start"));
            f.read(static_cast<char *>(p->second.host_data()), (std::streamsize)bytes);
            if (!f)
                throw ValidationError("Truncated DLPW data for " + kv.first);
            loaded.insert(kv.first);
        }
        if (!allow_missing)
            for (auto const &p : params_)
                if (!loaded.count(p.first))
                    throw ValidationError("No parameter " + p.first + " in the file");
        copy_parameters_to_device();
    }
    void save_parameters(std::string const &file)
    {
        json::value header;
        json::value &tensors = header["tensors"];
        tensors.object();
        size_t start = 0;
        for (auto &p : params_) {
            json::value &ts = tensors[p.first];
            ts["dtype"] = json::value("float");
            for (int i = 0; i < p.second.shape().size(); i++)
                ts["shape"][size_t(i)] = json::value((size_t)p.second.shape()[i]);
            ts["size"] = json::value(p.second.memory_size());
            ts["start"] = json::value(start);
            start += p.second.memory_size();
        }
        std::string text = header.save();
        std::ofstream f(file, std::ios::binary);
        f << "DLPW";
        for (int i = 0; i < 4; i++)
            f << (char)(0xFF & (text.size() >> (24 - i * 8)));
        f << text;
        for (auto &p : params_)
            f.write(static_cast<char *>(p.second.host_data()), (std::streamsize)p.second.memory_size());
        if (!f)
            throw ValidationError("I/O error in saving to " + file);
    }

    // host copies of the parameters -> device (with the folded / derived forms the operators read)
    void copy_parameters_to_device()
    {
        DLPRIM_CHECK(ready_);
        ExecutionContext e = ctx_.make_execution_context();
        for (auto &p : params_)
            p.second.to_device(e);
        for (auto &n : nodes_)
            if (!n.skipped)
                prepare_derived_parameters(n, e);
        e.finish();
    }

    std::map<std::string, Tensor> &tensors() { return tensors_; }
    std::map<std::string, Tensor> &params() { return params_; }
    Tensor &tensor(std::string const &name)
    {
        auto p = tensors_.find(name);
        if (p == tensors_.end())
            throw ValidationError("Unknown tensor name:" + name);
        return p->second;
    }
    Tensor &param(std::string const &name)
    {
        auto p = params_.find(name);
        if (p == params_.end())
            throw ValidationError("Unknown parameter name:" + name);
        return p->second;
    }
    std::vector<std::string> const &input_names() { return input_names_; }
    std::vector<std::string> const &output_names() { return output_names_; }
    Tensor &input(unsigned id) { return tensor(input_names_.at(id)); }
    Tensor &output(unsigned id) { return tensor(output_names_.at(id)); }

    void forward(ExecutionContext const &e, bool sync = false)
    {
        DLPRIM_CHECK(ready_);
        if (ctx_.is_cpu_context())
            throw NotImplementedError("Net::forward needs a device context");
        if (graph_ && graph_stream_ == e.stream())
            details::check_status(dlp_graph_launch(graph_.get(), e.stream()));
        else
            for (auto &n : nodes_)
                if (!n.skipped)
                    run(n, e);
        if (sync)
            e.finish();
    }

    // Record one forward pass on e's stream as a HIP graph; later forward(e) calls replay it with a
    // single launch (inputs, outputs and parameters stay where they are: refill them in place).  Not in
    // the reference: for networks whose step is bound by launch overhead.  Parameters loaded after the
    // capture need copy_parameters_to_device() only: the graph reads the same buffers.
    void capture_forward(ExecutionContext const &e)
    {
        DLPRIM_CHECK(ready_);
        release_graph();
        forward(e, true); // first-use allocations happen here, not under capture
        details::check_status(dlp_graph_capture_begin(e.stream()));
        try {
            for (auto &n : nodes_)
                if (!n.skipped)
                    run(n, e);
        } catch (...) {
            dlp_graph *broken = nullptr;
            dlp_graph_capture_end(e.stream(), &broken);
            dlp_graph_destroy(broken);
            throw;
        }
        dlp_graph *g = nullptr;
        details::check_status(dlp_graph_capture_end(e.stream(), &g));
        graph_.reset(g, dlp_graph_destroy);
        graph_stream_ = e.stream();
    }
    void release_graph()
    {
        graph_.reset();
        graph_stream_ = nullptr;
    }
    bool has_graph() const { return bool(graph_); }

    // bytes of device memory behind the tensors (after planning) and operators that run (after the rewrites)
    size_t tensor_memory() const { return tensor_memory_; }
    size_t operators_run() const
    {
        size_t c = 0;
        for (auto const &n : nodes_)
            c += n.skipped ? 0 : 1;
        return c;
    }

private:
    enum Kind { k_conv, k_bn, k_act, k_pool, k_gpool, k_eltwise, k_ip, k_softmax, k_flatten, k_tconv, k_concat, k_slice, k_view, k_pointwise, k_interp, k_reduce, k_param, k_mse_loss, k_nll_loss, k_softmax_loss };
    struct Node {
        std::string name, type;
        std::vector<std::string> inputs, outputs, param_names;
        json::value options;
        Kind kind = k_conv;
        bool skipped = false;
        StandardActivations activation = StandardActivations::identity;
        // Convolution2D / InnerProduct
        Convolution2DConfigBase conv;
        bool bias = false;
        std::string algo;
        int ip_inputs = -1, ip_outputs = -1;
        Node *folded_bn = nullptr; // BatchNorm folded into this operator
        bool residual = false;     // a residual sum runs in this convolution's epilogue: inputs[1] is the other branch, the output lies over it
        float residual_factor = 1.0f;
        bool is_packed = false, use_w_dev = false;
        std::unique_ptr<core::Conv2DForward> conv_op;
        std::unique_ptr<core::TransposedConv2DForward> tconv_op; // TransposedConvolution2D
        int dw_node = -1; // a 1x1 convolution that also runs the depthwise convolution in front of it: index of that (skipped) node
        int pool_node = -1; // a convolution that also runs the max pooling behind it: index of that (skipped) node
        std::unique_ptr<core::DepthwisePointwiseForward> dwpw_op;
        int output_pad[2] = {0, 0};
        std::unique_ptr<core::IPForward> ip_op;
        Tensor w_dev, b_dev; // what the kernel reads when a BatchNorm is folded in
        Tensor packed;       // the weights in the order the kernel loads them
        Shape planned_in;    // input shape the convolution operator was created for
        // BatchNorm
        float eps = 1e-5f;
        bool affine = true;
        Tensor scale, shift;
        // Pooling2D / GlobalPooling
        int kernel[2] = {1, 1}, stride[2] = {1, 1}, pad[2] = {0, 0};
        bool max_mode = true, count_include_pad = false, ceil_mode = false;
        std::unique_ptr<core::Pooling2DForward> pool_op;
        // Elementwise
        int eltwise_op = DLP_ELTWISE_SUM;
        float coef[2] = {1.0f, 1.0f};
        bool broadcast = false; // the inputs differ in shape
        // Softmax
        bool log_softmax = false;
        // Concat / Slice: the axis, and the range of a Slice (end -1: to the end of the axis)
        int dim = 1, slice_begin = 0, slice_end = -1;
        // Reshape (view_dims as given: 0 keeps the input's dimension, -1 is deduced) / Squeeze (view_dims: the axes; empty: all of extent 1)
        bool squeeze = false;
        std::vector<int> view_dims;
        // Threshold / Abs / Hardtanh
        int pointwise_op = 0;
        float pointwise_p[2] = {0.0f, 0.0f};
        // Interpolation: the method, the size (<= 0: from the scale) and the scale (<= 0: from the size)
        int interp_method = DLP_INTERPOLATE_NEAREST, out_hw[2] = {-1, -1};
        double scale_yx[2] = {-1.0, -1.0};
        bool align_corners = false;
        // Reduction: the method, the axes as given (negative: from the end) or the first reduced axis, and whether reduced axes stay as 1
        int reduce_method = DLP_REDUCE_SUM, start_axis = 0;
        float output_scale = 1.0f;
        bool keep_dim = true, has_dims = false;
        std::vector<int> reduce_dims;
        // MSELoss / NLLLoss: none, sum, mean
        int loss_reduce = DLP_LOSS_REDUCE_MEAN;
    };

    // numpy's rule, as Elementwise::setup applies it (src/ops/elementwise.cpp:223): shapes aligned at their last dimension, extents equal or 1
    static Shape broadcast_shape(Shape const &a, Shape const &b, std::string const &who)
    {
        const int rank = std::max(a.size(), b.size());
        std::vector<size_t> d(size_t(rank), 1);
        for (int j = 0; j < rank; j++) {
            const size_t da = j < a.size() ? a[a.size() - 1 - j] : 1, db = j < b.size() ? b[b.size() - 1 - j] : 1;
            if (da != db && da != 1 && db != 1)
                throw ValidationError("Elementwise inputs do not broadcast (" + who + ")");
            d[size_t(rank - 1 - j)] = da == 1 ? db : da;
        }
        return Shape::from_range(d.begin(), d.end());
    }
    static std::vector<int> int_list(json::value const &o, char const *key)
    {
        std::vector<int> r;
        json::value const &v = o.find(key);
        if (v.is_undefined())
            return r;
        if (v.type() == json::is_array) {
            for (size_t i = 0; i < v.size(); i++)
                r.push_back((int)v[i].number());
        } else
            r.push_back((int)v.number());
        return r;
    }
    // Concat: all inputs agree but for the axis (src/ops/concat.cpp:44-64)
    Shape concat_shape(Node const &n) const
    {
        Shape r = spec(n.inputs[0]);
        DLPRIM_CHECK(n.dim >= 0 && n.dim < r.size());
        size_t total = 0;
        for (auto const &name : n.inputs) {
            Shape const &in = spec(name);
            DLPRIM_CHECK(in.size() == r.size());
            for (int j = 0; j < r.size(); j++)
                if (j != n.dim && in[j] != r[j])
                    throw ValidationError("Concat inputs differ outside the axis (" + n.name + ")");
            total += in[n.dim];
        }
        r[n.dim] = total;
        return r;
    }
    // Slice (src/ops/concat.cpp:231-249)
    static Shape slice_shape(Node const &n, Shape const &in)
    {
        DLPRIM_CHECK(n.dim >= 0 && n.dim < in.size());
        const int end = n.slice_end == -1 ? int(in[n.dim]) : n.slice_end;
        DLPRIM_CHECK(n.slice_begin >= 0 && n.slice_begin < end && end <= int(in[n.dim]));
        Shape r = in;
        r[n.dim] = size_t(end - n.slice_begin);
        return r;
    }
    // Reshape / Squeeze (Shape::reshape and Shape::squeeze, src/shape.cpp:29-103)
    static Shape view_shape(Node const &n, Shape const &in)
    {
        std::vector<size_t> d;
        if (n.squeeze) {
            std::vector<int> axes = n.view_dims;
            if (axes.empty())
                for (int i = 0; i < in.size(); i++)
                    if (in[i] == 1)
                        axes.push_back(i);
            for (auto &a : axes) {
                if (a < 0)
                    a += in.size();
                DLPRIM_CHECK(a >= 0 && a < in.size() && in[a] == 1);
            }
            for (int i = 0; i < in.size(); i++)
                if (std::find(axes.begin(), axes.end(), i) == axes.end())
                    d.push_back(in[i]);
            if (d.empty())
                d.push_back(1);
        } else {
            int deduced = -1;
            size_t given = 1;
            for (size_t i = 0; i < n.view_dims.size(); i++) {
                const int v = n.view_dims[i];
                if (v == -1) {
                    if (deduced != -1)
                        throw ValidationError("At most one index may be -1 in reshape");
                    deduced = int(i);
                    d.push_back(1);
                } else if (v == 0) {
                    if (int(i) >= in.size())
                        throw ValidationError("0 reshape for index too large");
                    d.push_back(in[int(i)]);
                } else {
                    DLPRIM_CHECK(v > 0);
                    d.push_back(size_t(v));
                }
                given *= d.back();
            }
            if (deduced != -1) {
                if (given == 0 || in.total_size() % given != 0)
                    throw ValidationError("Can't computed deduced shape, original shape isn't multiple of provided");
                d[size_t(deduced)] = in.total_size() / given;
            }
        }
        Shape r = Shape::from_range(d.begin(), d.end());
        if (r.total_size() != in.total_size())
            throw ValidationError("Reshape changes the number of elements (" + n.name + ")");
        return r;
    }

    // Interpolation::calc_size (src/ops/interpolation.cpp:53-69)
    static Shape interpolation_shape(Node const &n, Shape const &in)
    {
        DLPRIM_CHECK(in.size() == 4);
        Shape r = in;
        if (n.out_hw[0] > 0) {
            r[2] = size_t(n.out_hw[0]);
            r[3] = size_t(n.out_hw[1]);
        } else {
            r[2] = size_t(int(in[2] * n.scale_yx[0]));
            r[3] = size_t(int(in[3] * n.scale_yx[1]));
        }
        DLPRIM_CHECK(r[2] > 0 && r[3] > 0);
        return r;
    }
    // Reduction::setup / calc_shapes (src/ops/reduction.cpp:49-69,133-151): which axes go, and the shape that is left
    static std::vector<int> reduced_axes(Node const &n, Shape const &in)
    {
        std::vector<int> mask(size_t(in.size()), 0);
        if (!n.has_dims) {
            int first = n.start_axis < 0 ? n.start_axis + in.size() : n.start_axis;
            DLPRIM_CHECK(first >= 0 && first < in.size());
            for (int a = first; a < in.size(); a++)
                mask[size_t(a)] = 1;
        } else
            for (int a : n.reduce_dims) {
                if (a < 0)
                    a += in.size();
                DLPRIM_CHECK(a >= 0 && a < in.size());
                mask[size_t(a)] = 1;
            }
        return mask;
    }
    static Shape reduction_shape(Node const &n, Shape const &in)
    {
        std::vector<int> mask = reduced_axes(n, in);
        std::vector<size_t> d;
        for (int a = 0; a < in.size(); a++) {
            if (!mask[size_t(a)])
                d.push_back(in[a]);
            else if (n.keep_dim)
                d.push_back(1);
        }
        if (d.empty())
            d.push_back(1);
        return Shape::from_range(d.begin(), d.end());
    }
    static int loss_reduce_option(json::value const &o)
    {
        std::string r = o.type() == json::is_object ? o.get("reduce", "mean") : "mean";
        if (r == "none")
            return DLP_LOSS_REDUCE_NONE;
        if (r == "sum")
            return DLP_LOSS_REDUCE_SUM;
        if (r != "mean")
            throw ValidationError("Unknown loss reduction " + r);
        return DLP_LOSS_REDUCE_MEAN;
    }
    // device memory an operator needs beside its tensors, at the current shapes
    size_t node_workspace(Node const &n) const
    {
        size_t bytes = 0;
        if (n.kind == k_reduce) {
            Shape const &in = spec(n.inputs[0]);
            std::vector<int> mask = reduced_axes(n, in), dims(size_t(in.size()));
            for (int a = 0; a < in.size(); a++)
                dims[size_t(a)] = int(in[a]);
            details::check_status(dlp_reduce_fwd_workspace(int(dtype_), n.reduce_method, in.size(), dims.data(), mask.data(), &bytes));
        } else if (n.kind == k_mse_loss)
            details::check_status(dlp_mse_loss_fwd_workspace(int(dtype_), n.loss_reduce, spec(n.inputs[0]).total_size(), &bytes));
        else if (n.kind == k_softmax_loss)
            details::check_status(dlp_softmax_loss_fwd_workspace(int(spec(n.inputs[0])[0]), &bytes));
        return bytes;
    }
    void check_labels(Node const &n) const
    {
        Shape const &x = spec(n.inputs[0]), &lbl = spec(n.inputs[1]);
        DLPRIM_CHECK(x.size() == 2 && lbl.total_size() == x[0] && lbl[0] == x[0]);
        if (dtype_ != float_data && !int_inputs_.count(n.inputs[1]))
            throw NotImplementedError("labels stored as bfloat16 (" + n.name + "): give the label input the dtype int");
    }

    static Shape shape_of(std::vector<int> const &d)
    {
        switch (d.size()) {
        case 1: return Shape(size_t(d[0]));
        case 2: return Shape(size_t(d[0]), d[1]);
        case 3: return Shape(size_t(d[0]), d[1], d[2]);
        case 4: return Shape(size_t(d[0]), d[1], d[2], d[3]);
        default: throw NotImplementedError("tensors of rank " + std::to_string(d.size()));
        }
    }
    static void pair_option(json::value const &o, char const *key, int (&dst)[2], bool required = false)
    {
        json::value const &v = o.find(key);
        if (v.is_undefined()) {
            if (required)
                throw ValidationError(std::string("Missing option ") + key);
            return;
        }
        if (v.type() == json::is_array) {
            DLPRIM_CHECK(v.size() == 2);
            dst[0] = (int)v[size_t(0)].number();
            dst[1] = (int)v[size_t(1)].number();
        } else
            dst[0] = dst[1] = (int)v.number();
    }
    Shape const &spec(std::string const &name) const
    {
        auto p = specs_.find(name);
        if (p == specs_.end())
            throw ValidationError("Tensor " + name + " is used before it is produced");
        return p->second;
    }
    std::string param_name(Node &n, size_t i)
    {
        if (n.param_names.size() <= i)
            n.param_names.resize(i + 1);
        if (n.param_names[i].empty())
            n.param_names[i] = n.name + "." + std::to_string(i); // the reference's default naming
        return n.param_names[i];
    }
    void make_param(Node &n, size_t i, Shape const &s)
    {
        std::string name = param_name(n, i);
        auto p = params_.find(name);
        if (p != params_.end()) { // shared parameter
            DLPRIM_CHECK(p->second.shape() == s);
            return;
        }
        Tensor t(ctx_, s);
        std::fill(t.data<float>(), t.data<float>() + s.total_size(), 0.0f);
        params_[name] = t;
    }

    void infer_and_create_params()
    {
        for (auto &n : nodes_) {
            json::value const &o = n.options;
            std::string act = o.type() == json::is_object ? o.get("activation", "identity") : "identity";
            n.activation = activation_from_name(act);
            if (n.type == "Convolution2D") {
                n.kind = k_conv;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                DLPRIM_CHECK(in.size() == 4);
                n.conv.channels_in = o.get("channels_in", int(in[1]));
                n.conv.channels_out = o.get<int>("channels_out");
                pair_option(o, "kernel", n.conv.kernel, true);
                pair_option(o, "stride", n.conv.stride);
                pair_option(o, "dilate", n.conv.dilate);
                pair_option(o, "pad", n.conv.pad);
                n.conv.groups = o.get("groups", 1);
                n.bias = o.get("bias", true);
                n.algo = o.get("fwd_algo", "auto");
                if (n.algo == "auto")
                    n.algo = "";
                DLPRIM_CHECK(n.conv.channels_in == int(in[1]));
                specs_[n.outputs[0]] = core::Conv2DBase::get_output_shape(n.conv, in);
                make_param(n, 0, Shape(size_t(n.conv.channels_out), n.conv.channels_in / n.conv.groups, n.conv.kernel[0], n.conv.kernel[1]));
                if (n.bias)
                    make_param(n, 1, Shape(size_t(n.conv.channels_out)));
            } else if (n.type == "TransposedConvolution2D") { // src/ops/conv2d.cpp:559-660: weights [channels_in, channels_out / groups, kh, kw]
                n.kind = k_tconv;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                DLPRIM_CHECK(in.size() == 4);
                if (dtype_ != float_data)
                    throw NotImplementedError("TransposedConvolution2D in a 16-bit storage type (" + n.name + ")");
                n.conv.channels_in = o.get("channels_in", int(in[1]));
                n.conv.channels_out = o.get<int>("channels_out");
                pair_option(o, "kernel", n.conv.kernel, true);
                pair_option(o, "stride", n.conv.stride);
                pair_option(o, "dilate", n.conv.dilate);
                pair_option(o, "pad", n.conv.pad);
                pair_option(o, "output_pad", n.output_pad);
                n.conv.groups = o.get("groups", 1);
                n.bias = o.get("bias", true);
                n.algo = o.get("bwd_data_algo", "auto"); // the forward pass is the data-gradient operator (:693-699)
                if (n.algo == "auto")
                    n.algo = "";
                DLPRIM_CHECK(n.conv.channels_in == int(in[1]));
                DLPRIM_CHECK(n.conv.channels_in % n.conv.groups == 0 && n.conv.channels_out % n.conv.groups == 0);
                specs_[n.outputs[0]] = core::Conv2DBase::get_output_shape_transposed(n.conv, in, n.output_pad);
                make_param(n, 0, Shape(size_t(n.conv.channels_in), n.conv.channels_out / n.conv.groups, n.conv.kernel[0], n.conv.kernel[1]));
                if (n.bias)
                    make_param(n, 1, Shape(size_t(n.conv.channels_out)));
            } else if (n.type == "InnerProduct") {
                n.kind = k_ip;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                n.ip_inputs = o.get("inputs", int(in.size_no_batch()));
                n.ip_outputs = o.get<int>("outputs");
                n.bias = o.get("bias", true);
                DLPRIM_CHECK(size_t(n.ip_inputs) == in.size_no_batch());
                specs_[n.outputs[0]] = Shape(in[0], n.ip_outputs);
                make_param(n, 0, Shape(size_t(n.ip_outputs), n.ip_inputs));
                if (n.bias)
                    make_param(n, 1, Shape(size_t(n.ip_outputs)));
            } else if (n.type == "BatchNorm") {
                n.kind = k_bn;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                DLPRIM_CHECK(in.size() >= 2);
                int features = o.get("features", -1);
                DLPRIM_CHECK(features == -1 || features == int(in[1]));
                n.eps = o.get("eps", 1e-5f);
                n.affine = o.get("affine", true);
                specs_[n.outputs[0]] = in;
                for (size_t i = 0; i < (n.affine ? 4u : 2u); i++) // running mean, running variance, gamma, beta
                    make_param(n, i, Shape(in[1]));
            } else if (n.type == "Activation") {
                n.kind = k_act;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                specs_[n.outputs[0]] = spec(n.inputs[0]);
            } else if (n.type == "Pooling2D") {
                n.kind = k_pool;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                DLPRIM_CHECK(in.size() == 4);
                pair_option(o, "kernel", n.kernel, true);
                pair_option(o, "stride", n.stride);
                pair_option(o, "pad", n.pad);
                std::string mode = o.get("mode", "max");
                DLPRIM_CHECK(mode == "max" || mode == "avg");
                n.max_mode = mode == "max";
                n.ceil_mode = o.get("ceil_mode", false);
                n.count_include_pad = o.get("count_include_pad", false);
                specs_[n.outputs[0]] = Shape(in[0], in[1], core::calc_pooling_output_size(int(in[2]), n.kernel[0], n.pad[0], n.stride[0], n.ceil_mode),
                                             core::calc_pooling_output_size(int(in[3]), n.kernel[1], n.pad[1], n.stride[1], n.ceil_mode));
            } else if (n.type == "GlobalPooling") {
                n.kind = k_gpool;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                DLPRIM_CHECK(in.size() == 4);
                std::string mode = o.get("mode", "max");
                DLPRIM_CHECK(mode == "max" || mode == "avg");
                n.max_mode = mode == "max";
                specs_[n.outputs[0]] = Shape(in[0], in[1], 1, 1);
            } else if (n.type == "Elementwise") {
                n.kind = k_eltwise;
                DLPRIM_CHECK(n.inputs.size() == 2 && n.outputs.size() == 1);
                n.broadcast = spec(n.inputs[0]) != spec(n.inputs[1]);
                std::string op = o.get("operation", "sum");
                if (op == "sum")
                    n.eltwise_op = DLP_ELTWISE_SUM;
                else if (op == "prod")
                    n.eltwise_op = DLP_ELTWISE_PROD;
                else if (op == "max")
                    n.eltwise_op = DLP_ELTWISE_MAX;
                else
                    throw ValidationError("Unsupported Elementwise operation " + op);
                n.coef[0] = o.get("coef1", 1.0f);
                n.coef[1] = o.get("coef2", 1.0f);
                specs_[n.outputs[0]] = n.broadcast ? broadcast_shape(spec(n.inputs[0]), spec(n.inputs[1]), n.name) : spec(n.inputs[0]);
            } else if (n.type == "Softmax") {
                n.kind = k_softmax;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                Shape const &in = spec(n.inputs[0]);
                DLPRIM_CHECK(in.size() == 2 || in.size() == 3); // as core::softmax_forward
                n.log_softmax = o.type() == json::is_object ? o.get("log", false) : false;
                specs_[n.outputs[0]] = in;
            } else if (n.type == "Threshold" || n.type == "Abs" || n.type == "Hardtanh") {
                n.kind = k_pointwise;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1);
                const bool has = o.type() == json::is_object;
                if (n.type == "Threshold") {
                    n.pointwise_op = DLP_POINTWISE_THRESHOLD;
                    n.pointwise_p[0] = has ? o.get("threshold", 0.0f) : 0.0f;
                } else if (n.type == "Abs")
                    n.pointwise_op = DLP_POINTWISE_ABS;
                else {
                    n.pointwise_op = DLP_POINTWISE_HARDTANH;
                    n.pointwise_p[0] = has ? o.get("min_val", -1.0f) : -1.0f;
                    n.pointwise_p[1] = has ? o.get("max_val", 1.0f) : 1.0f;
                }
                specs_[n.outputs[0]] = spec(n.inputs[0]);
            } else if (n.type == "Concat") {
                n.kind = k_concat;
                DLPRIM_CHECK(!n.inputs.empty() && n.outputs.size() == 1);
                for (auto const &name : n.inputs)
                    if (name == n.outputs[0])
                        throw ValidationError("Concat in place (" + n.name + ")");
                n.dim = o.type() == json::is_object ? o.get("dim", 1) : 1;
                specs_[n.outputs[0]] = concat_shape(n);
            } else if (n.type == "Slice") {
                n.kind = k_slice;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1 && n.inputs[0] != n.outputs[0]);
                n.dim = o.get("dim", 1);
                n.slice_begin = o.get("begin", 0);
                n.slice_end = o.get("end", -1);
                specs_[n.outputs[0]] = slice_shape(n, spec(n.inputs[0]));
            } else if (n.type == "Reshape" || n.type == "Squeeze") { // views: no kernel, no memory
                n.kind = k_view;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1 && n.inputs[0] != n.outputs[0]);
                n.squeeze = n.type == "Squeeze";
                n.view_dims = o.type() == json::is_object ? int_list(o, "dims") : std::vector<int>();
                if (n.squeeze) {
                    if (o.type() == json::is_object && o.get("all", n.view_dims.empty()) && !n.view_dims.empty())
                        throw ValidationError("Can't use both squeeze all and squeeze by dims");
                } else if (n.view_dims.empty())
                    throw ValidationError("Empty reshape dims");
                specs_[n.outputs[0]] = view_shape(n, spec(n.inputs[0]));
                alias_of_[n.outputs[0]] = n.inputs[0];
            } else if (n.type == "Interpolation") { // InterpolationConfig::from_json and the constructor's checks, src/ops/interpolation.cpp:18-46
                n.kind = k_interp;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1 && n.inputs[0] != n.outputs[0]);
                n.out_hw[0] = o.get("out_h", -1);
                n.out_hw[1] = o.get("out_w", -1);
                n.scale_yx[0] = o.get("scale_y", -1.0);
                n.scale_yx[1] = o.get("scale_x", -1.0);
                n.align_corners = o.get("align_corners", false);
                std::string method = o.get<std::string>("method");
                if (method == "nearest")
                    n.interp_method = DLP_INTERPOLATE_NEAREST;
                else if (method == "nearest-exact")
                    n.interp_method = DLP_INTERPOLATE_NEAREST_EXACT;
                else if (method == "bilinear")
                    n.interp_method = DLP_INTERPOLATE_BILINEAR;
                else
                    throw ValidationError("Unsupported interpolation method " + method);
                DLPRIM_CHECK((n.scale_yx[0] <= 0) == (n.scale_yx[1] <= 0));
                DLPRIM_CHECK((n.out_hw[0] <= 0) == (n.out_hw[1] <= 0));
                DLPRIM_CHECK((n.scale_yx[1] <= 0) != (n.out_hw[1] <= 0));
                DLPRIM_CHECK(n.interp_method == DLP_INTERPOLATE_BILINEAR || !n.align_corners);
                specs_[n.outputs[0]] = interpolation_shape(n, spec(n.inputs[0]));
            } else if (n.type == "Reduction") { // ReductionConfig::from_json, src/ops/reduction.cpp:15-35
                n.kind = k_reduce;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1 && n.inputs[0] != n.outputs[0]);
                const bool has = o.type() == json::is_object;
                std::string method = has ? o.get("method", "sum") : "sum";
                if (method == "sum")
                    n.reduce_method = DLP_REDUCE_SUM;
                else if (method == "sumsq")
                    n.reduce_method = DLP_REDUCE_SUMSQ;
                else if (method == "abssum")
                    n.reduce_method = DLP_REDUCE_ABSSUM;
                else if (method == "mean")
                    n.reduce_method = DLP_REDUCE_MEAN;
                else
                    throw ValidationError("Unknown reduction method " + method);
                n.output_scale = has ? o.get("output_scale", 1.0f) : 1.0f;
                n.keep_dim = has ? o.get("keep_dim", true) : true;
                n.has_dims = has && !o.find("dims").is_undefined();
                if (n.has_dims) {
                    if (!o.find("start_axis").is_undefined())
                        throw ValidationError("Can't use both dims and start_axis in Reduction");
                    n.reduce_dims = int_list(o, "dims");
                    if (n.reduce_dims.empty())
                        throw ValidationError("Using dims in Reduction requires providing at least 1 dimension");
                } else
                    n.start_axis = has ? o.get("start_axis", 0) : 0;
                specs_[n.outputs[0]] = reduction_shape(n, spec(n.inputs[0]));
            } else if (n.type == "Parameter") { // the output is the parameter itself (ParameterConfig::from_json, src/ops/parameter.cpp:13-21)
                n.kind = k_param;
                DLPRIM_CHECK(n.inputs.empty() && n.outputs.size() == 1);
                std::string dt = o.get("dtype", "float");
                if (dt != "float" && dt != "float32")
                    throw NotImplementedError("Parameter of dtype " + dt + " (" + n.name + ")");
                Shape s = shape_of(o.get<std::vector<int>>("shape"));
                specs_[n.outputs[0]] = s;
                make_param(n, 0, s);
            } else if (n.type == "MSELoss") { // src/ops/mse_loss.cpp:29-42
                n.kind = k_mse_loss;
                DLPRIM_CHECK(n.inputs.size() == 2 && n.outputs.size() == 1);
                DLPRIM_CHECK(spec(n.inputs[0]) == spec(n.inputs[1]));
                DLPRIM_CHECK(!int_inputs_.count(n.inputs[0]) && !int_inputs_.count(n.inputs[1]));
                n.loss_reduce = loss_reduce_option(o);
                specs_[n.outputs[0]] = n.loss_reduce == DLP_LOSS_REDUCE_NONE ? spec(n.inputs[0]) : Shape(size_t(1));
            } else if (n.type == "NLLLoss") { // src/ops/nll_loss.cpp:29-45
                n.kind = k_nll_loss;
                DLPRIM_CHECK(n.inputs.size() == 2 && n.outputs.size() == 1);
                check_labels(n);
                n.loss_reduce = loss_reduce_option(o);
                specs_[n.outputs[0]] = Shape(n.loss_reduce == DLP_LOSS_REDUCE_NONE ? spec(n.inputs[0])[0] : size_t(1));
            } else if (n.type == "SoftmaxWithLoss") { // src/ops/softmax.cpp:71-89
                n.kind = k_softmax_loss;
                DLPRIM_CHECK(n.inputs.size() == 2 && n.outputs.size() == 1);
                check_labels(n);
                specs_[n.outputs[0]] = Shape(size_t(1));
            } else if (n.type == "Flatten") { // a view: [B, everything else]; no kernel, no memory
                n.kind = k_flatten;
                DLPRIM_CHECK(n.inputs.size() == 1 && n.outputs.size() == 1 && n.inputs[0] != n.outputs[0]);
                Shape const &in = spec(n.inputs[0]);
                specs_[n.outputs[0]] = Shape(in[0], in.size_no_batch());
                alias_of_[n.outputs[0]] = n.inputs[0];
            } else
                throw NotImplementedError("Operator type " + n.type + " (" + n.name + ")");
        }
        for (auto const &name : output_names_)
            spec(name);
    }

    // index of the next node after `from` that reads or writes tensor `t`, or -1
    int next_user(size_t from, std::string const &t) const
    {
        for (size_t i = from + 1; i < nodes_.size(); i++) {
            if (nodes_[i].skipped)
                continue;
            for (auto const &s : nodes_[i].inputs)
                if (s == t)
                    return int(i);
            for (auto const &s : nodes_[i].outputs)
                if (s == t)
                    return int(i);
        }
        return -1;
    }
    int readers_after(size_t from, std::string const &t) const
    {
        int c = 0;
        for (size_t i = from + 1; i < nodes_.size(); i++) {
            if (nodes_[i].skipped)
                continue;
            for (auto const &s : nodes_[i].inputs)
                if (s == t)
                    c++;
            bool rewritten = false;
            for (auto const &s : nodes_[i].outputs)
                if (s == t && std::find(nodes_[i].inputs.begin(), nodes_[i].inputs.end(), t) == nodes_[i].inputs.end())
                    rewritten = true;
            if (rewritten)
                break; // a new value under the same name
        }
        return c;
    }
    bool is_net_output(std::string const &t) const { return std::find(output_names_.begin(), output_names_.end(), t) != output_names_.end(); }

    int producer_before(size_t before, std::string const &t) const
    {
        for (size_t i = before; i-- > 0;) {
            if (nodes_[i].skipped)
                continue;
            for (auto const &s : nodes_[i].outputs)
                if (s == t)
                    return int(i);
        }
        return -1;
    }
    bool is_net_input(std::string const &t) const { return std::find(input_names_.begin(), input_names_.end(), t) != input_names_.end(); }

    // BatchNorm into the convolution / inner product that feeds only it
    void try_fold_batch_norm(size_t i)
    {
        Node &p = nodes_[i];
        if (!((p.kind == k_conv || p.kind == k_ip) && p.activation == StandardActivations::identity && !p.folded_bn && !p.residual))
            return;
        std::string const &t = p.outputs[0];
        int u = next_user(i, t);
        if (u >= 0 && nodes_[u].kind == k_bn && nodes_[u].inputs[0] == t && !is_net_output(t) &&
            (nodes_[u].outputs[0] == t || readers_after(i, t) == 1)) {
            Node &bn = nodes_[u];
            p.folded_bn = &bn;
            p.activation = bn.activation;
            p.outputs[0] = bn.outputs[0];
            bn.skipped = true;
        }
    }
    // Activation into the fused slot of its producer
    void try_merge_activation(size_t i)
    {
        Node &p = nodes_[i];
        if (!((p.kind == k_conv || p.kind == k_ip || p.kind == k_eltwise || p.kind == k_bn || p.kind == k_tconv) && p.activation == StandardActivations::identity))
            return;
        std::string const &t = p.outputs[0];
        int u = next_user(i, t);
        if (u >= 0 && nodes_[u].kind == k_act && nodes_[u].inputs[0] == t &&
            (nodes_[u].outputs[0] == t || (!is_net_output(t) && readers_after(i, t) == 1))) {
            Node &a = nodes_[u];
            p.activation = a.activation;
            p.outputs[0] = a.outputs[0];
            a.skipped = true;
        }
    }
    // A residual sum into the convolution that produces its later branch: the convolution then writes
    // act(conv + bias + coef * other) over the other branch, which must be dead after the sum.
    // Returns the index of that convolution, or -1.
    // the tensor whose memory `name` shares in the end (views of views, sums written over a branch that is itself a view)
    std::string alias_root(std::string name) const
    {
        for (size_t hops = 0; hops <= alias_of_.size(); hops++) {
            auto it = alias_of_.find(name);
            if (it == alias_of_.end())
                break;
            name = it->second;
        }
        return name;
    }

    int try_fuse_residual(size_t e)
    {
        Node &el = nodes_[e];
        if (el.kind != k_eltwise || el.broadcast || el.eltwise_op != DLP_ELTWISE_SUM || keep_intermediate_ || el.inputs[0] == el.inputs[1])
            return -1;
        const int p0 = producer_before(e, el.inputs[0]), p1 = producer_before(e, el.inputs[1]);
        const int side = p0 > p1 ? 0 : 1; // the branch that is produced later
        const int pi = side == 0 ? p0 : p1, ri = side == 0 ? p1 : p0;
        if (pi < 0 || ri < 0)
            return -1; // the other branch is a network input (never written over) or unknown
        Node &p = nodes_[size_t(pi)];
        std::string const a = el.inputs[size_t(side)], r = el.inputs[size_t(1 - side)];
        if (p.kind != k_conv || p.conv.groups != 1 || p.activation != StandardActivations::identity || p.residual || el.coef[side] != 1.0f)
            return -1;
        // 1x1 convolutions only: their epilogue is a large share of a short kernel and hides the extra reads;
        // behind a 3x3 convolution (matrix-bound, epilogue exposed) the fused read cost what the sum saved
        if (p.conv.kernel[0] != 1 || p.conv.kernel[1] != 1)
            return -1;
        if (is_net_output(a) || is_net_output(r) || is_net_input(r) || readers_after(size_t(pi), a) != 1 || next_user(e, r) >= 0)
            return -1; // both branches must end in this sum
        if (spec(a) != spec(r) || std::find(p.inputs.begin(), p.inputs.end(), r) != p.inputs.end())
            return -1;
        for (size_t i = size_t(pi) + 1; i < e; i++) // nothing between the convolution and the sum may still read the other branch
            if (!nodes_[i].skipped && std::find(nodes_[i].inputs.begin(), nodes_[i].inputs.end(), r) != nodes_[i].inputs.end())
                return -1;
        p.residual = true;
        p.residual_factor = el.coef[1 - side];
        p.activation = el.activation;
        p.outputs[0] = el.outputs[0];
        p.inputs.push_back(r); // keeps the branch alive until the convolution has run
        alias_of_[el.outputs[0]] = r;
        el.skipped = true;
        return pi;
    }

    // A depthwise 3x3 convolution into the 1x1 convolution that is its only reader (the pair a MobileNet block ends in), where
    // the device code runs the pair as one kernel: the 1x1 node then reads the depthwise node's input and runs both.
    void try_fuse_depthwise_pointwise(size_t i)
    {
        Node &d = nodes_[i];
        if (d.kind != k_conv || d.residual || d.dw_node >= 0 || dtype_ != float_data || keep_intermediate_ || ctx_.is_cpu_context())
            return;
        if (d.conv.groups != d.conv.channels_in || d.conv.channels_out != d.conv.channels_in || d.conv.kernel[0] != 3 || d.conv.kernel[1] != 3)
            return;
        if (!d.algo.empty() && d.algo != "depthwise_separable")
            return; // the network file asks for another algorithm
        std::string const t = d.outputs[0];
        const int u = next_user(i, t);
        if (u < 0 || is_net_output(t) || readers_after(i, t) != 1)
            return;
        Node &p = nodes_[size_t(u)];
        if (p.kind != k_conv || p.dw_node >= 0 || p.inputs[0] != t || p.conv.groups != 1 || p.conv.kernel[0] != 1 || p.conv.kernel[1] != 1 ||
            p.conv.stride[0] != 1 || p.conv.stride[1] != 1 || p.conv.pad[0] != 0 || p.conv.pad[1] != 0 || (!p.algo.empty() && p.algo != "gemm"))
            return;
        std::string const &x = d.inputs[0];
        // a 1x1 node that already carries a residual sum writes over the skip branch: when that branch is the depthwise input
        // (x -> depthwise -> 1x1 -> + x), the fused kernel would store output rows over input rows that other workgroups still read
        if (p.residual && (alias_root(p.outputs[0]) == alias_root(x) || std::find(p.inputs.begin() + 1, p.inputs.end(), x) != p.inputs.end()))
            return;
        for (size_t k = i + 1; k <= size_t(u); k++) // the depthwise input must still hold its value when the 1x1 node runs
            if (!nodes_[k].skipped && std::find(nodes_[k].outputs.begin(), nodes_[k].outputs.end(), x) != nodes_[k].outputs.end())
                return;
        core::Conv2DSettings cfg(d.conv, spec(x), dtype_);
        if (!core::DepthwisePointwiseForward::supported(cfg, d.activation, p.conv.channels_out, p.activation))
            return;
        p.dw_node = int(i);
        p.inputs[0] = x;
        d.skipped = true;
    }

    // A max pooling into the convolution that feeds only it, where the device code runs the pair as one kernel (the bfloat16 7x7
    // stride-2 stem of a ResNet and its 3x3 stride-2 pooling): the convolution node then writes the pooling's tensor.
    void try_fuse_max_pool(size_t i)
    {
        Node &c = nodes_[i];
        if (!fuse_max_pool_ || c.kind != k_conv || c.residual || c.dw_node >= 0 || c.pool_node >= 0 || dtype_ != bfloat16_data || keep_intermediate_ || ctx_.is_cpu_context())
            return;
        std::string const t = c.outputs[0];
        const int u = next_user(i, t);
        if (u < 0 || is_net_output(t) || readers_after(i, t) != 1)
            return;
        Node &pl = nodes_[size_t(u)];
        if (pl.kind != k_pool || !pl.max_mode || pl.inputs[0] != t || pl.kernel[0] != pl.kernel[1] || pl.stride[0] != pl.stride[1] || pl.pad[0] != pl.pad[1])
            return;
        try { // the library decides: an operator of this geometry is asked
            core::Conv2DSettings cfg(c.conv, spec(c.inputs[0]), dtype_);
            core::Conv2DForward::create(ctx_, cfg, c.bias || c.folded_bn, c.activation, c.algo)->fuse_max_pool(pl.kernel[0], pl.stride[0], pl.pad[0], pl.ceil_mode);
        } catch (NotImplementedError const &) {
            return;
        }
        c.pool_node = u;
        c.outputs[0] = pl.outputs[0];
        pl.skipped = true;
    }

    void rewrite_graph()
    {
        for (size_t i = 0; i < nodes_.size(); i++) {
            if (nodes_[i].skipped)
                continue;
            try_fold_batch_norm(i);
            try_merge_activation(i);
            const int p = try_fuse_residual(i);
            if (p >= 0)
                try_merge_activation(size_t(p));
        }
        for (size_t i = 0; i < nodes_.size(); i++) // after the loop above: both nodes have their final activation and bias
            if (!nodes_[i].skipped)
                try_fuse_depthwise_pointwise(i);
        for (size_t i = 0; i < nodes_.size(); i++)
            if (!nodes_[i].skipped)
                try_fuse_max_pool(i);
    }

    void create_conv_operator(Node &n, Shape const &in)
    {
        if (n.dw_node >= 0) { // in: the input of the depthwise convolution
            Node &d = nodes_[size_t(n.dw_node)];
            core::Conv2DSettings dcfg(d.conv, in, dtype_);
            n.dwpw_op.reset(new core::DepthwisePointwiseForward(ctx_, dcfg, d.bias || d.folded_bn, d.activation, n.conv.channels_out, n.bias || n.folded_bn,
                                                                n.activation));
            if (n.residual)
                n.dwpw_op->accumulate_before_activation(true);
            n.planned_in = in;
            return;
        }
        core::Conv2DSettings cfg(n.conv, in, dtype_);
        n.conv_op = core::Conv2DForward::create(ctx_, cfg, n.bias || n.folded_bn, n.activation, n.algo);
        if (n.residual)
            n.conv_op->accumulate_before_activation(true);
        if (n.pool_node >= 0) {
            Node const &pl = nodes_[size_t(n.pool_node)];
            n.conv_op->fuse_max_pool(pl.kernel[0], pl.stride[0], pl.pad[0], pl.ceil_mode);
        }
        const bool x_cl = is_channels_last(n.inputs[0]), y_cl = is_channels_last(n.outputs[0]);
        if (x_cl || y_cl)
            n.conv_op->channels_last(x_cl, y_cl);
        n.planned_in = in;
        workspace_bytes_ = std::max(workspace_bytes_, n.conv_op->workspace());
    }
    void create_tconv_operator(Node &n, Shape const &in)
    {
        core::Conv2DSettings cfg(n.conv, in, dtype_);
        n.tconv_op.reset(new core::TransposedConv2DForward(ctx_, cfg, n.output_pad, n.bias, n.activation, n.algo));
        n.planned_in = in;
        workspace_bytes_ = std::max(workspace_bytes_, n.tconv_op->workspace());
    }
    void pack_conv_weights(Node &n, ExecutionContext const &e)
    {
        const size_t bytes = n.conv_op->packed_size();
        if (bytes > 0 && n.packed.shape().total_size() != bytes)
            n.packed = Tensor(ctx_, Shape(bytes), uint8_data);
        n.conv_op->pack(n.use_w_dev ? n.w_dev : param(n.param_names[0]), n.packed, e);
        n.is_packed = true;
    }

    // Which tensors are kept channels-last (bfloat16 only; intermediate tensors cannot be read from outside then, see
    // keep_intermediate_tensors).  Tensors that share memory -- views, the output of a fused residual sum and the branch it is written
    // over -- form a group with one layout.  A group goes channels-last when every operator that writes it is a convolution that can
    // (algorithm gemm on the bf16 matrix instruction: one group, channels in multiples of 32 in and of 8 out, relu-like activation),
    // every reader is such a convolution or a global pooling, none of its names is a network input or output, and at least one
    // reader gains: measured inside ResNet-50 at batch 128, the channels-last loader beats the others on 1x1 layers of more than 64
    // input channels, on everything with a stride and on images below 14 x 14, and loses to the LDS-patch kernel on larger 3x3
    // stride-1 layers and to the dense loader on 1x1 layers of 64 channels.
    void plan_layouts()
    {
        cl_groups_.clear();
        if (!channels_last_ || dtype_ != bfloat16_data || keep_intermediate_ || ctx_.is_cpu_context())
            return;
        struct Use {
            std::vector<Node const *> writers, readers;
            bool boundary = false;
        };
        std::map<std::string, Use> groups;
        for (auto const &n : nodes_) {
            if (n.skipped)
                continue;
            for (auto const &t : n.inputs)
                groups[alias_root(t)].readers.push_back(&n);
            for (auto const &t : n.outputs)
                groups[alias_root(t)].writers.push_back(&n);
        }
        for (auto const &t : input_names_)
            groups[alias_root(t)].boundary = true;
        for (auto const &t : output_names_)
            groups[alias_root(t)].boundary = true;
        for (auto const &al : alias_of_) // a view shares memory but not the layout question: its readers see another shape
            if (is_net_output(al.first) || is_net_input(al.first))
                groups[alias_root(al.first)].boundary = true;
        auto conv_ok = [&](Node const &n) {
            return n.kind == k_conv && n.dw_node < 0 && n.conv.groups == 1 && n.conv.channels_in % 32 == 0 && n.conv.channels_out % 8 == 0 &&
                   (n.algo.empty() || n.algo == "auto" || n.algo == "gemm") &&
                   (n.activation == StandardActivations::identity || n.activation == StandardActivations::relu || n.activation == StandardActivations::relu6);
        };
        auto gains = [&](Node const &n) {
            if (n.kind != k_conv)
                return false;
            Shape const &in = spec(n.inputs[0]);
            const bool unit_stride = n.conv.stride[0] == 1 && n.conv.stride[1] == 1;
            if (n.conv.kernel[0] == 3 && n.conv.kernel[1] == 3 && unit_stride)
                return in[2] * in[3] < 14 * 14;
            return !(n.conv.kernel[0] == 1 && n.conv.kernel[1] == 1 && unit_stride && n.conv.channels_in <= 64);
        };
        for (auto const &g : groups) {
            Use const &u = g.second;
            if (u.boundary || u.writers.empty() || u.readers.empty())
                continue;
            bool ok = true, any_gain = false;
            for (Node const *n : u.writers)
                ok = ok && conv_ok(*n);
            for (Node const *n : u.readers) {
                ok = ok && (conv_ok(*n) || n->kind == k_gpool);
                any_gain = any_gain || gains(*n);
            }
            if (ok && any_gain)
                cl_groups_.insert(g.first);
        }
    }
    bool is_channels_last(std::string const &t) const { return !cl_groups_.empty() && cl_groups_.count(alias_root(t)) != 0; }

    void create_operators()
    {
        workspace_bytes_ = 0;
        if (ctx_.is_cpu_context())
            return; // shapes and the memory plan only: the operators exist on a device
        for (auto &n : nodes_) {
            if (n.skipped)
                continue;
            Shape const &in = n.inputs.empty() ? spec(n.outputs[0]) : spec(n.inputs[0]);
            workspace_bytes_ = std::max(workspace_bytes_, node_workspace(n));
            switch (n.kind) {
            case k_conv: create_conv_operator(n, in); break;
            case k_tconv: create_tconv_operator(n, in); break;
            case k_ip: {
                core::IPSettings cfg;
                cfg.inputs = n.ip_inputs;
                cfg.outputs = n.ip_outputs;
                cfg.optimal_batch_size = int(in[0]);
                cfg.dtype = dtype_;
                n.ip_op = core::IPForward::create(ctx_, cfg, n.bias || n.folded_bn, n.activation);
                break;
            }
            case k_pool:
                n.pool_op = n.max_mode ? core::Pooling2DForward::create_max_pooling(ctx_, n.kernel, n.pad, n.stride, dtype_)
                                       : core::Pooling2DForward::create_avg_pooling(ctx_, n.kernel, n.pad, n.stride, n.count_include_pad, dtype_);
                break;
            case k_gpool:
                n.pool_op = n.max_mode ? core::Pooling2DForward::create_global_max_pooling(ctx_, in, dtype_)
                                       : core::Pooling2DForward::create_global_avg_pooling(ctx_, in, dtype_);
                if (is_channels_last(n.inputs[0]))
                    n.pool_op->channels_last(true);
                break;
            default: break;
            }
        }
        if (workspace_bytes_ > 0)
            workspace_ = Tensor(ctx_, Shape(workspace_bytes_), uint8_data);
    }

    // Tensor memory.  Network inputs and outputs own their memory; an intermediate tensor takes the
    // smallest free chunk that fits when its producer runs and gives it back after its last reader
    // (an operator's outputs are placed before its inputs are released, so they never alias).
    void allocate_tensors()
    {
        std::map<std::string, int> last_use;
        for (size_t i = 0; i < nodes_.size(); i++) {
            if (nodes_[i].skipped)
                continue;
            for (auto const &t : nodes_[i].inputs)
                last_use[t] = int(i);
            for (auto const &t : nodes_[i].outputs)
                last_use[t] = std::max(last_use.count(t) ? last_use[t] : -1, int(i));
        }
        // a network output that shares memory with an intermediate tensor (a view of it, a sum written over it) keeps that memory
        // for good: no later operator may be given the chunk
        for (auto const &name : output_names_)
            if (alias_of_.count(name))
                last_use[name] = int(nodes_.size());
        // a view and its source live as long as either is used, along chains of any length
        for (bool changed = true; changed;) {
            changed = false;
            for (auto const &al : alias_of_) {
                const int a = last_use.count(al.first) ? last_use[al.first] : -1, b = last_use.count(al.second) ? last_use[al.second] : -1;
                if (a != b) {
                    last_use[al.first] = last_use[al.second] = std::max(a, b);
                    changed = true;
                }
            }
        }
        tensor_memory_ = 0;
        auto own = [&](std::string const &name) {
            tensors_[name] = Tensor(ctx_, spec(name), int_inputs_.count(name) ? int32_data : dtype_);
            tensor_memory_ += tensors_[name].memory_size();
        };
        for (auto const &name : input_names_)
            own(name);
        struct Chunk {
            Tensor mem;
            size_t bytes;
        };
        std::vector<Chunk> free_chunks;
        std::map<std::string, Chunk> held;
        for (size_t i = 0; i < nodes_.size(); i++) {
            Node &n = nodes_[i];
            if (n.skipped)
                continue;
            for (auto const &t : n.outputs) {
                if (tensors_.count(t))
                    continue; // in place, or written before
                auto al = alias_of_.find(t);
                if (al != alias_of_.end()) { // written over the other branch of a residual sum: takes over its memory
                    tensors_[t] = tensors_.at(al->second);
                    tensors_[t].reshape(spec(t));
                    auto h = held.find(al->second);
                    if (h != held.end()) {
                        held[t] = h->second;
                        held.erase(h);
                    }
                    continue;
                }
                if (keep_intermediate_ || is_net_output(t)) {
                    own(t);
                    continue;
                }
                const size_t bytes = spec(t).total_size() * size_t(size_of_data_type(dtype_));
                int best = -1;
                for (size_t c = 0; c < free_chunks.size(); c++)
                    if (free_chunks[c].bytes >= bytes && (best < 0 || free_chunks[c].bytes < free_chunks[size_t(best)].bytes))
                        best = int(c);
                Chunk ch;
                if (best >= 0) {
                    ch = free_chunks[size_t(best)];
                    free_chunks.erase(free_chunks.begin() + best);
                } else {
                    ch.mem = Tensor(ctx_, Shape(bytes), uint8_data);
                    ch.bytes = bytes;
                    tensor_memory_ += bytes;
                }
                tensors_[t] = ch.mem.sub_tensor(0, spec(t), dtype_);
                held[t] = ch;
            }
            std::set<std::string> touched(n.inputs.begin(), n.inputs.end());
            touched.insert(n.outputs.begin(), n.outputs.end());
            for (auto const &t : touched) {
                auto h = held.find(t);
                if (h != held.end() && last_use[t] == int(i)) {
                    free_chunks.push_back(h->second);
                    held.erase(h);
                }
            }
        }
        for (auto const &name : output_names_)
            if (!tensors_.count(name))
                throw ValidationError("Output tensor " + name + " is not produced by any operator");
    }

    void prepare_derived_parameters(Node &n, ExecutionContext const &e)
    {
        auto bn_scale_shift = [&](Node &bn, std::vector<float> &scale, std::vector<float> &shift) {
            Tensor &mean = param(bn.param_names[0]), &var = param(bn.param_names[1]);
            const size_t c = mean.shape().total_size();
            scale.resize(c);
            shift.resize(c);
            for (size_t i = 0; i < c; i++) { // the order of operations of src/ops/batch_normalization.cpp:218-226
                float alpha = 1.0f / std::sqrt(var.data<float>()[i] + bn.eps);
                float beta = -mean.data<float>()[i] * alpha;
                if (bn.affine) {
                    const float g = param(bn.param_names[2]).data<float>()[i];
                    alpha *= g;
                    beta = g * beta + param(bn.param_names[3]).data<float>()[i];
                }
                scale[i] = alpha;
                shift[i] = beta;
            }
        };
        if (n.kind == k_bn) {
            std::vector<float> scale, shift;
            bn_scale_shift(n, scale, shift);
            n.scale = Tensor(ctx_, Shape(scale.size()));
            n.shift = Tensor(ctx_, Shape(shift.size()));
            std::copy(scale.begin(), scale.end(), n.scale.data<float>());
            std::copy(shift.begin(), shift.end(), n.shift.data<float>());
            n.scale.to_device(e);
            n.shift.to_device(e);
        } else if (n.kind == k_conv || n.kind == k_ip) {
            // the weights the kernel reads: the parameter itself, or a copy with the BatchNorm folded in
            // and / or in the 16-bit storage type
            Tensor &w = param(n.param_names[0]);
            const size_t total = w.shape().total_size();
            n.use_w_dev = n.folded_bn != nullptr || dtype_ != float_data;
            if (n.use_w_dev) {
                std::vector<float> wf(w.data<float>(), w.data<float>() + total);
                if (n.folded_bn) {
                    std::vector<float> scale, shift;
                    bn_scale_shift(*n.folded_bn, scale, shift);
                    const size_t cout = scale.size(), per = total / cout;
                    n.b_dev = Tensor(ctx_, Shape(cout));
                    for (size_t c = 0; c < cout; c++) {
                        for (size_t k = 0; k < per; k++)
                            wf[c * per + k] *= scale[c];
                        const float b = n.bias ? param(n.param_names[1]).data<float>()[c] : 0.0f;
                        n.b_dev.data<float>()[c] = shift[c] + b * scale[c];
                    }
                    n.b_dev.to_device(e);
                }
                n.w_dev = Tensor(ctx_, w.shape(), dtype_);
                if (dtype_ == float_data)
                    std::copy(wf.begin(), wf.end(), n.w_dev.data<float>());
                else
                    for (size_t k = 0; k < total; k++)
                        n.w_dev.data<uint16_t>()[k] = to_bf16_bits(wf[k]);
                n.w_dev.to_device(e);
            }
        }
        if (n.kind == k_param && dtype_ != float_data) { // the values in the storage type
            Tensor &w = param(n.param_names[0]);
            n.w_dev = Tensor(ctx_, w.shape(), dtype_);
            for (size_t k = 0; k < w.shape().total_size(); k++)
                n.w_dev.data<uint16_t>()[k] = to_bf16_bits(w.data<float>()[k]);
            n.w_dev.to_device(e);
        }
        if (n.kind == k_conv && prepack_ && n.conv_op)
            pack_conv_weights(n, e);
        if (n.kind == k_conv && n.dw_node >= 0) // the depthwise convolution that this node runs as well
            prepare_derived_parameters(nodes_[size_t(n.dw_node)], e);
    }

    void run(Node &n, ExecutionContext const &e)
    {
        Tensor &y = tensor(n.outputs[0]);
        Tensor &x = n.inputs.empty() ? y : tensor(n.inputs[0]);
        void *ws = workspace_bytes_ > 0 ? workspace_.device_ptr() : nullptr;
        const size_t ws_bytes = workspace_bytes_ > 0 ? workspace_.memory_size() : 0;
        switch (n.kind) {
        case k_interp: {
            Shape const &xs = x.shape(), &ys = y.shape();
            details::check_status(dlp_interpolate2d_fwd_enqueue(int(dtype_), n.interp_method, n.align_corners ? 1 : 0, n.scale_yx[0], n.scale_yx[1],
                                                                int(xs[0] * xs[1]), int(xs[2]), int(xs[3]), int(ys[2]), int(ys[3]), x.device_ptr(),
                                                                y.device_ptr(), e.stream()));
            break;
        }
        case k_reduce: {
            Shape const &xs = x.shape();
            std::vector<int> mask = reduced_axes(n, xs), dims(size_t(xs.size()));
            for (int a = 0; a < xs.size(); a++)
                dims[size_t(a)] = int(xs[a]);
            details::check_status(dlp_reduce_fwd_enqueue(int(dtype_), n.reduce_method, n.output_scale, xs.size(), dims.data(), mask.data(), x.device_ptr(),
                                                         y.device_ptr(), ws, ws_bytes, e.stream()));
            break;
        }
        case k_param: { // Parameter::forward copies the parameter into the output (src/ops/parameter.cpp:23-45)
            Tensor &w = dtype_ == float_data ? param(n.param_names[0]) : n.w_dev;
            details::check_status(dlp_copy2d_enqueue(y.device_ptr(), w.memory_size(), w.device_ptr(), w.memory_size(), w.memory_size(), 1, e.stream()));
            break;
        }
        case k_mse_loss:
            details::check_status(dlp_mse_loss_fwd_enqueue(int(dtype_), n.loss_reduce, x.shape().total_size(), x.device_ptr(),
                                                           tensor(n.inputs[1]).device_ptr(), y.device_ptr(), ws, ws_bytes, e.stream()));
            break;
        case k_nll_loss: {
            Tensor &lbl = tensor(n.inputs[1]);
            details::check_status(dlp_nll_loss_fwd_enqueue(int(dtype_), int(lbl.dtype()), n.loss_reduce, int(x.shape()[0]), int(x.shape()[1]), x.device_ptr(),
                                                           lbl.device_ptr(), y.device_ptr(), e.stream()));
            break;
        }
        case k_softmax_loss: {
            Tensor &lbl = tensor(n.inputs[1]);
            details::check_status(dlp_softmax_loss_fwd_enqueue(int(dtype_), int(lbl.dtype()), int(x.shape()[0]), int(x.shape()[1]), x.device_ptr(),
                                                               lbl.device_ptr(), y.device_ptr(), ws, ws_bytes, e.stream()));
            break;
        }
        case k_conv: {
            Tensor &w = n.use_w_dev ? n.w_dev : param(n.param_names[0]);
            Tensor *b = n.folded_bn ? &n.b_dev : n.bias ? &param(n.param_names[1]) : nullptr;
            const float factor = n.residual ? n.residual_factor : 0.0f;
            if (n.dw_node >= 0) {
                Node &d = nodes_[size_t(n.dw_node)];
                Tensor &dw = d.use_w_dev ? d.w_dev : param(d.param_names[0]);
                Tensor *db = d.folded_bn ? &d.b_dev : d.bias ? &param(d.param_names[1]) : nullptr;
                n.dwpw_op->enqueue(x, dw, db, w, b, y, factor, e);
                break;
            }
            if (n.is_packed)
                n.conv_op->enqueue_packed(x, w, n.packed, b, y, workspace_, factor, e);
            else
                n.conv_op->enqueue(x, w, b, y, workspace_, factor, e);
            break;
        }
        case k_ip: {
            Tensor &w = n.use_w_dev ? n.w_dev : param(n.param_names[0]);
            Tensor *b = n.folded_bn ? &n.b_dev : n.bias ? &param(n.param_names[1]) : nullptr;
            n.ip_op->enqueue(x, w, b, y, e);
            break;
        }
        case k_tconv:
            n.tconv_op->enqueue(x, param(n.param_names[0]), n.bias ? &param(n.param_names[1]) : nullptr, y, workspace_, e);
            break;
        case k_bn: {
            Shape const &s = x.shape();
            details::check_status(dlp_channel_affine_fwd_enqueue(int(dtype_), int(n.activation), int(s[0]), int(s[1]),
                                                                 int(s.total_size() / (s[0] * s[1])), x.device_ptr(),
                                                                 static_cast<const float *>(n.scale.device_ptr()),
                                                                 static_cast<const float *>(n.shift.device_ptr()), y.device_ptr(), e.stream()));
            break;
        }
        case k_act:
            details::check_status(dlp_activation_fwd_enqueue(int(dtype_), int(n.activation), x.shape().total_size(), x.device_ptr(), y.device_ptr(),
                                                             e.stream()));
            break;
        case k_pool:
        case k_gpool: n.pool_op->enqueue(x, y, e); break;
        case k_softmax: {
            Shape const &s = x.shape();
            details::check_status(dlp_softmax_fwd_enqueue(int(dtype_), n.log_softmax ? 1 : 0, int(s[0]), int(s[1]), s.size() == 3 ? int(s[2]) : 1,
                                                          x.device_ptr(), y.device_ptr(), e.stream()));
            break;
        }
        case k_pointwise:
            details::check_status(dlp_pointwise_fwd_enqueue(int(dtype_), n.pointwise_op, n.pointwise_p[0], n.pointwise_p[1], x.shape().total_size(), x.device_ptr(),
                                                            y.device_ptr(), e.stream()));
            break;
        case k_flatten:
        case k_view: break; // the output is a view of the input
        case k_concat: { // every input goes to its range of the axis: [outer][axis][inner]
            Shape const &ys = y.shape();
            size_t outer = 1, inner = size_t(size_of_data_type(dtype_));
            for (int j = 0; j < n.dim; j++)
                outer *= ys[j];
            for (int j = n.dim + 1; j < ys.size(); j++)
                inner *= ys[j];
            size_t offset = 0;
            for (auto const &name : n.inputs) {
                Tensor &xi = tensor(name);
                const size_t slice = xi.shape()[n.dim];
                details::check_status(dlp_copy2d_enqueue(static_cast<char *>(y.device_ptr()) + offset * inner, ys[n.dim] * inner, xi.device_ptr(), slice * inner,
                                                         slice * inner, outer, e.stream()));
                offset += slice;
            }
            break;
        }
        case k_slice: {
            Shape const &xs = x.shape();
            size_t outer = 1, inner = size_t(size_of_data_type(dtype_));
            for (int j = 0; j < n.dim; j++)
                outer *= xs[j];
            for (int j = n.dim + 1; j < xs.size(); j++)
                inner *= xs[j];
            const size_t slice = y.shape()[n.dim];
            details::check_status(dlp_copy2d_enqueue(y.device_ptr(), slice * inner, static_cast<const char *>(x.device_ptr()) + size_t(n.slice_begin) * inner,
                                                     xs[n.dim] * inner, slice * inner, outer, e.stream()));
            break;
        }
        case k_eltwise: {
            Tensor &x1 = tensor(n.inputs[1]);
            if (n.broadcast) {
                const int rank = y.shape().size();
                int sa[max_tensor_dim], sb[max_tensor_dim];
                for (int j = 0; j < rank; j++) {
                    const int ja = j - (rank - x.shape().size()), jb = j - (rank - x1.shape().size());
                    sa[j] = ja >= 0 ? int(x.shape()[ja]) : 1;
                    sb[j] = jb >= 0 ? int(x1.shape()[jb]) : 1;
                }
                details::check_status(dlp_eltwise_bcast_fwd_enqueue(int(dtype_), n.eltwise_op, n.coef[0], n.coef[1], int(n.activation), rank, sa, sb, x.device_ptr(),
                                                                    x1.device_ptr(), y.device_ptr(), e.stream()));
                break;
            }
            details::check_status(dlp_eltwise_fwd_enqueue_dtype(int(dtype_), n.eltwise_op, n.coef[0], n.coef[1], int(n.activation), x.shape().total_size(), x.device_ptr(),
                                                          x1.device_ptr(), y.device_ptr(), e.stream()));
            break;
        }
        }
    }

    Context ctx_;
    std::vector<Node> nodes_;
    std::vector<std::string> input_names_, output_names_;
    std::map<std::string, Shape> specs_;
    std::map<std::string, Tensor> tensors_, params_;
    std::set<std::string> int_inputs_; // inputs stored as int32 (labels), whatever the storage type of the others
    std::map<std::string, std::string> alias_of_; // output of a fused residual sum -> the branch it is written over
    Tensor workspace_;
    size_t workspace_bytes_ = 0, tensor_memory_ = 0;
    bool keep_intermediate_ = false, fuse_ = true, prepack_ = true, ready_ = false;
    bool channels_last_ = true;
    bool fuse_max_pool_ = true;
    std::set<std::string> cl_groups_; // tensors kept channels-last, by the name their memory goes by (alias_root)
    DataType dtype_ = float_data;
    std::shared_ptr<dlp_graph> graph_;
    void *graph_stream_ = nullptr;
};

} // namespace dlprim
