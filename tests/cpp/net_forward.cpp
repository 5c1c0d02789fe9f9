// Driver for dlprim::Net (include/dlprim/net.hpp), used by tests/test_net.py the way dlprimitives'
// own tools drive a network (tools/image_predict.cpp, docs/network_json_format.md):
//
//   net_forward json <file.json>
//       parse and print the document again (no GPU)
//   net_forward plan <net.json> [keep] [nofuse]
//       shape inference, graph rewrites and memory plan on a CPU context (no GPU); prints
//       "operators <n> tensor_memory <bytes>" and one "tensor <name> <dims...>" line per output
//   net_forward run <net.json> <params.dlpw> <inputs.bin> <outputs.bin> [keep] [nofuse] [nopack] [graph] [bf16] [nchw] [poolop] [batch=<n>] [resave=<file.dlpw>] [repeat=<n>]
//       (batch=<n>: the inputs are reshaped to n images and Net::reshape() is called before the pass)
//       (bf16: tensors and weights stored as bfloat16 on the device; files stay float32; nchw: no channels-last tensors between bf16 convolutions;
//        poolop: the max pooling behind a bf16 stem stays an operator of its own)
//       loads the network and its parameters on HIP device 0, reads the inputs (float32, in the
//       network's input order), runs forward and writes the outputs (float32, in output order)
//   net_forward time <net.json> [warmup=<n>] [iters=<n>] [keep] [nofuse] [graph] [bf16] [nchw] [poolop]
//       (graph: the forward pass is recorded once as a HIP graph and replayed)
//       random parameters and inputs, ms per forward pass on HIP device 0 (what the reference's
//       tools/benchmark.cpp reports for its docs/nets_for_benchmark files)
#include <dlprim/net.hpp>

#include <cstdio>
#include <cstring>
#include <fstream>
#include <chrono>
#include <iostream>
#include <random>
#include <sstream>
#include <vector>

namespace dp = dlprim;

static int usage()
{
    std::fprintf(stderr, "usage: net_forward json <file> | plan <net.json> [keep] [nofuse] | run <net.json> <params> <in.bin> <out.bin> [keep] [nofuse] [resave=<file>] [repeat=<n>] | time <net.json> [warmup=<n>] [iters=<n>] [keep] [nofuse]\n");
    return 2;
}

int main(int argc, char **argv)
{
    if (argc < 3)
        return usage();
    std::string cmd = argv[1];
    try {
        if (cmd == "json") {
            std::ifstream f(argv[2]);
            if (!f)
                throw dp::ValidationError(std::string("cannot open ") + argv[2]);
            dp::json::value v = dp::json::value::load(f);
            std::cout << v.save() << std::endl;
            return 0;
        }
        bool keep = false, fuse = true, graph = false, prepack = true, bf16 = false, nchw = false, poolop = false;
        std::string resave;
        int repeat = 1, warmup = 5, iters = 20, batch = 0;
        const int first_flag = (cmd == "plan" || cmd == "time") ? 3 : 6;
        for (int i = first_flag; i < argc; i++) {
            std::string a = argv[i];
            if (a == "keep")
                keep = true;
            else if (a == "nofuse")
                fuse = false;
            else if (a == "graph")
                graph = true;
            else if (a == "nopack")
                prepack = false;
            else if (a == "bf16")
                bf16 = true;
            else if (a == "nchw")
                nchw = true;
            else if (a == "poolop")
                poolop = true;
            else if (a.compare(0, 7, "resave=") == 0)
                resave = a.substr(7);
            else if (a.compare(0, 7, "repeat=") == 0)
                repeat = std::atoi(a.c_str() + 7);
            else if (a.compare(0, 6, "batch=") == 0)
                batch = std::atoi(a.c_str() + 6);
            else if (a.compare(0, 7, "warmup=") == 0)
                warmup = std::atoi(a.c_str() + 7);
            else if (a.compare(0, 6, "iters=") == 0)
                iters = std::atoi(a.c_str() + 6);
            else
                return usage();
        }
        if (cmd == "plan") {
            dp::Context ctx(dp::Context::cpu);
            dp::Net net(ctx);
            net.keep_intermediate_tensors(keep);
            net.fuse(fuse);
            net.prepack(prepack);
            net.channels_last(!nchw);
            net.fuse_max_pooling(!poolop);
            net.storage_type(bf16 ? dp::bfloat16_data : dp::float_data);
            net.load_from_json_file(argv[2]);
            net.setup();
            std::printf("operators %zu tensor_memory %zu\n", net.operators_run(), net.tensor_memory());
            for (auto const &name : net.output_names()) {
                dp::Shape const &s = net.tensor(name).shape();
                std::printf("tensor %s", name.c_str());
                for (int i = 0; i < s.size(); i++)
                    std::printf(" %zu", s[i]);
                std::printf("\n");
            }
            return 0;
        }
        if (cmd == "time") {
            dp::Context ctx(dp::Context::hip, 0, 0);
            dp::Net net(ctx);
            net.keep_intermediate_tensors(keep);
            net.fuse(fuse);
            net.prepack(prepack);
            net.channels_last(!nchw);
            net.fuse_max_pooling(!poolop);
            net.storage_type(bf16 ? dp::bfloat16_data : dp::float_data);
            net.load_from_json_file(argv[2]);
            net.setup();
            std::mt19937 rng(1);
            for (auto &p : net.params()) {
                dp::Shape const &s = p.second.shape();
                const size_t n = s.total_size();
                const bool variance = p.first.find("running_var") != std::string::npos;
                // keeps activations of order one: weights scaled by fan-in, variances near one
                const float range = s.size() > 1 ? std::sqrt(6.0f / float(n / s[0])) : 0.5f;
                std::uniform_real_distribution<float> d(variance ? 0.5f : -range, variance ? 1.5f : range);
                float *v = p.second.data<float>();
                for (size_t i = 0; i < n; i++)
                    v[i] = d(rng);
            }
            net.copy_parameters_to_device();
            dp::ExecutionContext e = ctx.make_execution_context();
            std::uniform_real_distribution<float> d(-1.0f, 1.0f);
            for (unsigned i = 0; i < net.input_names().size(); i++) {
                std::vector<float> v(net.input(i).shape().total_size());
                for (float &f : v)
                    f = d(rng);
                net.set_input(i, v.data(), e);
            }
            if (graph)
                net.capture_forward(e);
            for (int i = 0; i < warmup; i++)
                net.forward(e, false);
            e.finish();
            auto t0 = std::chrono::steady_clock::now();
            for (int i = 0; i < iters; i++)
                net.forward(e, false);
            e.finish();
            const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / iters;
            const size_t batch = net.input(0).shape()[0];
            std::printf("operators %zu tensor_memory %zu ms_per_forward %.4f images_per_s %.1f\nok\n", net.operators_run(), net.tensor_memory(), ms,
                        batch * 1000.0 / ms);
            return 0;
        }
        if (cmd != "run" || argc < 6)
            return usage();
        dp::Context ctx(dp::Context::hip, 0, 0);
        dp::Net net(ctx);
        net.keep_intermediate_tensors(keep);
        net.fuse(fuse);
        net.prepack(prepack);
            net.channels_last(!nchw);
            net.fuse_max_pooling(!poolop);
        net.storage_type(bf16 ? dp::bfloat16_data : dp::float_data);
        net.mode(dp::CalculationsMode::predict);
        net.load_from_json_file(argv[2]);
        net.setup();
        net.load_parameters(argv[3]);
        if (!resave.empty())
            net.save_parameters(resave);
        dp::ExecutionContext e = ctx.make_execution_context();
        if (batch > 0) { // run on fewer images than the network file says: Net::reshape
            for (unsigned i = 0; i < net.input_names().size(); i++) {
                dp::Shape s = net.input(i).shape();
                s[0] = size_t(batch);
                net.input(i).reshape(s);
            }
            net.reshape();
        }
        std::ifstream in(argv[4], std::ios::binary);
        if (!in)
            throw dp::ValidationError(std::string("cannot open ") + argv[4]);
        std::vector<std::vector<float>> inputs(net.input_names().size());
        for (unsigned i = 0; i < inputs.size(); i++) {
            inputs[i].resize(net.input(i).shape().total_size());
            in.read(reinterpret_cast<char *>(inputs[i].data()), (std::streamsize)(inputs[i].size() * sizeof(float)));
            if (!in)
                throw dp::ValidationError("input file is too short");
            net.set_input(i, inputs[i].data(), e);
        }
        std::vector<std::vector<float>> eager_out;
        if (graph) {
            // the eager result first; then the recording, made with other input values than the ones that count
            // (a replay must read the tensors anew); every replay below must reproduce the eager result bit for bit
            net.forward(e, true);
            eager_out.resize(net.output_names().size());
            for (unsigned i = 0; i < eager_out.size(); i++) {
                eager_out[i].resize(net.output(i).shape().total_size());
                net.get_output(i, eager_out[i].data(), e);
            }
            std::vector<float> other(inputs[0].size(), 0.25f);
            net.set_input(0, other.data(), e);
            net.capture_forward(e);
        }
        for (int r = 0; r < repeat; r++) { // later passes must give what the first one gave: shared chunks are rewritten
            if (graph)
                net.set_input(0, inputs[0].data(), e); // eager work between the replays
            net.forward(e, true);
            for (unsigned i = 0; graph && i < eager_out.size(); i++) {
                std::vector<float> v(eager_out[i].size());
                net.get_output(i, v.data(), e);
                if (std::memcmp(v.data(), eager_out[i].data(), v.size() * sizeof(float)) != 0)
                    throw dp::ValidationError("graph replay " + std::to_string(r) + " differs from the eager pass in output " + std::to_string(i));
            }
        }
        std::ofstream out(argv[5], std::ios::binary);
        for (unsigned i = 0; i < net.output_names().size(); i++) {
            std::vector<float> v(net.output(i).shape().total_size());
            net.get_output(i, v.data(), e);
            out.write(reinterpret_cast<char *>(v.data()), (std::streamsize)(v.size() * sizeof(float)));
        }
        std::printf("operators %zu tensor_memory %zu\nok\n", net.operators_run(), net.tensor_memory());
        return 0;
    } catch (std::exception const &ex) {
        std::fprintf(stderr, "error: %s\n", ex.what());
        return 1;
    }
}
