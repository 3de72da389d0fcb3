// C-ABI shim over the reference's public CPU API, for the checker only.
//
// This file is this repository's own code. It is compiled together with the
// reference's sources (where they lie, see the Makefile) into
// oracle/_ref/libexcalibur_ref.so and lets the Python tests and the
// cpu_baseline leg of bench.py drive single layers or whole topologies through
// glasssix::excalibur::pipeline<Dtype>(lines, model_file, -1)
// (reference include/Excalibur/pipeline.hpp:26) exactly as an application would.
// Nothing in the product library links or loads it.
//
// Errors inside the reference are LOG(FATAL) -> std::terminate
// (reference include/Primitives/logger.hpp:114-117); callers must pass
// topologies the reference accepts.

#include "Excalibur/pipeline.hpp"
#include "Primitives/tensor.hpp"

#include <chrono>
#include <cstring>
#include <memory>
#include <sstream>
#include <thread>
#include <string>
#include <unordered_map>
#include <vector>

using glasssix::excalibur::pipeline;
using glasssix::memory::tensor;

namespace {

template <typename T>
struct handle_t {
    std::unique_ptr<pipeline<T>> pipe;
    std::unordered_map<std::string, std::shared_ptr<tensor<T>>> outputs;
};

struct any_handle {
    int dtype;  // 0 float, 1 unsigned short (IEEE half bits)
    handle_t<float> f32;
    handle_t<unsigned short> f16;
};

std::vector<std::string> split_lines(const char* text) {
    std::vector<std::string> lines;
    std::istringstream in{std::string(text)};
    std::string line;
    while (std::getline(in, line)) lines.push_back(line);
    return lines;
}

template <typename T>
int forward_impl(handle_t<T>& h, const void* input, const int* shape) {
    std::vector<int> s{shape[0], shape[1], shape[2], shape[3]};
    auto t = std::make_shared<tensor<T>>(s, -1, glasssix::memory::NCHW);
    std::memcpy(t->mutable_cpu_data(), input, sizeof(T) * (size_t)t->count());
    h.outputs = h.pipe->forward(t);
    return 0;
}

template <typename T>
long get_impl(handle_t<T>& h, const char* name, void* out, long capacity, int* shape) {
    std::shared_ptr<tensor<T>> t;
    auto it = h.outputs.find(name);
    if (it != h.outputs.end()) t = it->second;
    else t = h.pipe->get_featmap(name);
    if (!t) return -1;
    auto s = t->data_shape();
    for (int i = 0; i < 4; ++i) shape[i] = i < (int)s.size() ? s[i] : 1;
    long n = t->count();
    if (out && n <= capacity) std::memcpy(out, t->cpu_data(), sizeof(T) * (size_t)n);
    return n;
}

}  // namespace

#define EXREF_API extern "C" __attribute__((visibility("default")))

// topology: the .phai text ('\n'-separated lines); model_path: a .racy file, or ""
// for the reference's dummy weights. dtype 0 = pipeline<float>, 1 = pipeline<unsigned short>.
EXREF_API void* exref_pipeline_create(const char* topology, const char* model_path, int dtype) {
    auto* h = new any_handle();
    h->dtype = dtype;
    auto lines = split_lines(topology);
    std::string model(model_path ? model_path : "");
    if (dtype == 0) h->f32.pipe.reset(new pipeline<float>(lines, model, -1));
    else h->f16.pipe.reset(new pipeline<unsigned short>(lines, model, -1));
    return h;
}

EXREF_API void exref_pipeline_destroy(void* p) { delete static_cast<any_handle*>(p); }

// input: dense NCHW, shape[4]; runs pipeline::forward on the CPU path.
EXREF_API int exref_pipeline_forward(void* p, const void* input, const int* shape) {
    auto* h = static_cast<any_handle*>(p);
    return h->dtype == 0 ? forward_impl(h->f32, input, shape) : forward_impl(h->f16, input, shape);
}

// Copies a named output (or any feature map) of the last forward into out when it
// fits in capacity elements; returns its element count and writes shape[4].
EXREF_API long exref_pipeline_get(void* p, const char* name, void* out, long capacity, int* shape) {
    auto* h = static_cast<any_handle*>(p);
    return h->dtype == 0 ? get_impl(h->f32, name, out, capacity, shape) : get_impl(h->f16, name, out, capacity, shape);
}

// Times `iters` forward calls after `warmup` untimed ones; returns seconds per call.
EXREF_API double exref_pipeline_time(void* p, const void* input, const int* shape, int warmup, int iters) {
    auto* h = static_cast<any_handle*>(p);
    for (int i = 0; i < warmup; ++i) exref_pipeline_forward(h, input, shape);
    auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) exref_pipeline_forward(h, input, shape);
    auto t1 = std::chrono::steady_clock::now();
    return std::chrono::duration<double>(t1 - t0).count() / (iters > 0 ? iters : 1);
}

// The batch-parallel form of the CPU baseline: `workers` threads, each with a pipeline of its own (an instance is
// single-threaded and keeps per-call state in its operators) and one image, run `iters` forwards after `warmup` untimed
// ones. Returns the wall-clock seconds of the timed part; images per second = workers * iters / that. The reference's own
// OpenMP use is off in this build and would be pinned to two threads (src/Excalibur/operation_convolution.cpp:436).
EXREF_API double exref_pipeline_time_parallel(const char* topology, const char* model_path, int dtype, const void* image,
                                              const int* shape, int workers, int warmup, int iters) {
    std::vector<void*> pipes;
    for (int w = 0; w < workers; ++w) pipes.push_back(exref_pipeline_create(topology, model_path, dtype));
    auto run = [&](int n) {
        std::vector<std::thread> threads;
        for (int w = 0; w < workers; ++w)
            threads.emplace_back([&, w]() {
                for (int i = 0; i < n; ++i) exref_pipeline_forward(pipes[w], image, shape);
            });
        for (auto& t : threads) t.join();
    };
    run(warmup);
    auto t0 = std::chrono::steady_clock::now();
    run(iters);
    auto t1 = std::chrono::steady_clock::now();
    for (void* p : pipes) exref_pipeline_destroy(p);
    return std::chrono::duration<double>(t1 - t0).count();
}
