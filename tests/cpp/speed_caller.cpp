// A C++ application written against the mirrored public header only, shaped like the reference's own harness
// (src/SpeedBenchmark/speedbenchmark.cpp:33-106): file-path constructor, 5 warm-up + N timed forward() calls with
// min / max / average, then a blob by name. It writes that blob's bytes to a file so that the test can compare them with
// what the C wrapper (include/excalibur_capi.h) returns for the same input.
//   speed_caller <topology.phai> <model.racy> <n> <c> <h> <w> <input.bin> <blob name> <output.bin> [timed forwards]
#include <cfloat>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "Excalibur/pipeline.hpp"

using namespace glasssix;

int main(int argc, char** argv) {
    if (argc < 10) {
        std::cerr << "usage: speed_caller topology model n c h w input.bin blob output.bin [forwards]\n";
        return 2;
    }
    const std::vector<int> shape = {std::atoi(argv[3]), std::atoi(argv[4]), std::atoi(argv[5]), std::atoi(argv[6])};
    const int loop_count = argc > 10 ? std::atoi(argv[10]) : 100, warmup_loop_count = 5;

    const std::string topology_file = argv[1], model_file = argv[2];
    excalibur::pipeline<float> pipe(topology_file, model_file, 0);

    std::shared_ptr<memory::tensor<float>> input_tensor(new memory::tensor<float>(shape, 0, memory::NCHW));
    {
        std::ifstream in(argv[7], std::ios::binary);
        in.read(reinterpret_cast<char*>(input_tensor->mutable_cpu_data()), sizeof(float) * input_tensor->count());
        if (!in) {
            std::cerr << "speed_caller: short input file\n";
            return 2;
        }
    }
    for (int j = 0; j < warmup_loop_count; j++) pipe.forward(input_tensor);
    pipe.synchronize();

    double time_min = DBL_MAX, time_max = -DBL_MAX, time_avg = 0;
    for (int j = 0; j < loop_count; j++) {
        const auto t0 = std::chrono::steady_clock::now();
        auto results = pipe.forward(input_tensor);
        pipe.synchronize();  // forward() returns when the work is queued: the reference's call is synchronous
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        time_min = std::min(time_min, ms);
        time_max = std::max(time_max, ms);
        time_avg += ms;
    }
    time_avg /= loop_count;
    std::cout << "Pipeline\t Min\t Max\t Ave " << std::endl;
    std::cout << argv[1] << "\t" << time_min << "\t" << time_max << "\t" << time_avg << std::endl;

    auto blob = pipe.get_featmap(argv[8]);
    if (!blob) {
        std::cerr << "speed_caller: no blob named " << argv[8] << "\n";
        return 3;
    }
    std::ofstream out(argv[9], std::ios::binary);
    const std::vector<int> s = blob->data_shape();
    std::cout << "blob " << argv[8] << " " << s[0] << "x" << s[1] << "x" << s[2] << "x" << s[3] << std::endl;
    out.write(reinterpret_cast<const char*>(blob->cpu_data()), sizeof(float) * blob->count());
    return out ? 0 : 4;
}
