// The reference's public entry point (include/Excalibur/pipeline.hpp:17-47): a pipeline is built from a
// `.phai` topology (file or lines) and a `.racy` model file (or dummy weights), and forward() returns the
// output blobs by name. device >= 0 selects this MI355X backend; device < 0 is fatal here (no CPU path).
#pragma once
#include <memory>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

#include "../Primitives/tensor.hpp"

namespace glasssix {
namespace excalibur {

template <typename Dtype>
class pipeline {
public:
    class impl;
    using blob_map = std::unordered_map<std::string, std::shared_ptr<memory::tensor<Dtype>>>;

    explicit pipeline();
    explicit pipeline(std::string_view param_file, std::string_view model_file, int device = -1);
    explicit pipeline(std::string_view param_file, int device = -1);
    explicit pipeline(const std::vector<std::string>& hardcode_params, std::string_view model_file, int device = -1);
    ~pipeline();

    blob_map forward(const std::shared_ptr<memory::tensor<Dtype>>& input_tensor);
    blob_map forward_cpu(const std::shared_ptr<memory::tensor<Dtype>>& input_tensor);
    blob_map forward_gpu(const std::shared_ptr<memory::tensor<Dtype>>& input_tensor);
    std::shared_ptr<memory::tensor<Dtype>> get_featmap(std::string_view featmap_name);

    void enable_profiler();   // per-layer HIP-event timings printed after each forward
    void disable_profiler();

    // Backend switch without a counterpart in the reference: run int8 convolution chains with fused
    // epilogues and int8 NHWC tensors between layers, let convolutions absorb the activation / sum layer
    // behind them (default on). A forward then stores only some blobs as float tensors; get_featmap() of
    // another blob runs the last input once more layer by layer. blob_stored() tells the two apart.
    void set_fusion(bool on);
    bool blob_stored(std::string_view featmap_name) const;
    // on: a fused int8 plan replays its launches (all but the input quantizer) as one HIP graph from its second
    // forward on; off (default: the replay measured no faster than the calls): one call per launch.
    void set_graphs(bool on);
    bool fused() const;
    double last_forward_ms() const;
    // Device time of part of a fused forward: with first_launch >= 0 every fused forward records one event in front
    // of its launch number first_launch (0 is the input quantizer, unless the stem kernel quantizes its own input; -2 stands
    // for the first convolution's launch, whichever number it has) and one behind its last launch;
    // last_span(&launches) waits for them and returns the milliseconds between the two and the launches in between.
    // The event pairs come from a ring of 32: recent_spans(ms, capacity) waits for the device and fills in the spans of
    // the latest forwards since time_fused_span was called (oldest first, at most 32 and at most capacity), so that
    // forwards queued back to back are read without a synchronisation between them; it returns how many it wrote.
    void time_fused_span(int first_launch);
    float last_span(int* launches);
    int recent_spans(float* ms, int capacity);

    // Stream slots (no counterpart in the reference, whose pipelines are synchronous): a pipeline does its device work on
    // the HIP stream of the slot its constructing thread was in (memory::set_stream_slot; 0 unless set), so pipelines made
    // in different slots may have forwards in flight at the same time. forward() returns when the work is queued;
    // reading a result (cpu_data) or synchronize() waits for it.
    int stream_slot() const;
    void synchronize();

    static std::string version();

private:
    impl* impl_;
    pipeline(const pipeline&) = delete;
    pipeline& operator=(const pipeline&) = delete;
};

}  // namespace excalibur
}  // namespace glasssix
