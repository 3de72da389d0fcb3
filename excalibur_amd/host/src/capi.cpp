// C ABI over pipeline<float> / pipeline<unsigned short> (include/excalibur_capi.h).
#include "../../../include/excalibur_capi.h"

#include <cstring>
#include <sstream>

#include "../include/Excalibur/operation_reflector.hpp"
#include "../include/Excalibur/pipeline.hpp"

using glasssix::excalibur::pipeline;
using glasssix::memory::tensor;

struct exc_pipeline {
    int dtype = 0, device = 0;
    int slot = glasssix::memory::stream_slot();  // the pipeline's stream slot: the input tensor lives there too
    std::unique_ptr<pipeline<float>> f32;
    std::unique_ptr<pipeline<unsigned short>> f16;
    std::shared_ptr<tensor<float>> in32;
    std::shared_ptr<tensor<unsigned short>> in16;
    pipeline<float>::blob_map out32;
    pipeline<unsigned short>::blob_map out16;
    std::vector<pipeline<float>::blob_map> kept32;  // results of earlier forwards held on purpose (exc_pipeline_run_keeping)
    std::vector<pipeline<unsigned short>::blob_map> kept16;
};

namespace {
std::vector<std::string> split_lines(const char* text) {
    std::vector<std::string> lines;
    std::istringstream in{std::string(text)};
    std::string line;
    while (std::getline(in, line)) lines.push_back(line);
    return lines;
}

template <typename T>
void set_input(std::shared_ptr<tensor<T>>& slot, int device, const void* data, const int* shape) {
    const std::vector<int> s{shape[0], shape[1], shape[2], shape[3]};
    if (!slot || slot->data_shape() != s) slot = std::make_shared<tensor<T>>(s, device, glasssix::memory::NCHW);
    std::memcpy(slot->mutable_cpu_data(), data, sizeof(T) * static_cast<size_t>(slot->count()));
    slot->gpu_data();  // upload now, so that timed runs start with the input resident in HBM
}

template <typename T, typename P, typename M>
long get_blob(P& pipe, M& outs, const char* name, void* out, long capacity, int* shape) {
    std::shared_ptr<tensor<T>> t;
    auto it = outs.find(name);
    t = it != outs.end() ? it->second : pipe.get_featmap(name);
    if (!t) return -1;
    const std::vector<int> s = t->data_shape();
    for (int i = 0; i < 4; ++i) shape[i] = s[i];
    const long n = t->count();
    if (out && n <= capacity) std::memcpy(out, t->cpu_data(), sizeof(T) * static_cast<size_t>(n));
    return n;
}
}  // namespace

extern "C" exc_pipeline* exc_pipeline_create(const char* topology, const char* model_path, int device, int dtype) {
    auto* p = new exc_pipeline();
    p->dtype = dtype;
    p->device = device;
    const std::vector<std::string> lines = split_lines(topology);
    const std::string model(model_path ? model_path : "");
    if (dtype == 0) p->f32.reset(new pipeline<float>(lines, model, device));
    else p->f16.reset(new pipeline<unsigned short>(lines, model, device));
    return p;
}

extern "C" exc_pipeline* exc_pipeline_create_from_files(const char* param_file, const char* model_file, int device, int dtype) {
    auto* p = new exc_pipeline();
    p->dtype = dtype;
    p->device = device;
    const bool dummy = !model_file || !*model_file;
    if (dtype == 0) p->f32.reset(dummy ? new pipeline<float>(param_file, device) : new pipeline<float>(param_file, model_file, device));
    else p->f16.reset(dummy ? new pipeline<unsigned short>(param_file, device) : new pipeline<unsigned short>(param_file, model_file, device));
    return p;
}

extern "C" void exc_pipeline_destroy(exc_pipeline* p) { delete p; }

extern "C" void exc_pipeline_set_fusion(exc_pipeline* p, int on) {
    if (p->f32) p->f32->set_fusion(on != 0);
    if (p->f16) p->f16->set_fusion(on != 0);
}

extern "C" int exc_set_option(const char* name, int value) {
    if (name && !std::strcmp(name, "f16_nchw_only")) {
        glasssix::excalibur::set_f16_nchw_only(value != 0);
        return 0;
    }
    return exhip_set_option(name, value);
}

extern "C" int exc_pipeline_blob_stored(exc_pipeline* p, const char* name) {
    return p->f32 ? p->f32->blob_stored(name) : p->f16 ? p->f16->blob_stored(name) : 0;
}

extern "C" void exc_pipeline_set_graphs(exc_pipeline* p, int on) {
    if (p->f32) p->f32->set_graphs(on != 0);
}

extern "C" int exc_pipeline_last_fused(exc_pipeline* p) { return p->f32 ? p->f32->fused() : 0; }

extern "C" void exc_pipeline_time_fused_span(exc_pipeline* p, int first_launch) {
    if (p->f32) p->f32->time_fused_span(first_launch);
}

extern "C" float exc_pipeline_last_span(exc_pipeline* p, int* launches) {
    if (launches) *launches = 0;
    return p->f32 ? p->f32->last_span(launches) : 0.f;
}

extern "C" int exc_pipeline_recent_spans(exc_pipeline* p, float* ms, int capacity) {
    return p->f32 ? p->f32->recent_spans(ms, capacity) : 0;
}

extern "C" int exc_pipeline_set_input(exc_pipeline* p, const void* input, const int shape[4]) {
    glasssix::memory::stream_scope scope(p->slot);  // the input's device block belongs to the pipeline's slot
    if (p->dtype == 0) set_input(p->in32, p->device, input, shape);
    else set_input(p->in16, p->device, input, shape);
    return 0;
}

extern "C" int exc_pipeline_run(exc_pipeline* p) {
    // the previous results are released first: a result still held when a forward starts stays its holder's, and the
    // pipeline would write into newly allocated tensors
    if (p->dtype == 0) {
        p->out32.clear();
        p->out32 = p->f32->forward(p->in32);
    } else {
        p->out16.clear();
        p->out16 = p->f16->forward(p->in16);
    }
    return 0;
}

extern "C" int exc_pipeline_run_keeping(exc_pipeline* p) {
    if (p->dtype == 0) {
        p->kept32.push_back(std::move(p->out32));
        p->out32 = p->f32->forward(p->in32);
    } else {
        p->kept16.push_back(std::move(p->out16));
        p->out16 = p->f16->forward(p->in16);
    }
    return 0;
}

extern "C" long exc_pipeline_get_kept(exc_pipeline* p, int back, const char* name, void* out, long capacity, int shape[4]) {
    std::shared_ptr<tensor<float>> t32;
    std::shared_ptr<tensor<unsigned short>> t16;
    if (back < 1) return -1;
    if (p->dtype == 0) {
        if (static_cast<size_t>(back) > p->kept32.size()) return -1;
        auto& m = p->kept32[p->kept32.size() - back];
        auto it = m.find(name);
        if (it == m.end()) return -1;
        t32 = it->second;
    } else {
        if (static_cast<size_t>(back) > p->kept16.size()) return -1;
        auto& m = p->kept16[p->kept16.size() - back];
        auto it = m.find(name);
        if (it == m.end()) return -1;
        t16 = it->second;
    }
    const std::vector<int> s = t32 ? t32->data_shape() : t16->data_shape();
    for (int i = 0; i < 4; ++i) shape[i] = s[i];
    const long n = t32 ? t32->count() : t16->count();
    if (out && n <= capacity) {
        if (t32) std::memcpy(out, t32->cpu_data(), sizeof(float) * static_cast<size_t>(n));
        else std::memcpy(out, t16->cpu_data(), sizeof(unsigned short) * static_cast<size_t>(n));
    }
    return n;
}

extern "C" int exc_pipeline_sync(exc_pipeline* p) { return exhip_sync(glasssix::memory::device_context(p->device, p->slot)); }

extern "C" int exc_set_stream_slot(int slot) {
    if (slot < 0 || slot >= glasssix::memory::kMaxStreamSlots) return -1;
    glasssix::memory::set_stream_slot(slot);
    return 0;
}

extern "C" int exc_pipeline_stream_slot(exc_pipeline* p) { return p->slot; }

extern "C" int exc_pipeline_forward(exc_pipeline* p, const void* input, const int shape[4]) {
    exc_pipeline_set_input(p, input, shape);
    exc_pipeline_run(p);
    return exc_pipeline_sync(p);
}

extern "C" long exc_pipeline_get(exc_pipeline* p, const char* name, void* out, long capacity, int shape[4]) {
    if (p->dtype == 0) return get_blob<float>(*p->f32, p->out32, name, out, capacity, shape);
    return get_blob<unsigned short>(*p->f16, p->out16, name, out, capacity, shape);
}

extern "C" size_t exc_registered_operations(int dtype, char* buf, size_t len) {
    std::string all;
    const std::vector<std::string> names = dtype == 0   ? glasssix::excalibur::operation_reflector<float>::instance().registered()
                                           : dtype == 1 ? glasssix::excalibur::operation_reflector<unsigned short>::instance().registered()
                                                        : glasssix::excalibur::operation_reflector<double>::instance().registered();
    for (const std::string& n : names) all += n + "\n";
    if (buf && len) {
        std::strncpy(buf, all.c_str(), len - 1);
        buf[len - 1] = 0;
    }
    return all.size() + 1;
}
