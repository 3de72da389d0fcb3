// pipeline: `.phai` topology parsing, operator creation through the registry, `.racy` weight loading and the two
// executors of this backend. Parsing and bookkeeping follow the reference (src/Excalibur/pipeline.cpp:35-194,
// 218-232, 406-451): line 0 is the magic and optional name, line 1 is ignored, every further line is
// "<Type> <name> <n_in> <n_out> <inputs...> <outputs...> <key=value...>"; a layer with n_in == 0 gets the input
// "<name>_input"; blobs nobody produces are pipeline inputs (the first one is fed), blobs nobody consumes are
// outputs; layers run in file order.
//
// Executors:
//  * per-layer: every operator's forward_gpu on float (or half) NCHW blobs, exactly the reference's contract;
//  * fused (pipeline<float>, int8 networks made of Convolution / max Pooling / Split / BinaryOp add / ReLU):
//    int8 NHWC tensors between layers, each convolution's epilogue doing dequantization + bias + activation
//    (+ shortcut add + ReLU) and writing what its consumers read. Same values as the per-layer executor.
#include "../include/Excalibur/pipeline.hpp"

#include <array>
#include <type_traits>
#include <chrono>
#include <cmath>
#include <cstring>
#include <deque>
#include <fstream>
#include <functional>
#include <map>
#include <set>

#include "../include/Excalibur/operation_reflector.hpp"
#include "../include/Excalibur/operators.hpp"

namespace glasssix {
namespace excalibur {

using memory::tensor;

namespace {
inline int pad_to(int v, int m) { return (v + m - 1) / m * m; }

struct dev_buffer {  // device allocation owned by a fused plan
    int device = -1;
    void* ptr = nullptr;
    size_t bytes = 0;
    dev_buffer() {}
    dev_buffer(int dev, size_t n) : device(dev), ptr(memory::device_alloc(dev, n)), bytes(n) {}
    dev_buffer(dev_buffer&& o) noexcept : device(o.device), ptr(o.ptr), bytes(o.bytes) { o.ptr = nullptr; }
    dev_buffer& operator=(dev_buffer&& o) noexcept {
        release();
        device = o.device; ptr = o.ptr; bytes = o.bytes; o.ptr = nullptr;
        return *this;
    }
    ~dev_buffer() { release(); }
    void release() {
        if (ptr) memory::device_release(device, ptr, bytes);
        ptr = nullptr;
    }
    dev_buffer(const dev_buffer&) = delete;
    dev_buffer& operator=(const dev_buffer&) = delete;
};
}  // namespace

template <typename Dtype>
class pipeline<Dtype>::impl {
public:
    using tensor_ptr = std::shared_ptr<tensor<Dtype>>;

    impl() : device_(-1) {}  // the reference's default-constructed pipeline (pipeline.cpp:575-577): no layers; forward is fatal

    // the plan lets go of the operators' packed weights: it goes first, while the operators still exist
    ~impl() {
        plan_.reset();
        for (auto& pair : span_ev_)
            for (void* ev : pair)
                if (ev) exhip_event_destroy(ev);
    }

    impl(const std::vector<std::string>& lines, std::string_view model_file, int device) : device_(device) {
        if (device >= 0) memory::device_context(device);  // opens the device, fatal if it is not an MI355X
        if (lines.empty()) LOG(FATAL) << "Incorrect param file.";
        const std::vector<std::string> head = split_string(lines[0], " ");
        if (head.empty() || (head[0] != "glsv1" && head[0] != "7767517")) LOG(FATAL) << "Incorrect param file version.";
        if (head.size() > 1) name_ = head[1];
        for (size_t i = 2; i < lines.size(); ++i) {
            std::vector<std::string> tok;
            for (const std::string& t : split_string(lines[i], " "))
                if (!t.empty() && t != "\r") tok.push_back(t);
            if (tok.empty()) continue;
            if (tok.size() < 4) LOG(FATAL) << "Incorrect layer line: " << lines[i];
            operation_param p;
            p.type_ = tok[0];
            p.name_ = tok[1];
            p.device_ = device_;
            p.input_count_ = std::atoi(tok[2].c_str());
            p.output_count_ = std::atoi(tok[3].c_str());
            const size_t n_in = static_cast<size_t>(std::max(p.input_count_, 0)), n_out = static_cast<size_t>(std::max(p.output_count_, 0));
            if (tok.size() < 4 + n_in + n_out) LOG(FATAL) << "Incorrect layer line: " << lines[i];
            for (size_t j = 0; j < n_out; ++j) p.output_featmaps_.push_back(tok[4 + n_in + j]);
            for (size_t j = 4 + n_in + n_out; j < tok.size(); ++j) p.specific_params_ += tok[j] + " ";
            if (p.input_count_ <= 0) {
                p.input_count_ = 1;
                p.input_featmaps_ = {p.name_ + "_input"};
            } else {
                for (size_t j = 0; j < n_in; ++j) p.input_featmaps_.push_back(tok[4 + j]);
            }
            op_params_.push_back(p);
        }
        for (const operation_param& p : op_params_) operations_.push_back(operation_reflector<Dtype>::instance().create_object(p));

        if (model_file.empty()) {
            LOG(WARNING) << "THIS PIPELINE IS LOADED WITH DUMMY DATA.";
            for (auto& op : operations_) weights_mem_cost_ += op->init_weights();
        } else {
            const std::string path(model_file);
            FILE* fp = std::fopen(path.c_str(), "rb");
            if (!fp) LOG(FATAL) << "Cannot open " << path;
            for (auto& op : operations_) weights_mem_cost_ += op->init_weights(fp);
            CHECK_EQ(std::fclose(fp), 0) << "Cannot close " << path;
        }

        // blob table, producers, consumers
        std::map<std::string, int> produced_by;
        for (size_t i = 0; i < op_params_.size(); ++i)
            for (const std::string& o : op_params_[i].output_featmaps_) produced_by[o] = static_cast<int>(i);
        std::set<std::string> consumed;
        auto blob_id = [&](const std::string& name) {
            auto it = blob_index_.find(name);
            if (it != blob_index_.end()) return it->second;
            const int id = static_cast<int>(blob_index_.size());
            blob_index_[name] = id;
            blob_names_.push_back(name);
            return id;
        };
        for (size_t i = 0; i < op_params_.size(); ++i) {
            std::vector<int> in, out;
            for (const std::string& b : op_params_[i].input_featmaps_) {
                in.push_back(blob_id(b));
                consumed.insert(b);
                if (!produced_by.count(b) && std::find(input_names_.begin(), input_names_.end(), b) == input_names_.end())
                    input_names_.push_back(b);
            }
            for (const std::string& b : op_params_[i].output_featmaps_) out.push_back(blob_id(b));
            op_inputs_.push_back(in);
            op_outputs_.push_back(out);
        }
        for (size_t i = 0; i < op_params_.size(); ++i)
            for (const std::string& b : op_params_[i].output_featmaps_)
                if (!consumed.count(b)) output_names_.push_back(b);
        if (input_names_.empty()) LOG(FATAL) << "the topology has no input blob";
        featmaps_.resize(blob_names_.size());
        find_activation_pairs();
    }

    // A convolution whose only reader is the activation layer on the next line runs that layer in its epilogue: the
    // values are the ones the two layers produce one after the other, and the blob between them is never stored. The
    // pair qualifies when the activation writes over its input (the blob name is reused) or when nothing else reads
    // the convolution's blob and it is not a result of the network.
    void find_activation_pairs() {
        pair_.assign(operations_.size(), post_activation{});
        std::vector<int> readers(blob_names_.size(), 0);
        for (const auto& in : op_inputs_)
            for (int b : in) ++readers[b];
        for (size_t i = 0; i + 1 < operations_.size(); ++i) {
            auto* conv = dynamic_cast<operation_convolution<Dtype>*>(operations_[i].get());
            if (!conv || op_outputs_[i].size() != 1 || op_inputs_[i + 1].size() != 1 || op_outputs_[i + 1].size() != 1) continue;
            const int mid = op_outputs_[i][0];
            if (op_inputs_[i + 1][0] != mid) continue;
            post_activation pa;
            if (auto* u = dynamic_cast<operation_unary<Dtype>*>(operations_[i + 1].get())) {
                pa.post_op = 1 + u->op_; pa.alpha = u->alpha_; pa.beta = u->beta_;
            } else if (dynamic_cast<operation_relu<Dtype>*>(operations_[i + 1].get())) {
                pa.relu = true;
            } else if (auto* pr = dynamic_cast<operation_prelu<Dtype>*>(operations_[i + 1].get())) {
                if (!pr->share_channel_ && pr->num_slope_ != conv->output_channel_) continue;
                pa.prelu = pr;
            } else {
                continue;
            }
            const bool in_place = op_outputs_[i + 1][0] == mid;
            const bool is_result = std::find(output_names_.begin(), output_names_.end(), blob_names_[mid]) != output_names_.end();
            if (!in_place && (readers[mid] != 1 || is_result)) continue;
            static const float probe = 0.f;  // any non-null address: asks whether the layer can, sets nothing up for a launch
            if (!(pa.prelu ? conv->set_post_prelu(&probe, true) : conv->set_post_activation(pa.post_op, pa.alpha, pa.beta, pa.relu))) continue;
            conv->clear_post();
            pa.on = true;
            pair_[i] = pa;
        }
        find_quantized_links();
        find_sum_pairs();
        find_glue_chains();
    }

    // fp16 pipeline: a convolution whose only reader is the two-input sum on the next line (Eltwise SUM with unit
    // coefficients, BinaryOp ADD of two blobs: the residual add of a bottleneck block) adds the other operand in its
    // epilogue, to its own result rounded to half as the sum layer would read it. Whether it can is known only when the
    // blobs are there (both NHWC, same shape), so the convolution reports it and the sum layer runs if it could not.
    // The sum may also stand behind the activation layer that already runs in the convolution's epilogue (convolution ->
    // HardSwish -> add, the bottleneck of the detection topologies): the epilogue then adds behind the activation.
    void find_sum_pairs() {
        sum_other_.assign(operations_.size(), -1);
        if constexpr (std::is_same_v<Dtype, unsigned short>) {
            std::vector<int> readers(blob_names_.size(), 0);
            for (const auto& in : op_inputs_)
                for (int b : in) ++readers[b];
            for (size_t i = 0; i + 1 < operations_.size(); ++i) {
                auto* conv = dynamic_cast<operation_convolution<Dtype>*>(operations_[i].get());
                if (!conv || dynamic_cast<operation_convolutiondepthwise<Dtype>*>(conv)) continue;
                // the layer whose top the sum reads: the convolution, or the activation layer that runs in its epilogue
                const size_t last = pair_[i].on ? i + 1 : i;
                if (last + 1 >= operations_.size()) continue;
                if (op_outputs_[last].size() != 1 || op_inputs_[last + 1].size() != 2 || op_outputs_[last + 1].size() != 1) continue;
                const int mid = op_outputs_[last][0];
                const int a = op_inputs_[last + 1][0], b = op_inputs_[last + 1][1];
                if ((a == mid) == (b == mid)) continue;  // exactly one operand is the blob
                bool plain_sum = false;
                if (auto* e = dynamic_cast<operation_eltwise<Dtype>*>(operations_[last + 1].get()))
                    plain_sum = e->type_ == 1 && e->coeffs_.size() == 2 && e->coeffs_[0] == 1.f && e->coeffs_[1] == 1.f;
                else if (auto* bo = dynamic_cast<operation_binaryop<Dtype>*>(operations_[last + 1].get()))
                    plain_sum = bo->op_type_ == 0 && !bo->with_scalar_;
                // an activation writing over its input reads the blob as well
                const int own_readers = pair_[i].on && op_outputs_[i][0] == mid ? 2 : 1;
                if (!plain_sum || readers[mid] != own_readers || op_outputs_[last + 1][0] == mid) continue;
                if (std::find(output_names_.begin(), output_names_.end(), blob_names_[mid]) != output_names_.end()) continue;
                sum_other_[i] = a == mid ? b : a;
            }
        }
    }

    // fp16 pipeline: a Concat whose only reader is the BatchNorm layer on the next line, and a BatchNorm (behind a Concat or
    // not) whose only reader is the activation layer on the next line, run those layers in their own kernel: the blobs
    // between them are never stored. Whether the kernel takes the NHWC path is known when the blobs are there, so the
    // layer reports it and the absorbed layers run if it could not.
    void find_glue_chains() {
        chain_.assign(operations_.size(), glue_chain{});
        if constexpr (std::is_same_v<Dtype, unsigned short>) {
            std::vector<int> readers(blob_names_.size(), 0);
            for (const auto& in : op_inputs_)
                for (int b : in) ++readers[b];
            // layer j (one input, one output) is the only reader of layer i's blob, which nobody asks for by name
            auto follows = [&](size_t i, size_t j) {
                if (j >= operations_.size() || op_outputs_[i].size() != 1 || op_inputs_[j].size() != 1 || op_outputs_[j].size() != 1) return false;
                const int mid = op_outputs_[i][0];
                if (op_inputs_[j][0] != mid) return false;
                const bool in_place = op_outputs_[j][0] == mid;
                const bool is_result = std::find(output_names_.begin(), output_names_.end(), blob_names_[mid]) != output_names_.end();
                return in_place || (readers[mid] == 1 && !is_result);
            };
            auto activation = [&](size_t j) -> operation_unary<Dtype>* {
                auto* u = j < operations_.size() ? dynamic_cast<operation_unary<Dtype>*>(operations_[j].get()) : nullptr;
                return u && u->op_ != EXHIP_UNARY_SIGMOID ? u : nullptr;
            };
            for (size_t i = 0; i + 1 < operations_.size(); ++i) {
                glue_chain g;
                size_t last = i;
                if (dynamic_cast<operation_concat<Dtype>*>(operations_[i].get())) {
                    if (!follows(i, i + 1)) continue;
                    if (dynamic_cast<operation_batchnorm<Dtype>*>(operations_[i + 1].get())) {
                        g.bn = static_cast<int>(i + 1);
                        last = i + 1;
                    }
                } else if (!dynamic_cast<operation_batchnorm<Dtype>*>(operations_[i].get())) {
                    continue;
                }
                if (follows(last, last + 1) && activation(last + 1)) {
                    g.unary = static_cast<int>(last + 1);
                    last = last + 1;
                }
                if (last == i) continue;
                g.last = static_cast<int>(last);
                chain_[i] = g;
                i = last;  // the absorbed layers start no chain of their own
            }
        }
    }

    // An int8 convolution whose result is read by int8 convolutions writes the int8 NHWC tensor those readers would
    // make of it (their feature-map scale, their channel stride) from its epilogue, and they skip their quantizer:
    // q8(v * fs) of the value the layer stores is what the reader's quantizer computes from the stored value. Readers
    // are found through Split layers (their tops are the bottom itself) and behind the activation layer paired with the
    // convolution; if every reader is such a convolution and the blob is no result of the network, the float tensor
    // is not written at all.
    void find_quantized_links() {
        link_.assign(operations_.size(), quantized_link{});
        for (size_t i = 0; i < operations_.size(); ++i) {
            auto* conv = dynamic_cast<operation_convolution<Dtype>*>(operations_[i].get());
            if (!conv || op_outputs_[i].size() != 1 || !conv->set_quantized_output(1.f, 1 << 20, false)) continue;
            conv->set_quantized_output(0.f, 0, false);
            const size_t last = pair_[i].on ? i + 1 : i;  // the layer whose top the readers see
            std::vector<int> names{op_outputs_[last][0]};
            quantized_link lk;
            bool float_reader = false;
            for (size_t b = 0; b < names.size(); ++b) {
                if (std::find(output_names_.begin(), output_names_.end(), blob_names_[names[b]]) != output_names_.end()) float_reader = true;
                for (size_t j = 0; j < operations_.size(); ++j) {
                    if (j == last && pair_[i].on) continue;  // the paired activation writing over its input
                    if (std::find(op_inputs_[j].begin(), op_inputs_[j].end(), names[b]) == op_inputs_[j].end()) continue;
                    if (j <= last) { float_reader = true; continue; }  // a reused name: not this layer's blob, stay safe
                    if (dynamic_cast<operation_split<Dtype>*>(operations_[j].get())) {
                        for (int t : op_outputs_[j])
                            if (std::find(names.begin(), names.end(), t) == names.end()) names.push_back(t);
                        continue;
                    }
                    float fs = 0.f;
                    int stride = 0;
                    if (auto* reader = dynamic_cast<operation_convolution<Dtype>*>(operations_[j].get())) reader->quantized_input(&fs, &stride);
                    if (fs == 0.f || stride % 32 != 0) { float_reader = true; continue; }
                    if (!lk.on) { lk.on = true; lk.fs = fs; lk.stride = stride; }
                    else if (lk.fs != fs || lk.stride != stride) float_reader = true;  // that reader runs its quantizer
                }
            }
            if (!lk.on || !conv->set_quantized_output(lk.fs, lk.stride, false)) continue;
            conv->set_quantized_output(0.f, 0, false);
            lk.only = !float_reader;
            link_[i] = lk;
        }
    }

    blob_map forward(const tensor_ptr& input) {
        if (device_ >= 0) return forward_gpu(input);
        return forward_cpu(input);
    }

    blob_map forward_cpu(const tensor_ptr&) {
        NO_CPU;
        return {};
    }

    blob_map forward_gpu(const tensor_ptr& input) {
        if (device_ < 0) LOG(FATAL) << "forward_gpu on a pipeline created with device < 0";
        const auto t0 = std::chrono::steady_clock::now();
        blob_map results;
        if (!try_fused(input, &results)) results = forward_layers(input);
        if (profile_) {
            exhip_sync(memory::device_context(device_));
            last_ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            LOG(INFO) << name_ << ": forward " << last_ms_ << " ms (" << (last_fused_ ? "fused int8 plan" : "per-layer") << ")";
        }
        return results;
    }

    // A blob of the last forward by name, NCHW (nullptr for an unknown name, as in the reference). The fused executors
    // do not store every blob (a fused plan keeps int8 tensors between layers, a convolution absorbs the activation or
    // sum behind it, int8 readers get an int8 form only): asking for such a blob runs the last input once more through the
    // per-layer executor with fusion off, which stores them all, so what comes back always belongs to the last input. If the
    // caller has written to the input tensor since that forward, the rerun would mix two inputs' blobs: the request is
    // refused (nullptr and an error line) until the next forward.
    tensor_ptr get_featmap(std::string_view name) {
        auto it = blob_index_.find(std::string(name));
        if (it == blob_index_.end()) return nullptr;
        auto missing = [&]() {
            const tensor_ptr& t = featmaps_[it->second];
            return !t || (t->quantized && t->quantized->only);
        };
        if (missing() && last_input_ && !all_blobs_stored_ && last_input_->writes() != last_input_writes_) {
            LOG(ERROR) << name_ << ": blob " << name << " was not stored by the last forward and the input tensor has been written to since; "
                       << "run forward again before asking for it";
            return nullptr;
        }
        if (missing() && last_input_ && !all_blobs_stored_) {
            const bool fusion = fusion_, fused = last_fused_;
            fusion_ = false;
            forward_layers(last_input_);
            fusion_ = fusion;
            last_fused_ = fused;
        }
        if (missing()) return nullptr;
        return nchw(featmaps_[it->second]);
    }

    // Whether the last forward itself stored blob `name` in float form (false for blobs a fused executor skipped).
    bool blob_stored(std::string_view name) const {
        auto it = blob_index_.find(std::string(name));
        if (it == blob_index_.end()) return false;
        const tensor_ptr& t = featmaps_[it->second];
        return t && !(t->quantized && t->quantized->only);
    }

    // The fp16 layers pass NHWC blobs among themselves; what leaves the pipeline is NCHW as in the reference.
    tensor_ptr nchw(const tensor_ptr& t) const {
        if constexpr (std::is_same_v<Dtype, unsigned short>) {
            if (t && t->order() == memory::NHWC) {
                auto out = std::make_shared<tensor<Dtype>>(std::vector<int>{t->num(), t->channels(), t->height(), t->width()}, device_);
                EXHIP_FATAL(exhip_nhwc_f16_to_nchw_f16(memory::device_context(device_), t->gpu_data(), t->num(), t->channels(),
                                                       t->height(), t->width(), t->channels(), out->mutable_gpu_data()));
                return out;
            }
        }
        return t;
    }

    bool profile_ = false;
    bool fusion_ = true;
    // Fused plans can replay their launches as one HIP graph (set_graphs). Off by default: measured on MI355X the replay
    // is no faster than the calls (the pause between two dependent launches is the device's own hand-over and is there
    // inside a graph too), at batch 32 x 640 x 640 as at one 64 x 64 image.
    bool graphs_ = false;
    bool last_fused_ = false;
    double last_ms_ = 0;
    // time_fused_span / last_span / recent_spans: timed forwards take their event pair from a ring, so that a run of
    // forwards queued back to back can be read after one synchronisation at its end
    static constexpr int kSpanRing = 32;
    int span_first_ = -1, span_launches_ = 0;
    long long span_count_ = 0;  // timed forwards since time_fused_span was last called
    void* span_ev_[kSpanRing][2] = {};
    int device() const { return device_; }
    const int slot_ = memory::stream_slot();  // the stream slot the constructing thread was in: all device work goes there

private:
    // ---------------------------------------------------------------- per-layer executor
    blob_map forward_layers(const tensor_ptr& input) {
        last_fused_ = false;
        last_input_ = input;
        last_input_writes_ = input->writes();
        all_blobs_stored_ = !fusion_;
        featmaps_[blob_index_[input_names_[0]]] = input;
        for (size_t i = 0; i < operations_.size(); ++i) {
            std::vector<tensor_ptr> in, out(op_outputs_[i].size());
            for (int b : op_inputs_[i]) {
                if (!featmaps_[b]) LOG(FATAL) << "layer " << op_params_[i].name_ << " reads blob " << blob_names_[b] << " before it is produced";
                in.push_back(featmaps_[b]);
            }
            if constexpr (std::is_same_v<Dtype, unsigned short>) {
                if (fusion_ && sum_other_[i] >= 0 && featmaps_[sum_other_[i]]) {
                    auto* conv = static_cast<operation_convolution<Dtype>*>(operations_[i].get());
                    const bool paired = pair_[i].on;  // the activation layer between the convolution and the sum
                    if (paired && pair_[i].prelu)
                        conv->set_post_prelu(pair_[i].prelu->weights_f32()[0]->gpu_data(), pair_[i].prelu->share_channel_);
                    else if (paired)
                        conv->set_post_activation(pair_[i].post_op, pair_[i].alpha, pair_[i].beta, pair_[i].relu);
                    conv->set_post_sum(featmaps_[sum_other_[i]], paired);
                    conv->forward_gpu(in, out);
                    const bool summed = conv->post_sum_used();
                    conv->clear_post();
                    size_t done = i;  // the last layer whose work the launch did
                    if (paired) featmaps_[op_outputs_[done++][0]] = nullptr;
                    if (summed) featmaps_[op_outputs_[done++][0]] = nullptr;
                    featmaps_[op_outputs_[done][0]] = out[0];
                    i = done;
                    continue;
                }
            }
            if constexpr (std::is_same_v<Dtype, unsigned short>) {
                if (fusion_ && chain_[i].last > static_cast<int>(i)) {
                    const glue_chain& g = chain_[i];
                    auto* bn = g.bn >= 0 ? static_cast<operation_batchnorm<Dtype>*>(operations_[g.bn].get()) : nullptr;
                    auto* un = g.unary >= 0 ? static_cast<operation_unary<Dtype>*>(operations_[g.unary].get()) : nullptr;
                    bool used = false;
                    if (auto* cat = dynamic_cast<operation_concat<Dtype>*>(operations_[i].get())) {
                        cat->set_post(bn ? bn->a_->gpu_data() : nullptr, bn ? bn->b_->gpu_data() : nullptr, un ? un->op_ : -1,
                                      un ? un->alpha_ : 0.f, un ? un->beta_ : 0.f);
                        cat->forward_gpu(in, out);
                        used = cat->post_used();
                        cat->clear_post();
                    } else {
                        auto* first = static_cast<operation_batchnorm<Dtype>*>(operations_[i].get());
                        first->set_post_unary(un->op_, un->alpha_, un->beta_);
                        first->forward_gpu(in, out);
                        used = first->post_used();
                        first->clear_post();
                    }
                    if (used) {
                        for (int j = static_cast<int>(i); j < g.last; ++j) featmaps_[op_outputs_[j][0]] = nullptr;
                        featmaps_[op_outputs_[g.last][0]] = out[0];
                        i = static_cast<size_t>(g.last);  // the absorbed layers have run
                    } else {
                        featmaps_[op_outputs_[i][0]] = out[0];
                    }
                    continue;
                }
            }
            if (fusion_ && (pair_[i].on || link_[i].on)) {
                auto* conv = static_cast<operation_convolution<Dtype>*>(operations_[i].get());
                if (pair_[i].on && pair_[i].prelu)
                    conv->set_post_prelu(pair_[i].prelu->weights_f32()[0]->gpu_data(), pair_[i].prelu->share_channel_);
                else if (pair_[i].on)
                    conv->set_post_activation(pair_[i].post_op, pair_[i].alpha, pair_[i].beta, pair_[i].relu);
                if (link_[i].on) conv->set_quantized_output(link_[i].fs, link_[i].stride, link_[i].only);
                conv->forward_gpu(in, out);
                conv->clear_post();
                conv->set_quantized_output(0.f, 0, false);
                if (pair_[i].on) {
                    featmaps_[op_outputs_[i][0]] = nullptr;
                    featmaps_[op_outputs_[i + 1][0]] = out[0];
                    ++i;  // the activation layer has run
                } else {
                    featmaps_[op_outputs_[i][0]] = out[0];
                }
                continue;
            }
            operations_[i]->forward_gpu(in, out);
            for (size_t j = 0; j < out.size(); ++j) featmaps_[op_outputs_[i][j]] = out[j];
        }
        blob_map results;
        for (const std::string& o : output_names_) {
            tensor_ptr& blob = featmaps_[blob_index_[o]];
            blob = nchw(blob);
            results[o] = blob;
        }
        return results;
    }

    // ---------------------------------------------------------------- fused int8 executor
    bool try_fused(const tensor_ptr& input, blob_map* results);
    bool build_block_plan(const tensor_ptr& input, const std::vector<int>& shape);  // residual networks: Convolution / max Pooling / Split / add / ReLU
    bool build_graph_plan(const tensor_ptr& input, const std::vector<int>& shape);  // + activation layers, Concat, BatchNorm, Interp, Focus
    struct fused_plan;
    std::shared_ptr<fused_plan> plan_;
    bool fused_unsupported_ = false;

    std::string name_ = "Unknown Pipeleine Name";
    int device_ = -1;
    std::vector<operation_param> op_params_;
    std::vector<std::shared_ptr<operation<Dtype>>> operations_;
    std::map<std::string, int> blob_index_;
    std::vector<std::string> blob_names_;
    std::vector<std::vector<int>> op_inputs_, op_outputs_;
    std::vector<std::string> input_names_, output_names_;
    std::vector<tensor_ptr> featmaps_;
    tensor_ptr last_input_;           // for get_featmap of a blob the fused executors did not store
    unsigned long long last_input_writes_ = 0;  // its write count when the last forward took it
    bool all_blobs_stored_ = false;   // the last forward was a per-layer one with fusion off
    struct post_activation {
        bool on = false, relu = false;
        int post_op = 0;
        float alpha = 0.f, beta = 0.f;
        operation_prelu<Dtype>* prelu = nullptr;
    };
    std::vector<post_activation> pair_;  // per layer: the activation layer on the next line runs in this one's epilogue
    struct quantized_link {
        bool on = false, only = false;
        float fs = 0.f;
        int stride = 0;
    };
    std::vector<int> sum_other_;         // per layer: the other operand's blob of the sum layer this convolution absorbs, or -1
    struct glue_chain {
        int bn = -1, unary = -1, last = -1;  // layer numbers of the absorbed BatchNorm / activation, and of the last absorbed layer
    };
    std::vector<glue_chain> chain_;      // per layer (fp16 pipeline): the layers behind a Concat or BatchNorm that run in its kernel
    std::vector<quantized_link> link_;   // per layer: an int8 convolution that writes its readers' int8 input
    int weights_mem_cost_ = 0;
};

// The plan: device buffers per value and the launches in execution order.
template <typename Dtype>
struct pipeline<Dtype>::impl::fused_plan {
    std::vector<int> in_shape;
    std::vector<dev_buffer> buffers;
    std::vector<std::function<void()>> launches;
    // Results: the launches write through `slot` into `t`, which forward() hands out. A result the caller still holds
    // when the next forward starts is left to the caller: the plan then writes into a new tensor.
    struct result {
        std::string name;         // the network outputs it is, one per line (empty: only a tail layer reads it)
        std::vector<int> blobs;   // blob ids a tail layer reads it by
        std::shared_ptr<tensor<float>> t;
        std::vector<int> shape;
        float* slot = nullptr;
    };
    std::deque<result> outputs;  // stable addresses: the launches keep pointers to the slots
    // Layers in front of the first convolution that work on the caller's NCHW tensor (Input, YoloV5Focus) and layers
    // behind the last one that only rearrange a result (Reshape, Transpose) run as in the per-layer executor, before
    // and after the launches; input_ptr is then the last front layer's blob.
    std::vector<int> front_ops, tail_ops;
    std::shared_ptr<tensor<float>> front_blob;
    const float* input_ptr = nullptr;
    int first_conv_launch = 1;  // 1: launch 0 is the input quantizer; 0: the stem kernel quantizes its own input
    // Launches 1 .. end (everything behind the input quantizer, which alone reads the caller's input pointer) recorded as
    // one HIP graph: made on the plan's second forward (the first runs eagerly, which also sets the kernels' attributes),
    // replayed afterwards, made again when a result tensor was replaced.
    void* graph = nullptr;
    std::vector<float*> graph_slots;
    int forwards = 0;
    std::vector<std::function<void()>> pinned;  // releases of the packed weight copies the launches point to
    ~fused_plan() {
        if (graph) exhip_graph_destroy(graph);
        for (auto& release : pinned) release();
    }
    float** new_result(const std::vector<int>& shape, int device) {
        outputs.emplace_back();
        result& r = outputs.back();
        r.shape = shape;
        r.t = std::make_shared<tensor<float>>(shape, device);
        r.slot = r.t->mutable_gpu_data();
        return &r.slot;
    }
};

template <>
bool pipeline<unsigned short>::impl::try_fused(const tensor_ptr&, blob_map*) { return false; }
template <>
bool pipeline<double>::impl::try_fused(const tensor_ptr&, blob_map*) { return false; }

template <>
bool pipeline<unsigned short>::impl::build_block_plan(const tensor_ptr&, const std::vector<int>&) { return false; }
template <>
bool pipeline<double>::impl::build_block_plan(const tensor_ptr&, const std::vector<int>&) { return false; }
template <>
bool pipeline<unsigned short>::impl::build_graph_plan(const tensor_ptr&, const std::vector<int>&) { return false; }
template <>
bool pipeline<double>::impl::build_graph_plan(const tensor_ptr&, const std::vector<int>&) { return false; }

template <>
bool pipeline<float>::impl::build_block_plan(const tensor_ptr& input, const std::vector<int>& shape) {
    {
        // ---- classify layers; anything outside the fusable set leaves the network to the other planner ----
        using conv_t = operation_convolution<float>;
        const int n_ops = static_cast<int>(operations_.size());
        auto give_up = [&]() { plan_.reset(); return false; };
        if (input->order() != memory::NCHW) return give_up();
        std::vector<int> alias(blob_names_.size());
        for (size_t b = 0; b < alias.size(); ++b) alias[b] = static_cast<int>(b);
        std::vector<char> kind(n_ops, 0);  // c conv, p max pool, s split, a add, r relu
        for (int i = 0; i < n_ops; ++i) {
            operation<float>* op = operations_[i].get();
            if (dynamic_cast<operation_convolutiondepthwise<float>*>(op)) return give_up();
            if (auto* c = dynamic_cast<conv_t*>(op)) {
                if (!c->param().int8_quantization_ || c->group_ != 1 || c->stride_h_ != c->stride_w_ || c->dilation_h_ != 1 ||
                    c->dilation_w_ != 1 || c->activation_type_ > 1 || c->weights_i8().empty())
                    return give_up();
                kind[i] = 'c';
            } else if (auto* p = dynamic_cast<operation_pooling<float>*>(op)) {
                if (p->type_ != 0 || p->global_pooling_) return give_up();
                kind[i] = 'p';
            } else if (dynamic_cast<operation_split<float>*>(op)) {
                kind[i] = 's';
                for (int o : op_outputs_[i]) alias[o] = alias[op_inputs_[i][0]];
            } else if (auto* b = dynamic_cast<operation_binaryop<float>*>(op)) {
                if (b->op_type_ != 0 || b->with_scalar_ || op_inputs_[i].size() != 2) return give_up();
                kind[i] = 'a';
            } else if (dynamic_cast<operation_relu<float>*>(op)) {
                kind[i] = 'r';
            } else {
                return give_up();
            }
        }
        auto root = [&](int b) { return alias[b]; };
        // consumers of every value (through Split aliases)
        std::vector<std::vector<int>> consumers(blob_names_.size());
        for (int i = 0; i < n_ops; ++i)
            if (kind[i] != 's')
                for (int b : op_inputs_[i]) consumers[root(b)].push_back(i);
        std::vector<char> is_output(blob_names_.size(), 0);
        for (const std::string& o : output_names_) is_output[root(blob_index_[o])] = 1;

        // ---- group layers into nodes: conv [+ add] [+ relu], max pool ----
        struct node {
            char kind;            // 'c' or 'p'
            int op;               // conv / pool layer
            int at;               // position in file order at which the node runs
            int in_value, res_value = -1, out_value;
            bool post_relu = false;
            int pool_op = -1;     // conv node: the max pooling layer that reads its output and nothing else does
        };
        std::vector<node> nodes;
        std::vector<char> absorbed(n_ops, 0);
        for (int i = 0; i < n_ops; ++i) {
            if (kind[i] == 'p') {
                if (absorbed[i]) continue;
                nodes.push_back({'p', i, i, root(op_inputs_[i][0]), -1, root(op_outputs_[i][0]), false});
            } else if (kind[i] == 'c') {
                node nd{'c', i, i, root(op_inputs_[i][0]), -1, root(op_outputs_[i][0]), false};
                auto sole = [&](int v, char want) -> int {  // the single consumer of v if it is a layer of kind `want`
                    if (is_output[v] || consumers[v].size() != 1) return -1;
                    const int c = consumers[v][0];
                    return (kind[c] == want && !absorbed[c]) ? c : -1;
                };
                int a = sole(nd.out_value, 'a');
                if (a >= 0) {
                    const int x = root(op_inputs_[a][0]), y = root(op_inputs_[a][1]);
                    nd.res_value = (x == nd.out_value) ? y : x;
                    if (nd.res_value == nd.out_value) return give_up();
                    absorbed[a] = 1;
                    nd.at = a;
                    nd.out_value = root(op_outputs_[a][0]);
                }
                int r = sole(nd.out_value, 'r');
                if (r >= 0) {
                    absorbed[r] = 1;
                    nd.at = r;
                    nd.post_relu = true;
                    nd.out_value = root(op_outputs_[r][0]);
                }
                if (a < 0 && r < 0) {
                    const int pl = sole(nd.out_value, 'p');
                    if (pl >= 0) {
                        absorbed[pl] = 1;
                        nd.at = pl;
                        nd.pool_op = pl;
                        nd.out_value = root(op_outputs_[pl][0]);
                    }
                }
                nodes.push_back(nd);
            }
        }
        for (int i = 0; i < n_ops; ++i)
            if ((kind[i] == 'a' || kind[i] == 'r') && !absorbed[i]) return give_up();  // free-standing elementwise layers
        std::stable_sort(nodes.begin(), nodes.end(), [](const node& a, const node& b) { return a.at < b.at; });

        // ---- what each value must exist as ----
        struct value_info {
            bool need_f32 = false, need_i8 = false;
            float fs = 0.f;
            int n = 0, c = 0, h = 0, w = 0, cs = 0;
            void *f32 = nullptr, *i8 = nullptr;
            float** nchw = nullptr;  // pipeline outputs: the plan's result slot
        };
        std::vector<value_info> vals(blob_names_.size());
        const int in_value = root(blob_index_[input_names_[0]]);
        for (const node& nd : nodes) {
            if (nd.kind == 'c') {
                auto* c = static_cast<conv_t*>(operations_[nd.op].get());
                value_info& v = vals[nd.in_value];
                const float fs = c->featmap_scale();
                if (v.need_i8 && v.fs != fs) return give_up();  // one int8 copy per tensor
                v.need_i8 = true;
                v.fs = fs;
                if (nd.res_value >= 0) vals[nd.res_value].need_f32 = true;
            } else {
                vals[nd.in_value].need_f32 = true;
            }
        }
        if (vals[in_value].need_f32) return give_up();  // the network input is read by int8 convolutions only

        // ---- shapes, buffers, launches ----
        auto plan = std::make_shared<fused_plan>();
        plan->in_shape = shape;
        exhip_ctx* ctx = memory::device_context(device_);
        const int dev = device_;
        auto alloc = [&](size_t bytes) {
            plan->buffers.emplace_back(dev, bytes);
            return plan->buffers.back().ptr;
        };
        {
            value_info& v = vals[in_value];
            v.n = shape[0]; v.c = shape[1]; v.h = shape[2]; v.w = shape[3];
            int kw_first = 0;
            for (const node& nd : nodes)
                if (nd.kind == 'c' && nd.in_value == in_value) kw_first = std::max(kw_first, static_cast<conv_t*>(operations_[nd.op].get())->kernel_size_w_);
            v.cs = (v.c <= 4 && kw_first <= 8) ? 4 : pad_to(v.c, 32);
            v.i8 = alloc(static_cast<size_t>(v.n) * v.h * v.w * v.cs);
            int8_t* q = static_cast<int8_t*>(v.i8);
            const value_info vi = v;
            fused_plan* pl = plan.get();
            plan->launches.push_back([=]() {
                EXHIP_FATAL(exhip_quantize_nchw_f32_to_nhwc_i8(ctx, pl->input_ptr, vi.n, vi.c, vi.h, vi.w, vi.fs, nullptr, vi.cs, q));
            });
            plan->first_conv_launch = 1;
        }
        // A block's projection shortcut (a 1x1 convolution without activation whose result only the block's sum reads) is
        // held back until the convolution that absorbs the sum is planned: exhip_conv2d_i8_projection computes it in that
        // convolution's kernel and its float32 tensor never exists. Where the library declines, the projection is
        // launched on its own right before that convolution.
        struct pending_projection {
            exhip_conv_desc d;
            const int8_t* x;
            const void* wp;
            const float *scale, *bias;
            size_t elems;
        };
        std::map<int, pending_projection> pending;  // by the value the projection produces
        auto launch_projection = [&](int value, const pending_projection& pp) {
            float* yf = static_cast<float*>(vals[value].f32 = alloc(pp.elems * sizeof(float)));
            plan->launches.push_back([=]() { EXHIP_FATAL(exhip_conv2d_i8(ctx, &pp.d, pp.x, pp.wp, pp.scale, pp.bias, nullptr, nullptr, yf, nullptr, nullptr)); });
        };
        for (const node& nd : nodes) {
            const value_info in = vals[nd.in_value];
            value_info& out = vals[nd.out_value];
            if (in.n == 0) return give_up();  // produced by something outside the plan
            if (nd.kind == 'c') {
                auto* c = static_cast<conv_t*>(operations_[nd.op].get());
                if (in.c != c->input_channels() || !in.i8) return give_up();
                const int ks = pad_to(c->output_channel_, 32);
                exhip_conv_desc d = c->describe(in.n, in.h, in.w, in.cs, ks);
                d.post_relu = nd.post_relu ? 1 : 0;
                d.fs_out = out.need_i8 ? out.fs : 0.f;
                int oh, ow;
                EXHIP_FATAL(exhip_conv_out_hw(&d, &oh, &ow));
                out.n = in.n; out.c = c->output_channel_; out.h = oh; out.w = ow; out.cs = ks;
                const size_t elems = static_cast<size_t>(out.n) * oh * ow * ks;
                const bool pooled_node = nd.pool_op >= 0;  // its output tensors have the pooled size: allocated below
                if (!pooled_node && nd.res_value < 0 && !nd.post_relu && d.kh == 1 && d.kw == 1 && d.act == 0 && !is_output[nd.out_value] &&
                    out.need_f32 && !out.need_i8 && consumers[nd.out_value].size() == 1 && kind[consumers[nd.out_value][0]] == 'a') {
                    const void* wp = c->pin_packed_weights(EXHIP_I8, d);
                    plan->pinned.emplace_back([c, wp]() { c->unpin_packed_weights(wp); });
                    pending[nd.out_value] = {d, static_cast<const int8_t*>(in.i8), wp, c->scale_gpu(), c->bias_gpu(), elems};
                    continue;
                }
                if (out.need_i8 && !pooled_node) out.i8 = alloc(elems);
                if (out.need_f32 && !pooled_node) out.f32 = alloc(elems * sizeof(float));
                float** nchw = nullptr;
                if (is_output[nd.out_value] && !pooled_node) nchw = out.nchw = plan->new_result({out.n, out.c, oh, ow}, dev);
                const float* res = nullptr;
                bool with_projection = false;
                pending_projection proj{};
                if (nd.res_value >= 0 && pending.count(nd.res_value)) {
                    proj = pending[nd.res_value];
                    pending.erase(nd.res_value);
                    const value_info& r = vals[nd.res_value];
                    with_projection = !pooled_node && out.i8 && out.f32 && !nchw && r.n == out.n && r.h == oh && r.w == ow && r.cs == ks;
                    if (with_projection) {
                        const void* wp_main = c->pin_packed_weights(EXHIP_I8, d);
                        const int rc = exhip_conv2d_i8_projection(ctx, &d, static_cast<const int8_t*>(in.i8), wp_main, c->scale_gpu(), c->bias_gpu(),
                                                                  &proj.d, proj.x, proj.wp, proj.scale, proj.bias, static_cast<int8_t*>(out.i8),
                                                                  static_cast<float*>(out.f32));  // trial launch
                        c->unpin_packed_weights(wp_main);
                        if (rc == EXHIP_ERR_UNSUPPORTED) with_projection = false;
                        else EXHIP_FATAL(rc);
                    }
                    if (!with_projection) launch_projection(nd.res_value, proj);
                }
                if (nd.res_value >= 0 && !with_projection) {
                    const value_info& r = vals[nd.res_value];
                    if (!r.f32 || r.n != out.n || r.h != oh || r.w != ow || r.cs != ks) return give_up();
                    res = static_cast<const float*>(r.f32);
                }
                const void* wp = c->pin_packed_weights(EXHIP_I8, d);  // the launches below keep this pointer
                plan->pinned.emplace_back([c, wp]() { c->unpin_packed_weights(wp); });
                const float *scale = c->scale_gpu(), *bias = c->bias_gpu();
                const int8_t* x = static_cast<const int8_t*>(in.i8);
                if (nd.pool_op >= 0) {
                    // convolution + max pooling: one kernel when the pool is 3x3 stride 2 and the layer's tiling
                    // allows it, else the two kernels with a float32 tensor between them
                    auto* p = static_cast<operation_pooling<float>*>(operations_[nd.pool_op].get());
                    int kh, kw, sh, sw, pt, pb, pl, pr, ph, pw;
                    p->geometry(oh, ow, &kh, &kw, &sh, &sw, &pt, &pb, &pl, &pr, &ph, &pw);
                    out.h = ph; out.w = pw;
                    const size_t pooled = static_cast<size_t>(out.n) * ph * pw * ks;
                    const bool out_is_result = is_output[nd.out_value];
                    if (out.need_i8) out.i8 = alloc(pooled);
                    if (out.need_f32 || out_is_result || !out.need_i8) out.f32 = alloc(pooled * sizeof(float));
                    int8_t* yq = static_cast<int8_t*>(out.i8);
                    float* yf = static_cast<float*>(out.f32);
                    const value_info o = out;
                    bool one_kernel = kh == 3 && kw == 3 && sh == 2 && sw == 2 && pt <= 1 && pl <= 1 && ks == c->output_channel_ &&
                                      c->output_channel_ % 64 == 0;
                    if (one_kernel) {
                        d.fs_out = o.fs;
                        const int rc = exhip_conv2d_i8_maxpool3x3s2(ctx, &d, pt, pl, ph, pw, x, wp, scale, bias, yq, yf);  // trial launch
                        if (rc == EXHIP_ERR_UNSUPPORTED) one_kernel = false;
                        else EXHIP_FATAL(rc);
                    }
                    // the network's input read by this layer alone: the stem kernel quantizes it on the way in
                    bool stem_kernel = false;
                    if (one_kernel && nd.in_value == in_value && consumers[in_value].size() == 1 && plan->launches.size() == 1) {
                        bool nonneg = true;
                        for (float sc : c->dequantize_scales()) nonneg = nonneg && sc >= 0.f;
                        fused_plan* fp = plan.get();
                        const float fs_in = in.fs;
                        const int nn = nonneg ? 1 : 0;
                        const int rc = exhip_stem_f32_conv_i8_maxpool3x3s2(ctx, &d, pt, pl, ph, pw, input->gpu_data(), fs_in, wp, scale, nn, bias, yq, yf);
                        if (rc == 0) {
                            stem_kernel = true;
                            plan->launches.clear();  // the quantizer's launch
                            plan->first_conv_launch = 0;
                            plan->launches.push_back([=]() {
                                EXHIP_FATAL(exhip_stem_f32_conv_i8_maxpool3x3s2(ctx, &d, pt, pl, ph, pw, fp->input_ptr, fs_in, wp, scale, nn, bias, yq, yf));
                            });
                        } else if (rc != EXHIP_ERR_UNSUPPORTED) {
                            EXHIP_FATAL(rc);
                        }
                    }
                    if (stem_kernel) {
                    } else if (one_kernel) {
                        plan->launches.push_back(
                            [=]() { EXHIP_FATAL(exhip_conv2d_i8_maxpool3x3s2(ctx, &d, pt, pl, ph, pw, x, wp, scale, bias, yq, yf)); });
                    } else {
                        d.fs_out = 0.f;
                        float* mid = static_cast<float*>(alloc(static_cast<size_t>(out.n) * oh * ow * ks * sizeof(float)));
                        const int n = in.n, ch = c->output_channel_;
                        plan->launches.push_back([=]() {
                            EXHIP_FATAL(exhip_conv2d_i8(ctx, &d, x, wp, scale, bias, nullptr, nullptr, mid, nullptr, nullptr));
                            EXHIP_FATAL(exhip_maxpool2d_nhwc_f32(ctx, mid, yf, yq, o.fs, n, ch, oh, ow, ks, ph, pw, kh, kw, sh, sw, pt, pl));
                        });
                    }
                    if (out_is_result) {
                        float** nchw = out.nchw = plan->new_result({out.n, out.c, ph, pw}, dev);
                        plan->launches.push_back([=]() { EXHIP_FATAL(exhip_nhwc_f32_to_nchw_f32(ctx, yf, o.n, o.c, ph, pw, o.cs, *nchw)); });
                    }
                    continue;
                }
                int8_t* yq = static_cast<int8_t*>(out.i8);
                float* yf = static_cast<float*>(out.f32);
                if (!yq && !yf && !nchw) yf = static_cast<float*>(out.f32 = alloc(elems * sizeof(float)));  // dead value: still computed
                if (with_projection) {
                    plan->launches.push_back([=]() {
                        EXHIP_FATAL(exhip_conv2d_i8_projection(ctx, &d, x, wp, scale, bias, &proj.d, proj.x, proj.wp, proj.scale, proj.bias, yq, yf));
                    });
                    continue;
                }
                plan->launches.push_back(
                    [=]() { EXHIP_FATAL(exhip_conv2d_i8(ctx, &d, x, wp, scale, bias, res, yq, yf, nchw ? *nchw : nullptr, nullptr)); });
            } else {
                auto* p = static_cast<operation_pooling<float>*>(operations_[nd.op].get());
                if (!in.f32) return give_up();
                int kh, kw, sh, sw, pt, pb, pl, pr, oh, ow;
                p->geometry(in.h, in.w, &kh, &kw, &sh, &sw, &pt, &pb, &pl, &pr, &oh, &ow);
                out.n = in.n; out.c = in.c; out.h = oh; out.w = ow; out.cs = in.cs;
                const size_t elems = static_cast<size_t>(out.n) * oh * ow * out.cs;
                if (out.need_i8) out.i8 = alloc(elems);
                if (out.need_f32 || is_output[nd.out_value] || !out.need_i8) out.f32 = alloc(elems * sizeof(float));
                const float* x = static_cast<const float*>(in.f32);
                float* yf = static_cast<float*>(out.f32);
                int8_t* yq = static_cast<int8_t*>(out.i8);
                const value_info o = out;
                plan->launches.push_back([=]() {
                    EXHIP_FATAL(exhip_maxpool2d_nhwc_f32(ctx, x, yf, yq, o.fs, in.n, in.c, in.h, in.w, in.cs, oh, ow, kh, kw, sh, sw, pt, pl));
                });
                if (is_output[nd.out_value]) {
                    float** nchw = out.nchw = plan->new_result({out.n, out.c, oh, ow}, dev);
                    plan->launches.push_back([=]() { EXHIP_FATAL(exhip_nhwc_f32_to_nchw_f32(ctx, yf, o.n, o.c, oh, ow, o.cs, *nchw)); });
                }
            }
        }
        for (const auto& kv : pending) launch_projection(kv.first, kv.second);  // never claimed: a sum this plan did not absorb
        // several output names may be Split copies of one value: they share its tensor, as in the per-layer executor
        for (const std::string& o : output_names_) {
            const value_info& v = vals[root(blob_index_[o])];
            if (!v.nchw) return give_up();
            for (auto& r : plan->outputs)
                if (&r.slot == v.nchw) r.name += (r.name.empty() ? "" : "\n") + o;
        }
        plan_ = plan;
    }
    return true;
}

// The planner for int8 networks beyond residual blocks (the detection topologies): every tensor between layers is kept
// in the form its readers take it in -- int8 NHWC at the readers' feature-map scale, float32 NHWC where a sum, a
// BatchNorm or a pooling layer reads it, float32 NCHW where it leaves the network -- and the layers between convolutions
// run on those forms:
//   * Convolution [-> activation layer] [-> add] [-> ReLU] is one launch (the general epilogue applies them in that
//     order, the sum in front of or behind the activation as the layers stand);
//   * Concat [-> BatchNorm] [-> activation] is one launch that also writes the int8 tensor its readers' quantizers would
//     make of the result; a Concat read by int8 convolutions only concatenates int8 tensors (the quantizer works
//     value by value, so it commutes with layers that only move or select values: Concat, nearest Interp, max pooling);
//   * Input and YoloV5Focus in front of the first convolution and Reshape / Transpose behind the last run as layers.
// Values are those of the per-layer executor. Anything else in the topology returns false (the per-layer executor runs).
template <>
bool pipeline<float>::impl::build_graph_plan(const tensor_ptr& input, const std::vector<int>& shape) {
    // EXCALIBUR_PLAN_DEBUG=1 in the environment names the check (by its line in this file) that left a network to the
    // per-layer executor
    auto refuse = [&](int line) {
        if (std::getenv("EXCALIBUR_PLAN_DEBUG")) LOG(INFO) << name_ << ": int8 graph plan not used (the check at pipeline.cpp:" << line << ")";
        return false;
    };
    using conv_t = operation_convolution<float>;
    const int n_ops = static_cast<int>(operations_.size());
    const int n_blobs = static_cast<int>(blob_names_.size());
    if (input->order() != memory::NCHW || shape.size() != 4 || input_names_.size() != 1) return refuse(__LINE__);

    // ---- classify; blobs must be written once (a layer writing over its input is left to the per-layer executor) ----
    std::vector<int> alias(n_blobs), producer(n_blobs, -1);
    for (int b = 0; b < n_blobs; ++b) alias[b] = b;
    std::vector<char> kind(n_ops, 0);  // c conv, u activation, r relu, s split, a add, k concat, b batchnorm, i interp, p max pool, n input, f focus, t tail
    for (int i = 0; i < n_ops; ++i) {
        operation<float>* op = operations_[i].get();
        for (int o : op_outputs_[i]) {
            if (producer[o] >= 0 || o == blob_index_[input_names_[0]]) return refuse(__LINE__);
            producer[o] = i;
        }
        // A layer the plan has no launch for is a tail layer ('t'): it runs as a layer behind the launches, on the NCHW results
        // of the plan. That is right where such layers end a network (a depthwise or float convolution, a sigmoid, an inner
        // product, Reshape / Transpose); one in the middle, whose result a planned layer reads, makes the plan refuse below.
        kind[i] = 't';
        if (dynamic_cast<operation_convolutiondepthwise<float>*>(op)) {
        } else if (auto* c = dynamic_cast<conv_t*>(op)) {
            if (c->param().int8_quantization_ && c->group_ == 1 && c->stride_h_ == c->stride_w_ && c->dilation_h_ == 1 && c->dilation_w_ == 1 &&
                c->activation_type_ <= 1 && !c->weights_i8().empty() && op_inputs_[i].size() == 1 && op_outputs_[i].size() == 1)
                kind[i] = 'c';
        } else if (auto* u = dynamic_cast<operation_unary<float>*>(op)) {
            if (u->op_ != EXHIP_UNARY_SIGMOID) kind[i] = 'u';
        } else if (dynamic_cast<operation_relu<float>*>(op)) {
            kind[i] = 'r';
        } else if (dynamic_cast<operation_split<float>*>(op)) {
            kind[i] = 's';
            for (int o : op_outputs_[i]) alias[o] = alias[op_inputs_[i][0]];
        } else if (auto* b = dynamic_cast<operation_binaryop<float>*>(op)) {
            if (b->op_type_ == 0 && !b->with_scalar_ && op_inputs_[i].size() == 2) kind[i] = 'a';
        } else if (auto* e = dynamic_cast<operation_eltwise<float>*>(op)) {
            // a two-input SUM with unit coefficients is the same sum (x * 1 is exact, fused or not)
            if (e->type_ == 1 && op_inputs_[i].size() == 2 && e->coeffs_.size() == 2 && e->coeffs_[0] == 1.f && e->coeffs_[1] == 1.f) kind[i] = 'a';
        } else if (auto* k = dynamic_cast<operation_concat<float>*>(op)) {
            if (k->axis_ + 2 == 1 && op_inputs_[i].size() <= 8) kind[i] = 'k';
        } else if (dynamic_cast<operation_batchnorm<float>*>(op)) {
            kind[i] = 'b';
        } else if (auto* ip = dynamic_cast<operation_interp<float>*>(op)) {
            if (ip->resize_type_ == 1 && ip->align_corner_ == 0) kind[i] = 'i';
        } else if (auto* p = dynamic_cast<operation_pooling<float>*>(op)) {
            if (p->type_ == 0 && !p->global_pooling_) kind[i] = 'p';
        } else if (dynamic_cast<operation_input<float>*>(op)) {
            kind[i] = 'n';
        } else if (dynamic_cast<operation_yolov5focus<float>*>(op)) {
            kind[i] = 'f';
        }
        if (kind[i] != 's' && kind[i] != 'a' && kind[i] != 'k' && kind[i] != 't' && (op_inputs_[i].size() != 1 || op_outputs_[i].size() != 1))
            return refuse(__LINE__);
        if (op_outputs_[i].size() != 1 && kind[i] != 's' && kind[i] != 't') return refuse(__LINE__);
    }
    auto root = [&](int b) { return alias[b]; };
    std::vector<std::vector<int>> consumers(n_blobs);
    for (int i = 0; i < n_ops; ++i)
        if (kind[i] != 's')
            for (int b : op_inputs_[i]) consumers[root(b)].push_back(i);
    std::vector<char> is_output(n_blobs, 0);
    for (const std::string& o : output_names_) is_output[root(blob_index_[o])] = 1;
    const int in_value = root(blob_index_[input_names_[0]]);

    // ---- the layers in front (a chain from the input, each blob read once until the convolutions) and behind ----
    auto plan = std::make_shared<fused_plan>();
    plan->in_shape = shape;
    std::vector<char> where(n_blobs, 0);  // 0 a value of the plan, 1 an NCHW blob of the front chain, 2 a blob of the tail
    where[in_value] = 1;
    int front_value = in_value;
    std::vector<int> front_shape = shape;
    for (int i = 0; i < n_ops; ++i) {
        if (kind[i] != 'n' && kind[i] != 'f') continue;
        if (root(op_inputs_[i][0]) != front_value || consumers[front_value].size() != 1 || is_output[front_value]) return refuse(__LINE__);
        plan->front_ops.push_back(i);
        front_value = root(op_outputs_[i][0]);
        where[front_value] = 1;
        if (kind[i] == 'f') front_shape = {front_shape[0], front_shape[1] * 4, front_shape[2] / 2, front_shape[3] / 2};
    }
    if (is_output[front_value] || consumers[front_value].empty()) return refuse(__LINE__);
    for (int c : consumers[front_value])
        if (kind[c] != 'c') return refuse(__LINE__);

    // ---- nodes ----
    struct node {
        char kind;  // c convolution, g glue (Concat / BatchNorm / activation), i interp, p max pool
        int op, at;
        std::vector<int> in;
        int res = -1, out = -1;
        int unary = -1, bn = -1;  // layer numbers of the absorbed activation / BatchNorm
        bool post_relu = false, residual_last = false, as_f32 = true;
        int cascade = -1, cascade_k = 0;  // max pool: the value of a smaller pool of the same input to pool again, and with which window
        int head_reshape = -1;            // convolution: the Reshape layer of a detection head (Reshape -> Transpose) it absorbs
        // A Concat [-> BatchNorm] [-> activation] whose inputs are plain 1x1 convolutions read by nothing else and whose result
        // only int8 convolutions read: each producer applies its channels' BatchNorm and the activation in its own
        // epilogue and writes its int8 slice of the joined tensor (`joined`; the producers carry `into` = the Concat's
        // node and their first channel there), so the join costs no launch and no float32 tensor.
        bool joined = false;
        int into = -1, into_offset = 0;
    };
    std::vector<node> nodes;
    std::vector<char> absorbed(n_ops, 0);
    auto sole = [&](int v, char want) -> int {  // the single reader of v if it is an unclaimed layer of kind `want`
        if (is_output[v] || consumers[v].size() != 1) return -1;
        const int c = consumers[v][0];
        return (kind[c] == want && !absorbed[c]) ? c : -1;
    };
    for (int i = 0; i < n_ops; ++i) {
        if (absorbed[i] || kind[i] == 's' || kind[i] == 'n' || kind[i] == 'f' || kind[i] == 't') continue;
        node nd;
        nd.kind = kind[i] == 'c' ? 'c' : kind[i] == 'i' ? 'i' : kind[i] == 'p' ? 'p' : 'g';
        nd.op = nd.at = i;
        for (int b : op_inputs_[i]) nd.in.push_back(root(b));
        nd.out = root(op_outputs_[i][0]);
        auto absorb = [&](int layer) {
            absorbed[layer] = 1;
            nd.at = layer;
            nd.out = root(op_outputs_[layer][0]);
        };
        if (kind[i] == 'c') {
            int act = sole(nd.out, 'u');
            if (act >= 0) {
                nd.unary = act;
                absorb(act);
            } else if ((act = sole(nd.out, 'r')) >= 0) {
                nd.post_relu = true;
                absorb(act);
            }
            // a detection head: convolution -> Reshape (channels into groups) -> Transpose of the last two axes
            const int rs = act < 0 ? sole(nd.out, 't') : -1;
            if (rs >= 0 && dynamic_cast<operation_reshape<float>*>(operations_[rs].get())) {
                const int tp = sole(root(op_outputs_[rs][0]), 't');
                auto* transpose = tp >= 0 ? dynamic_cast<operation_transpose<float>*>(operations_[tp].get()) : nullptr;
                if (transpose && transpose->perms_.size() == 3 && transpose->perms_[0] == 1 && transpose->perms_[1] == 0 && transpose->perms_[2] == 2) {
                    nd.head_reshape = rs;
                    absorb(rs);
                    absorb(tp);
                }
            }
            const int sum = nd.head_reshape < 0 ? sole(nd.out, 'a') : -1;
            if (sum >= 0) {
                const int x = root(op_inputs_[sum][0]), y = root(op_inputs_[sum][1]);
                nd.res = x == nd.out ? y : x;
                if (nd.res == nd.out) return refuse(__LINE__);
                nd.residual_last = act >= 0;
                absorb(sum);
                if (act < 0) {  // the activation behind the sum
                    int behind = sole(nd.out, 'r');
                    if (behind >= 0) {
                        nd.post_relu = true;
                        absorb(behind);
                    } else if ((behind = sole(nd.out, 'u')) >= 0) {
                        nd.unary = behind;
                        absorb(behind);
                    }
                }
            }
        } else if (kind[i] == 'k' || kind[i] == 'b' || kind[i] == 'u') {
            if (kind[i] == 'b') nd.bn = i;
            if (kind[i] == 'u') nd.unary = i;
            if (kind[i] == 'k') {
                const int bn = sole(nd.out, 'b');
                if (bn >= 0) {
                    nd.bn = bn;
                    absorb(bn);
                }
            }
            if (kind[i] != 'u') {
                const int act = sole(nd.out, 'u');
                if (act >= 0) {
                    nd.unary = act;
                    absorb(act);
                }
            }
        } else if (kind[i] == 'a' || kind[i] == 'r') {
            return refuse(__LINE__);  // a sum or ReLU no convolution's epilogue takes
        }
        nodes.push_back(nd);
    }
    std::stable_sort(nodes.begin(), nodes.end(), [](const node& a, const node& b) { return a.at < b.at; });
    for (int i = 0; i < n_ops; ++i) {
        if (absorbed[i]) continue;
        if (kind[i] == 't') {
            for (int b : op_inputs_[i])
                if (where[root(b)] == 1) return refuse(__LINE__);  // the front chain's blobs are not kept
            plan->tail_ops.push_back(i);
            for (int o : op_outputs_[i]) where[root(o)] = 2;
        } else if (kind[i] == 's' && where[root(op_inputs_[i][0])] == 2) {
            plan->tail_ops.push_back(i);  // a Split of a tail blob runs as a layer too: its tops are blobs the tail reads by name
        }
    }
    if (plan->tail_ops.size() == static_cast<size_t>(n_ops)) return refuse(__LINE__);  // nothing left to plan
    for (int i = 0; i < n_ops; ++i)  // nothing but the tail reads the tail
        if (kind[i] != 't' && kind[i] != 's')
            for (int b : op_inputs_[i])
                if (where[root(b)] == 2) return refuse(__LINE__);

    // ---- what each value must exist as: readers first ----
    struct value_info {
        bool need_f32 = false, need_i8 = false, need_nchw = false;
        float fs = 0.f;
        int n = 0, c = 0, h = 0, w = 0, cs = 0;
        void *f32 = nullptr, *i8 = nullptr;
        float** nchw = nullptr;
        // readers with other feature-map scales than `fs`: their int8 forms are made from the float32 form by a quantizer launch
        std::vector<std::pair<float, void*>> more_i8;
        const void* int8_at(float scale) const {
            if (i8 && fs == scale) return i8;
            for (const auto& m : more_i8)
                if (m.first == scale) return m.second;
            return nullptr;
        }
    };
    std::vector<value_info> vals(n_blobs);
    for (int b = 0; b < n_blobs; ++b)
        if (is_output[b] && where[b] == 0) vals[b].need_nchw = true;
    for (int t : plan->tail_ops)
        for (int b : op_inputs_[t])
            if (where[root(b)] == 0) vals[root(b)].need_nchw = true;
    auto want_i8 = [&](int v, float fs) {
        if (!(fs > 0.f)) return refuse(__LINE__);
        value_info& val = vals[v];
        if (!val.need_i8) {
            val.need_i8 = true;
            val.fs = fs;
        } else if (val.fs != fs) {
            // a second scale: that form comes from the float32 form (the network's input has none: layer by layer then)
            if (where[v] != 0) return refuse(__LINE__);
            bool known = false;
            for (const auto& m : val.more_i8) known = known || m.first == fs;
            if (!known) val.more_i8.emplace_back(fs, nullptr);
            val.need_f32 = true;
        }
        return true;
    };
    // channel counts are known from the layers alone; an int8 Concat needs inputs without pad channels
    vals[front_value].c = front_shape[1];
    for (const node& nd : nodes) {
        int c = 0;
        if (nd.kind == 'c') c = static_cast<conv_t*>(operations_[nd.op].get())->output_channel_;
        else if (nd.kind == 'g') for (int v : nd.in) c += vals[v].c;
        else c = vals[nd.in[0]].c;
        vals[nd.out].c = c;
    }
    std::vector<int> node_of(n_blobs, -1);  // the node that produces a value
    for (size_t i = 0; i < nodes.size(); ++i) node_of[nodes[i].out] = static_cast<int>(i);
    for (auto it = nodes.rbegin(); it != nodes.rend(); ++it) {
        node& nd = *it;
        const value_info out = vals[nd.out];
        if (where[nd.out] != 0) return refuse(__LINE__);
        if (nd.kind == 'c') {
            auto* c = static_cast<conv_t*>(operations_[nd.op].get());
            if (!want_i8(nd.in[0], c->featmap_scale())) return refuse(__LINE__);
            if (nd.res >= 0) {
                if (where[nd.res] != 0) return refuse(__LINE__);
                vals[nd.res].need_f32 = true;
            }
            continue;
        }
        if (!out.need_i8 && !out.need_f32 && !out.need_nchw) return refuse(__LINE__);  // nobody reads it
        for (int v : nd.in)
            if (where[v] != 0) return refuse(__LINE__);
        if (nd.kind == 'g') {
            if (kind[nd.op] == 'k' && out.need_i8 && !out.need_f32 && !out.need_nchw && out.more_i8.empty() && vals[nd.out].c % 32 == 0) {
                bool ok = true;
                for (int v : nd.in) {
                    const int pn = node_of[v];
                    ok = ok && pn >= 0 && !is_output[v] && consumers[v].size() == 1 && vals[v].c % 32 == 0;
                    if (!ok) break;
                    const node& pr = nodes[pn];
                    auto* c = pr.kind == 'c' ? static_cast<conv_t*>(operations_[pr.op].get()) : nullptr;
                    ok = c && pr.unary < 0 && !pr.post_relu && pr.res < 0 && pr.head_reshape < 0 && pr.into < 0 && c->kernel_size_h_ == 1 &&
                         c->kernel_size_w_ == 1 && c->stride_h_ == 1 && c->stride_w_ == 1 && c->pad_top_ == 0 && c->pad_bottom_ == 0 &&
                         c->pad_left_ == 0 && c->pad_right_ == 0;
                }
                if (nd.unary >= 0 && static_cast<operation_unary<float>*>(operations_[nd.unary].get())->op_ == EXHIP_UNARY_SIGMOID) ok = false;
                if (ok) {
                    nd.joined = true;
                    int offset = 0;
                    const int self = static_cast<int>(&nd - nodes.data());
                    for (int v : nd.in) {
                        nodes[node_of[v]].into = self;
                        nodes[node_of[v]].into_offset = offset;
                        offset += vals[v].c;
                    }
                    continue;
                }
            }
            nd.as_f32 = nd.bn >= 0 || nd.unary >= 0 || out.need_f32 || out.need_nchw;
            for (int v : nd.in)
                if (vals[v].c % 32 != 0) nd.as_f32 = true;
            for (int v : nd.in) {
                if (nd.as_f32) vals[v].need_f32 = true;
                else if (!want_i8(v, out.fs)) return refuse(__LINE__);
            }
        } else if (nd.kind == 'i') {
            if (out.need_i8 && !want_i8(nd.in[0], out.fs)) return refuse(__LINE__);
            if (out.need_f32 || out.need_nchw) vals[nd.in[0]].need_f32 = true;
        } else {
            // A pyramid of stride-1 "same" max pools over one tensor (windows 5 / 9 / 13): the maximum over a window of k is
            // the maximum over a window of k - k' + 1 of the maxima over windows of k' (taps outside the image count in
            // neither), so each pool reads the next smaller one's result with a 5-wide window instead of 81 or 169 taps.
            auto same_window = [&](const node& q) {
                auto* p = static_cast<operation_pooling<float>*>(operations_[q.op].get());
                const int k = p->kernel_size_w_;
                const bool same = k == p->kernel_size_h_ && (k & 1) && p->stride_w_ == 1 && p->stride_h_ == 1 && p->pad_left_ == k / 2 &&
                                  p->pad_right_ == k / 2 && p->pad_top_ == k / 2 && p->pad_bottom_ == k / 2;
                return same ? k : 0;
            };
            const int k = same_window(nd);
            int best = 0;
            if (k > 0)
                for (const node& q : nodes) {
                    if (q.kind != 'p' || q.op == nd.op || q.at > nd.at || q.in[0] != nd.in[0]) continue;
                    const int kq = same_window(q);
                    if (kq > best && kq < k) {
                        best = kq;
                        nd.cascade = q.out;
                        nd.cascade_k = k - kq + 1;
                    }
                }
            // read by int8 convolutions only (at one scale): the pool runs on the int8 tensor, the quantizer being monotone
            nd.as_f32 = out.need_f32 || out.need_nchw || !out.need_i8 || !out.more_i8.empty();
            const int source = nd.cascade >= 0 ? nd.cascade : nd.in[0];
            if (nd.as_f32) vals[source].need_f32 = true;
            else if (!want_i8(source, out.fs)) return refuse(__LINE__);
        }
    }

    // ---- shapes, buffers, launches ----
    struct {  // the int8 pooling pyramid whose launch is the plan's last one
        const int8_t* x = nullptr;
        int8_t* y[3] = {nullptr, nullptr, nullptr};
        int levels = 0, k = 0, n = 0, h = 0, w = 0, cs = 0;
        size_t launch = 0;
    } pyramid;
    exhip_ctx* ctx = memory::device_context(device_);
    const int dev = device_;
    auto alloc = [&](size_t bytes) {
        plan->buffers.emplace_back(dev, bytes);
        return plan->buffers.back().ptr;
    };
    auto blobs_of = [&](int value) {  // the names a tail layer may read the value by
        std::vector<int> ids;
        for (int b = 0; b < n_blobs; ++b)
            if (root(b) == value) ids.push_back(b);
        return ids;
    };
    auto nchw_result = [&](value_info& v, int value) {
        v.nchw = plan->new_result({v.n, v.c, v.h, v.w}, dev);
        plan->outputs.back().blobs = blobs_of(value);
        return v.nchw;
    };
    {
        value_info& v = vals[front_value];
        if (!v.need_i8 || v.need_f32 || v.need_nchw) return refuse(__LINE__);
        v.n = front_shape[0]; v.c = front_shape[1]; v.h = front_shape[2]; v.w = front_shape[3];
        int kw_first = 0;
        for (int c : consumers[front_value]) kw_first = std::max(kw_first, static_cast<conv_t*>(operations_[c].get())->kernel_size_w_);
        v.cs = (v.c <= 4 && kw_first <= 8) ? 4 : pad_to(v.c, 32);
        v.i8 = alloc(static_cast<size_t>(v.n) * v.h * v.w * v.cs);
        int8_t* q = static_cast<int8_t*>(v.i8);
        const value_info vi = v;
        fused_plan* pl = plan.get();
        // Input -> YoloV5Focus -> quantizer as one kernel where the library has it; else the two layers run as layers
        bool one_kernel = false;
        if (plan->front_ops.size() == 2 && kind[plan->front_ops[0]] == 'n' && kind[plan->front_ops[1]] == 'f') {
            auto* in_op = static_cast<operation_input<float>*>(operations_[plan->front_ops[0]].get());
            const int ch = shape[1];
            if ((ch == 1 || ch == 3) && static_cast<int>(in_op->means_.size()) == ch && static_cast<int>(in_op->vars_.size()) >= ch) {
                std::array<float, 4> means{}, scales{};
                for (int c = 0; c < ch; ++c) { means[c] = in_op->means_[c]; scales[c] = in_op->vars_[c]; }
                const int n0 = shape[0], h0 = shape[2], w0 = shape[3];
                const int rc = exhip_input_focus_quantize_nchw_f32_to_nhwc_i8(ctx, input->gpu_data(), n0, ch, h0, w0, means.data(), scales.data(),
                                                                              vi.fs, vi.cs, q);  // trial launch
                if (rc == 0) {
                    one_kernel = true;
                    plan->front_ops.clear();
                    plan->launches.push_back([=]() {
                        EXHIP_FATAL(exhip_input_focus_quantize_nchw_f32_to_nhwc_i8(ctx, pl->input_ptr, n0, ch, h0, w0, means.data(), scales.data(), vi.fs,
                                                                                    vi.cs, q));
                    });
                } else if (rc != EXHIP_ERR_UNSUPPORTED) {
                    EXHIP_FATAL(rc);
                }
            }
        }
        if (!one_kernel)
            plan->launches.push_back(
                [=]() { EXHIP_FATAL(exhip_quantize_nchw_f32_to_nhwc_i8(ctx, pl->input_ptr, vi.n, vi.c, vi.h, vi.w, vi.fs, nullptr, vi.cs, q)); });
        plan->first_conv_launch = 1;
    }
    // a value that leaves as NCHW from a layer other than a convolution: converted from its float32 NHWC form
    auto nchw_from_f32 = [&](value_info& v, int value) {
        if (!v.need_nchw) return;
        float** slot = nchw_result(v, value);
        const value_info o = v;
        plan->launches.push_back(
            [=]() { EXHIP_FATAL(exhip_nhwc_f32_to_nchw_f32(ctx, static_cast<const float*>(o.f32), o.n, o.c, o.h, o.w, o.cs, *slot)); });
    };
    // the int8 forms of a value at its readers' other scales: the quantizer on the float32 NHWC form
    auto more_forms = [&](value_info& v) {
        if (v.more_i8.empty()) return true;
        if (!v.f32 || v.c % 4 != 0 || v.cs % 4 != 0) return false;
        const size_t pixels = static_cast<size_t>(v.n) * v.h * v.w;
        for (auto& m : v.more_i8) {
            m.second = alloc(pixels * v.cs);
            const float* src = static_cast<const float*>(v.f32);
            int8_t* dst = static_cast<int8_t*>(m.second);
            const int ch = v.c, stride = v.cs;
            const float scale = m.first;
            plan->launches.push_back([=]() {
                EXHIP_FATAL(exhip_concat_batchnorm_unary_nhwc_f32(ctx, &src, &ch, &stride, 1, pixels, nullptr, nullptr, -1, 0.f, 0.f, stride, nullptr, dst,
                                                                  scale));
            });
        }
        return true;
    };
    for (const node& nd : nodes) {
        const value_info in = vals[nd.in[0]];
        value_info& out = vals[nd.out];
        if (in.n == 0) return refuse(__LINE__);
        if (nd.kind == 'c') {
            auto* c = static_cast<conv_t*>(operations_[nd.op].get());
            const int8_t* x = static_cast<const int8_t*>(in.int8_at(c->featmap_scale()));
            if (in.c != c->input_channels() || !x) return refuse(__LINE__);
            const int ks = pad_to(c->output_channel_, 32);
            exhip_conv_desc d = c->describe(in.n, in.h, in.w, in.cs, ks);
            d.post_relu = nd.post_relu ? 1 : 0;
            d.residual_last = nd.residual_last ? 1 : 0;
            if (nd.unary >= 0) {
                auto* u = static_cast<operation_unary<float>*>(operations_[nd.unary].get());
                d.post_op = 1 + u->op_; d.post_alpha = u->alpha_; d.post_beta = u->beta_;
            }
            d.fs_out = out.need_i8 ? out.fs : 0.f;
            int oh, ow;
            EXHIP_FATAL(exhip_conv_out_hw(&d, &oh, &ow));
            out.n = in.n; out.c = c->output_channel_; out.h = oh; out.w = ow; out.cs = ks;
            const size_t elems = static_cast<size_t>(out.n) * oh * ow * ks;
            if (nd.into >= 0) {
                // a producer of a joined Concat: BatchNorm and activation of its channels in its own epilogue, its int8 slice
                // written into the joined tensor
                const node& jn = nodes[nd.into];
                value_info& jo = vals[jn.out];
                const int total = jo.c;
                if (!jo.i8) {
                    jo.n = in.n; jo.h = oh; jo.w = ow; jo.cs = total;
                    jo.i8 = alloc(static_cast<size_t>(in.n) * oh * ow * total);
                } else if (jo.n != in.n || jo.h != oh || jo.w != ow) {
                    return refuse(__LINE__);
                }
                d.k_stride = total;
                d.exact_k = 1;
                d.fs_out = jo.fs;
                if (jn.bn >= 0) {
                    auto* bn = static_cast<operation_batchnorm<float>*>(operations_[jn.bn].get());
                    if (bn->channels_ != total || !bn->a_ || !bn->b_) return refuse(__LINE__);
                    d.post_bn_a = bn->a_->gpu_data() + nd.into_offset;
                    d.post_bn_b = bn->b_->gpu_data() + nd.into_offset;
                }
                if (jn.unary >= 0) {
                    auto* u = static_cast<operation_unary<float>*>(operations_[jn.unary].get());
                    d.post_op = 1 + u->op_; d.post_alpha = u->alpha_; d.post_beta = u->beta_;
                }
                const void* wp = c->pin_packed_weights(EXHIP_I8, d);
                plan->pinned.emplace_back([c, wp]() { c->unpin_packed_weights(wp); });
                const float *scale = c->scale_gpu(), *bias = c->bias_gpu();
                int8_t* yq = static_cast<int8_t*>(jo.i8) + nd.into_offset;
                const int rc = exhip_conv2d_i8(ctx, &d, x, wp, scale, bias, nullptr, yq, nullptr, nullptr, nullptr);  // trial launch
                if (rc == EXHIP_ERR_UNSUPPORTED) return refuse(__LINE__);
                EXHIP_FATAL(rc);
                plan->launches.push_back([=]() { EXHIP_FATAL(exhip_conv2d_i8(ctx, &d, x, wp, scale, bias, nullptr, yq, nullptr, nullptr, nullptr)); });
                continue;
            }
            if (nd.head_reshape >= 0) {
                // [n, K, oh, ow] -> Reshape [n, G, J, oh * ow] -> Transpose [n, G, oh * ow, J]: the convolution writes float32
                // NHWC and one kernel regroups the channels of every pixel
                auto* rs = static_cast<operation_reshape<float>*>(operations_[nd.head_reshape].get());
                const std::vector<int> to = rs->new_shape({in.n, c->output_channel_, oh, ow}, in.n * c->output_channel_ * oh * ow);
                if (to.size() != 4 || to[0] != in.n || to[1] * to[2] != c->output_channel_ || to[3] != oh * ow) return refuse(__LINE__);
                if (out.need_i8 || out.need_f32 || !out.need_nchw || nd.res >= 0) return refuse(__LINE__);
                const int groups = to[1], per_group = to[2], hw = oh * ow, n0 = in.n;
                out.n = in.n; out.c = groups; out.h = hw; out.w = per_group; out.cs = 0;
                float* mid = static_cast<float*>(alloc(elems * sizeof(float)));
                float** slot = nchw_result(out, nd.out);
                const void* wp = c->pin_packed_weights(EXHIP_I8, d);
                plan->pinned.emplace_back([c, wp]() { c->unpin_packed_weights(wp); });
                const float *scale = c->scale_gpu(), *bias = c->bias_gpu();
                plan->launches.push_back([=]() {
                    EXHIP_FATAL(exhip_conv2d_i8(ctx, &d, x, wp, scale, bias, nullptr, nullptr, mid, nullptr, nullptr));
                    EXHIP_FATAL(exhip_nhwc_f32_to_grouped_f32(ctx, mid, n0, hw, groups, per_group, ks, *slot));
                });
                continue;
            }
            if (out.need_i8) out.i8 = alloc(elems);
            if (out.need_f32 || (!out.need_i8 && !out.need_nchw)) out.f32 = alloc(elems * sizeof(float));
            float** nchw = out.need_nchw ? nchw_result(out, nd.out) : nullptr;
            const float* res = nullptr;
            if (nd.res >= 0) {
                const value_info& r = vals[nd.res];
                if (!r.f32 || r.n != out.n || r.h != oh || r.w != ow || r.cs != ks || r.c != out.c) return refuse(__LINE__);
                res = static_cast<const float*>(r.f32);
            }
            const void* wp = c->pin_packed_weights(EXHIP_I8, d);  // the launch keeps this pointer
            plan->pinned.emplace_back([c, wp]() { c->unpin_packed_weights(wp); });
            const float *scale = c->scale_gpu(), *bias = c->bias_gpu();
            int8_t* yq = static_cast<int8_t*>(out.i8);
            float* yf = static_cast<float*>(out.f32);
            plan->launches.push_back(
                [=]() { EXHIP_FATAL(exhip_conv2d_i8(ctx, &d, x, wp, scale, bias, res, yq, yf, nchw ? *nchw : nullptr, nullptr)); });
        } else if (nd.kind == 'g' && nd.joined) {
            if (!out.i8 || out.n != in.n || out.h != in.h || out.w != in.w) return refuse(__LINE__);  // its producers wrote it
            continue;
        } else if (nd.kind == 'g') {
            int total = 0;
            std::vector<const void*> ptrs;
            std::vector<int> channels, strides;
            for (int v : nd.in) {
                const value_info& s = vals[v];
                if (s.n != in.n || s.h != in.h || s.w != in.w || s.c % 4 != 0) return refuse(__LINE__);
                const void* form = nd.as_f32 ? s.f32 : s.int8_at(out.fs);
                if (!form || (!nd.as_f32 && (s.cs != s.c || s.c % 16 != 0))) return refuse(__LINE__);
                ptrs.push_back(form);
                channels.push_back(s.c);
                strides.push_back(s.cs);
                total += s.c;
            }
            out.n = in.n; out.c = total; out.h = in.h; out.w = in.w; out.cs = pad_to(total, 32);
            const size_t pixels = static_cast<size_t>(out.n) * out.h * out.w;
            const size_t elems = pixels * out.cs;
            if (out.need_i8) out.i8 = alloc(elems);
            const int n_in = static_cast<int>(ptrs.size());
            if (nd.as_f32) {
                if (out.need_f32 || out.need_nchw) out.f32 = alloc(elems * sizeof(float));
                const float *bn_a = nullptr, *bn_b = nullptr;
                if (nd.bn >= 0) {
                    auto* bn = static_cast<operation_batchnorm<float>*>(operations_[nd.bn].get());
                    if (bn->channels_ != total || !bn->a_ || !bn->b_) return refuse(__LINE__);
                    bn_a = bn->a_->gpu_data();
                    bn_b = bn->b_->gpu_data();
                }
                int uop = -1;
                float alpha = 0.f, beta = 0.f;
                if (nd.unary >= 0) {
                    auto* u = static_cast<operation_unary<float>*>(operations_[nd.unary].get());
                    uop = u->op_; alpha = u->alpha_; beta = u->beta_;
                }
                const value_info o = out;
                plan->launches.push_back([=]() {
                    EXHIP_FATAL(exhip_concat_batchnorm_unary_nhwc_f32(ctx, reinterpret_cast<const float* const*>(ptrs.data()), channels.data(),
                                                                      strides.data(), n_in, pixels, bn_a, bn_b, uop, alpha, beta, o.cs,
                                                                      static_cast<float*>(o.f32), static_cast<int8_t*>(o.i8), o.fs));
                });
                nchw_from_f32(out, nd.out);
            } else {
                if (out.cs != total) return refuse(__LINE__);
                std::vector<int> pairs;  // the byte tensors as tensors of two-byte elements
                for (int ch : channels) pairs.push_back(ch / 2);
                uint16_t* y = static_cast<uint16_t*>(out.i8);
                plan->launches.push_back([=]() {
                    EXHIP_FATAL(exhip_concat_channels_nhwc_f16(ctx, reinterpret_cast<const uint16_t* const*>(ptrs.data()), pairs.data(), n_in, pixels, y));
                });
            }
        } else if (nd.kind == 'i') {
            auto* ip = static_cast<operation_interp<float>*>(operations_[nd.op].get());
            int oh = ip->output_height_, ow = ip->output_width_;
            if (oh == 0 || ow == 0) {
                oh = static_cast<int>(in.h * ip->height_scale_);
                ow = static_cast<int>(in.w * ip->width_scale_);
            }
            if (oh <= 0 || ow <= 0) return refuse(__LINE__);
            out.n = in.n; out.c = in.c; out.h = oh; out.w = ow; out.cs = in.cs;
            const size_t elems = static_cast<size_t>(out.n) * oh * ow * out.cs;
            if (out.need_i8) {
                const uint16_t* x = static_cast<const uint16_t*>(in.int8_at(out.fs));
                if (!x || in.cs % 16 != 0) return refuse(__LINE__);
                out.i8 = alloc(elems);
                uint16_t* y = static_cast<uint16_t*>(out.i8);
                plan->launches.push_back([=]() { EXHIP_FATAL(exhip_interp_nearest_nhwc_f16(ctx, x, y, in.n, in.cs / 2, in.h, in.w, oh, ow)); });
            }
            if (out.need_f32 || out.need_nchw) {
                if (!in.f32 || in.cs % 4 != 0) return refuse(__LINE__);
                out.f32 = alloc(elems * sizeof(float));
                const uint16_t* x = static_cast<const uint16_t*>(in.f32);
                uint16_t* y = static_cast<uint16_t*>(out.f32);
                plan->launches.push_back([=]() { EXHIP_FATAL(exhip_interp_nearest_nhwc_f16(ctx, x, y, in.n, in.cs * 2, in.h, in.w, oh, ow)); });
                nchw_from_f32(out, nd.out);
            }
        } else {
            auto* p = static_cast<operation_pooling<float>*>(operations_[nd.op].get());
            int kh, kw, sh, sw, pt, pb, pl, pr, oh, ow;
            p->geometry(in.h, in.w, &kh, &kw, &sh, &sw, &pt, &pb, &pl, &pr, &oh, &ow);
            const void* source = nd.as_f32 ? in.f32 : in.int8_at(out.fs);
            if (nd.cascade >= 0) {  // the smaller pool's result, pooled again (same size as the input: stride 1, "same" padding)
                const value_info& q = vals[nd.cascade];
                if (q.n != in.n || q.h != in.h || q.w != in.w || q.cs != in.cs || oh != in.h || ow != in.w) return refuse(__LINE__);
                source = nd.as_f32 ? q.f32 : q.int8_at(out.fs);
                kh = kw = nd.cascade_k;
                pt = pl = nd.cascade_k / 2;
            }
            if (!source) return refuse(__LINE__);
            out.n = in.n; out.c = in.c; out.h = oh; out.w = ow; out.cs = in.cs;
            const size_t elems = static_cast<size_t>(out.n) * oh * ow * out.cs;
            if (out.need_i8) out.i8 = alloc(elems);
            if (out.need_f32 || out.need_nchw) out.f32 = alloc(elems * sizeof(float));
            int8_t* yq = static_cast<int8_t*>(out.i8);
            if (!nd.as_f32) {
                if (in.cs % 16 != 0 || pt >= kh || pl >= kw) return refuse(__LINE__);
                const int8_t* xq = static_cast<const int8_t*>(source);
                // A pool that pools the result of the pool launched just before it with the same window (the 5 / 9 / 13
                // pyramid as 5, 5 of 5, 5 of that) joins that launch: one kernel keeps the map in LDS for all levels.
                const bool same = kh == kw && (kh & 1) && sh == 1 && sw == 1 && pt == kh / 2 && pl == kh / 2 && oh == in.h && ow == in.w;
                if (same && nd.cascade >= 0 && pyramid.levels > 0 && pyramid.levels < 3 && pyramid.launch + 1 == plan->launches.size() &&
                    xq == pyramid.y[pyramid.levels - 1] && kh == pyramid.k && in.n == pyramid.n && in.h == pyramid.h && in.w == pyramid.w &&
                    in.cs == pyramid.cs) {
                    pyramid.y[pyramid.levels++] = yq;
                    const auto py = pyramid;
                    const int c = in.c;
                    plan->launches.back() = [=]() {
                        EXHIP_FATAL(exhip_maxpool_same_pyramid_nhwc_i8(ctx, py.x, py.y[0], py.y[1], py.y[2], py.n, c, py.h, py.w, py.cs, py.k));
                    };
                } else {
                    plan->launches.push_back(
                        [=]() { EXHIP_FATAL(exhip_maxpool2d_nhwc_i8(ctx, xq, yq, in.n, in.c, in.h, in.w, in.cs, oh, ow, kh, kw, sh, sw, pt, pl)); });
                    pyramid = {};
                    if (same) {
                        pyramid.x = xq; pyramid.y[0] = yq; pyramid.levels = 1; pyramid.launch = plan->launches.size() - 1;
                        pyramid.k = kh; pyramid.n = in.n; pyramid.h = in.h; pyramid.w = in.w; pyramid.cs = in.cs;
                    }
                }
            } else {
                const float* x = static_cast<const float*>(source);
                float* yf = static_cast<float*>(out.f32);
                const float fs = out.fs;
                plan->launches.push_back([=]() {
                    EXHIP_FATAL(exhip_maxpool2d_nhwc_f32(ctx, x, yf, yq, fs, in.n, in.c, in.h, in.w, in.cs, oh, ow, kh, kw, sh, sw, pt, pl));
                });
                nchw_from_f32(out, nd.out);
            }
        }
        if (!more_forms(out)) return refuse(__LINE__);
    }
    // the network's outputs: results of the plan by name (Split copies share their tensor), the rest comes from the tail
    for (const std::string& o : output_names_) {
        const int v = root(blob_index_[o]);
        if (where[v] == 2) continue;
        if (where[v] != 0 || !vals[v].nchw) return refuse(__LINE__);
        for (auto& r : plan->outputs)
            if (&r.slot == vals[v].nchw) r.name += (r.name.empty() ? "" : "\n") + o;
    }
    plan_ = plan;
    return true;
}

template <>
bool pipeline<float>::impl::try_fused(const tensor_ptr& input, blob_map* results) {
    if (!fusion_ || fused_unsupported_) return false;
    const std::vector<int> shape = input->data_shape();
    if (!plan_ || plan_->in_shape != shape) {
        plan_.reset();
        if (!build_block_plan(input, shape) && !build_graph_plan(input, shape)) {
            fused_unsupported_ = true;  // the per-layer executor from now on
            plan_.reset();
            return false;
        }
    }
    // layers in front of the first convolution that work on the caller's NCHW tensor
    {
        tensor_ptr blob = input;
        for (int op : plan_->front_ops) {
            std::vector<tensor_ptr> in{blob}, out(1);
            operations_[op]->forward_gpu(in, out);
            blob = out[0];
        }
        plan_->front_blob = blob;
        plan_->input_ptr = blob->gpu_data();
    }
    last_input_ = input;
    last_input_writes_ = input->writes();
    all_blobs_stored_ = false;
    for (tensor_ptr& t : featmaps_) t = nullptr;  // nothing of an earlier input stays readable
    featmaps_[blob_index_[input_names_[0]]] = input;
    for (auto& r : plan_->outputs) {
        if (r.t.use_count() > 1) {  // a result of an earlier forward is still held outside: it stays the caller's
            r.t = std::make_shared<tensor<float>>(r.shape, device_);
            r.slot = r.t->mutable_gpu_data();
        } else if (r.t->data_shape() != r.shape) {
            r.t->reshape(r.shape);  // a Reshape layer behind it gave the tensor another shape in the last forward
        }
    }
    exhip_ctx* const ctx = memory::device_context(device_);
    const int n_launches = static_cast<int>(plan_->launches.size());
    const int span_first = span_first_ == -2 ? plan_->first_conv_launch : span_first_;  // -2: from the first convolution on
    const bool timed = span_first >= 0 && span_first < n_launches;
    void** const span_ev = span_ev_[span_count_ % kSpanRing];
    if (timed && !span_ev[0]) {
        EXHIP_FATAL(exhip_event_create(&span_ev[0]));
        EXHIP_FATAL(exhip_event_create(&span_ev[1]));
    }
    // the graph form: launch 0 eagerly, the rest as one replay (a timed span must start at launch 0 or 1 to use it)
    bool use_graph = graphs_ && n_launches > 2 && plan_->forwards >= 1 && (!timed || span_first <= 1);
    if (use_graph) {
        std::vector<float*> slots;
        for (auto& r : plan_->outputs) slots.push_back(r.slot);
        if (plan_->graph && slots != plan_->graph_slots) {
            EXHIP_FATAL(exhip_graph_destroy(plan_->graph));
            plan_->graph = nullptr;
        }
        if (!plan_->graph) {
            EXHIP_FATAL(exhip_graph_begin(ctx));
            for (int i = 1; i < n_launches; ++i) plan_->launches[i]();
            EXHIP_FATAL(exhip_graph_end(ctx, &plan_->graph));
            plan_->graph_slots = slots;
        }
        if (timed && span_first == 0) EXHIP_FATAL(exhip_event_record(ctx, span_ev[0]));
        plan_->launches[0]();
        if (timed && span_first == 1) EXHIP_FATAL(exhip_event_record(ctx, span_ev[0]));
        EXHIP_FATAL(exhip_graph_launch(ctx, plan_->graph));
        if (timed) EXHIP_FATAL(exhip_event_record(ctx, span_ev[1]));
        span_launches_ = timed ? n_launches - span_first : 0;
    } else if (timed) {
        for (int i = 0; i < n_launches; ++i) {
            if (i == span_first) EXHIP_FATAL(exhip_event_record(ctx, span_ev[0]));
            plan_->launches[i]();
        }
        EXHIP_FATAL(exhip_event_record(ctx, span_ev[1]));
        span_launches_ = n_launches - span_first;
    } else {
        for (auto& launch : plan_->launches) launch();
        span_launches_ = 0;
    }
    if (timed) ++span_count_;
    ++plan_->forwards;
    last_fused_ = true;
    for (auto& r : plan_->outputs) {
        r.t->mutable_gpu_data();  // the kernels just wrote it: the device copy is the newest
        for (int b : r.blobs) featmaps_[b] = r.t;
        if (r.name.empty()) continue;
        for (const std::string& name : split_string(r.name, "\n")) {
            (*results)[name] = r.t;
            featmaps_[blob_index_[name]] = r.t;
        }
    }
    // layers that only rearrange a result
    for (int op : plan_->tail_ops) {
        std::vector<tensor_ptr> in, out(op_outputs_[op].size());
        for (int b : op_inputs_[op]) in.push_back(featmaps_[b]);
        operations_[op]->forward_gpu(in, out);
        for (size_t j = 0; j < out.size(); ++j) featmaps_[op_outputs_[op][j]] = out[j];
    }
    if (!plan_->tail_ops.empty())
        for (const std::string& o : output_names_)
            if (!results->count(o)) (*results)[o] = featmaps_[blob_index_[o]];
    return true;
}

// ---------------------------------------------------------------- public wrappers
namespace {
std::vector<std::string> read_lines(std::string_view path) {
    std::vector<std::string> lines;
    std::ifstream in{std::string(path)};
    std::string line;
    while (in.is_open() && std::getline(in, line)) lines.push_back(line);
    return lines;
}
}  // namespace

template <typename Dtype>
pipeline<Dtype>::pipeline() : impl_(new impl()) {}
template <typename Dtype>
pipeline<Dtype>::pipeline(std::string_view param_file, std::string_view model_file, int device)
    : impl_(new impl(read_lines(param_file), model_file, device)) {}
template <typename Dtype>
pipeline<Dtype>::pipeline(std::string_view param_file, int device) : impl_(new impl(read_lines(param_file), std::string_view(), device)) {}
template <typename Dtype>
pipeline<Dtype>::pipeline(const std::vector<std::string>& hardcode_params, std::string_view model_file, int device)
    : impl_(new impl(hardcode_params, model_file, device)) {}
// Every entry that touches the device works in the pipeline's own stream slot, whichever slot the caller is in.
template <typename Dtype>
pipeline<Dtype>::~pipeline() {
    memory::stream_scope scope(impl_->slot_);
    delete impl_;
}
template <typename Dtype>
typename pipeline<Dtype>::blob_map pipeline<Dtype>::forward(const std::shared_ptr<memory::tensor<Dtype>>& t) {
    memory::stream_scope scope(impl_->slot_);
    return impl_->forward(t);
}
template <typename Dtype>
typename pipeline<Dtype>::blob_map pipeline<Dtype>::forward_cpu(const std::shared_ptr<memory::tensor<Dtype>>& t) { return impl_->forward_cpu(t); }
template <typename Dtype>
typename pipeline<Dtype>::blob_map pipeline<Dtype>::forward_gpu(const std::shared_ptr<memory::tensor<Dtype>>& t) {
    memory::stream_scope scope(impl_->slot_);
    return impl_->forward_gpu(t);
}
template <typename Dtype>
std::shared_ptr<memory::tensor<Dtype>> pipeline<Dtype>::get_featmap(std::string_view name) {
    memory::stream_scope scope(impl_->slot_);
    return impl_->get_featmap(name);
}
template <typename Dtype>
int pipeline<Dtype>::stream_slot() const { return impl_->slot_; }
template <typename Dtype>
void pipeline<Dtype>::synchronize() {
    if (impl_->device() >= 0) EXHIP_FATAL(exhip_sync(memory::device_context(impl_->device(), impl_->slot_)));
}
template <typename Dtype>
bool pipeline<Dtype>::blob_stored(std::string_view name) const { return impl_->blob_stored(name); }
template <typename Dtype>
void pipeline<Dtype>::enable_profiler() { impl_->profile_ = true; }
template <typename Dtype>
void pipeline<Dtype>::disable_profiler() { impl_->profile_ = false; }
template <typename Dtype>
void pipeline<Dtype>::set_fusion(bool on) { impl_->fusion_ = on; }
template <typename Dtype>
bool pipeline<Dtype>::fused() const { return impl_->last_fused_; }
template <typename Dtype>
void pipeline<Dtype>::set_graphs(bool on) { impl_->graphs_ = on; }

template <typename Dtype>
void pipeline<Dtype>::time_fused_span(int first_launch) {
    impl_->span_first_ = first_launch;
    impl_->span_count_ = 0;
}

template <typename Dtype>
float pipeline<Dtype>::last_span(int* launches) {
    if (launches) *launches = impl_->span_launches_;
    float ms = 0.f;
    return recent_spans(&ms, 1) ? ms : 0.f;
}
template <typename Dtype>
int pipeline<Dtype>::recent_spans(float* ms, int capacity) {
    if (!impl_->span_launches_ || capacity <= 0) return 0;
    EXHIP_FATAL(exhip_sync(memory::device_context(impl_->device(), impl_->slot_)));
    const long long have = std::min<long long>(impl_->span_count_, impl::kSpanRing);
    const int n = static_cast<int>(std::min<long long>(have, capacity));
    for (int i = 0; i < n; ++i) {  // oldest of the n first
        void** const ev = impl_->span_ev_[(impl_->span_count_ - n + i) % impl::kSpanRing];
        EXHIP_FATAL(exhip_event_elapsed_ms(ev[0], ev[1], &ms[i]));
    }
    return n;
}
template <typename Dtype>
double pipeline<Dtype>::last_forward_ms() const { return impl_->last_ms_; }
template <typename Dtype>
std::string pipeline<Dtype>::version() { return "1.0.0"; }

template class pipeline<float>;
template class pipeline<double>;
template class pipeline<unsigned short>;

}  // namespace excalibur
}  // namespace glasssix
