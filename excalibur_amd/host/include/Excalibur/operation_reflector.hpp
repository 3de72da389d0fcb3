// Name -> factory registry of operators with the reference's macros
// (include/Excalibur/operation_reflector.hpp:17-93): REGISTE(CLASS) creates static register_action
// objects that register "CLASS" at library load; create_object() resolves a topology type by
// "operation_" + lower-cased type and is fatal for unknown types.
#pragma once
#include <algorithm>
#include <functional>
#include <map>

#include "operation.hpp"

namespace glasssix {
namespace excalibur {

template <typename Dtype>
class operation_reflector {
public:
    using factory = std::function<std::shared_ptr<operation<Dtype>>(const operation_param&)>;

    static operation_reflector& instance() {
        static operation_reflector self;
        return self;
    }

    std::shared_ptr<operation<Dtype>> create_object(const operation_param& param) {
        std::string key = param.type_;
        std::transform(key.begin(), key.end(), key.begin(), ::tolower);
        auto it = object_map_.find("operation_" + key);
        if (it == object_map_.end()) {
            LOG(FATAL) << "Un-suppoted operation type: " << param.type_ << ". ";
            return nullptr;
        }
        return it->second(param);
    }

    void registe(const std::string& class_name, factory&& generator) { object_map_[class_name] = std::move(generator); }
    bool has(const std::string& class_name) const { return object_map_.count(class_name) != 0; }
    std::vector<std::string> registered() const {
        std::vector<std::string> names;
        for (auto& kv : object_map_) names.push_back(kv.first);
        return names;
    }

private:
    std::map<std::string, factory> object_map_;
};

template <typename Dtype>
class register_action {
public:
    register_action(const std::string& class_name, typename operation_reflector<Dtype>::factory&& generator) {
        operation_reflector<Dtype>::instance().registe(class_name, std::move(generator));
    }
};

// The three element types of the reference (operation_reflector.hpp:55-93). Operators of a pipeline<double> can be
// created and loaded; their forward is NOT_IMPLEMENTED, as the reference's forward_*_d64 defaults are
// (include/Excalibur/operation.hpp:185-201).
#define INSTANCE_CLASS(CLASS_NAME)     \
    template class CLASS_NAME<float>;  \
    template class CLASS_NAME<double>; \
    template class CLASS_NAME<unsigned short>;

#define REGISTE_SHORT(CLASS_NAME)                                                                  \
    register_action<unsigned short> g_us_register_action_##CLASS_NAME(                             \
        #CLASS_NAME, [](const operation_param& param) -> std::shared_ptr<operation<unsigned short>> { \
            return std::make_shared<CLASS_NAME<unsigned short>>(param);                            \
        });
#define REGISTE_FLOAT(CLASS_NAME)                                                    \
    register_action<float> g_f_register_action_##CLASS_NAME(                         \
        #CLASS_NAME, [](const operation_param& param) -> std::shared_ptr<operation<float>> { \
            return std::make_shared<CLASS_NAME<float>>(param);                       \
        });
#define REGISTE_DOUBLE(CLASS_NAME)                                                     \
    register_action<double> g_d_register_action_##CLASS_NAME(                         \
        #CLASS_NAME, [](const operation_param& param) -> std::shared_ptr<operation<double>> { \
            return std::make_shared<CLASS_NAME<double>>(param);                       \
        });
#define REGISTE(CLASS_NAME)   \
    REGISTE_SHORT(CLASS_NAME) \
    REGISTE_FLOAT(CLASS_NAME) \
    REGISTE_DOUBLE(CLASS_NAME)

// The reference's way of giving an operator without device code a forward_gpu_f32 that stops
// (include/Excalibur/operation_reflector.hpp:95-100): kept so that operator sources written against it compile.
#define STUB_GPU(Operation_Name)                                                                          \
    template <typename Dtype>                                                                            \
    void Operation_Name<Dtype>::forward_gpu_f32(const std::vector<std::shared_ptr<memory::tensor<float>>>& bottoms, \
                                                std::vector<std::shared_ptr<memory::tensor<float>>>& tops) {        \
        NO_GPU;                                                                                          \
    }

}  // namespace excalibur
}  // namespace glasssix
