// What the runtime above the userdriver hands it: the description of an operator list (the model graph's operators,
// feature maps and parameters), the table of host buffers of one execution, and the execute request.
//
// The reference passes model::component::OperatorList / Operator / FeatureMap / Parameter objects built by its model
// loader (src/model/component/operator/operator.hpp, tensor/feature_map.hpp, tensor/parameter.hpp), a
// model::memory::BufferTable (src/model/memory/buffer_table.hpp:19-44: buffer index -> host address and size) and a
// runtime::OperatorListExecuteRequest (operator list id, executable id, buffer table; read at
// src/userdriver/gpu/gpu_userdriver.cc:82-101).  The loader is not part of this backend, so the same information is
// carried by plain structs: OperatorListDesc / OperatorDesc / TensorDesc, and small classes with the accessors the
// userdriver calls.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "Common.hpp"
#include "TFliteSchema.hpp"

namespace enn {
namespace ud {
namespace hip {

// An edge of the model graph: a feature map (is_const false, buffer_index names its storage) or a
// parameter (is_const true, data points at the host bytes).
struct TensorDesc {
    std::string name;
    NDims shape;
    TFlite::TensorType data_type = TFlite::TensorType_UINT8;
    float scale = 1.0f;
    int32_t zero_point = 0;
    bool is_const = false;
    const void *data = nullptr;
    int32_t buffer_index = UNDEFINED;
    std::vector<float> per_channel_scales;  // symmetric per-channel quantization of a filter; empty otherwise
};

struct OperatorDesc {
    std::string name;
    uint64_t id = 0;
    TFlite::BuiltinOperator code = TFlite::BuiltinOperator_CONV_2D;
    std::vector<std::shared_ptr<TensorDesc>> in_tensors, out_tensors;
    std::shared_ptr<void> option;  // the TFlite::*Options struct that belongs to `code`
};

struct OperatorListDesc {
    uint64_t id = 0;
    TFlite::LegacyModel legacy_model = TFlite::LegacyModel_TENSORFLOW_NHWC;
    std::vector<OperatorDesc> operators;
};

// host memory of one buffer index for one execution
class AllocatedBuffer {
public:
    AllocatedBuffer() = default;
    AllocatedBuffer(const void *addr, size_t size) : addr_(addr), size_(size) {}
    const void *get_addr() const { return addr_; }
    size_t get_size() const { return size_; }

private:
    const void *addr_ = nullptr;
    size_t size_ = 0;
};

class BufferTable {
public:
    const AllocatedBuffer &operator[](int32_t index) const { return buffer_map_.at(index); }
    bool exist(int32_t index) const { return buffer_map_.find(index) != buffer_map_.end(); }
    void add(int32_t index, const void *addr, size_t size) { buffer_map_.insert({index, AllocatedBuffer(addr, size)}); }

private:
    std::map<int32_t, AllocatedBuffer> buffer_map_;
};

class OperatorListExecuteRequest {
public:
    OperatorListExecuteRequest(uint64_t operator_list_id, uint64_t executable_id, const BufferTable &table)
        : operator_list_id_(operator_list_id), executable_id_(executable_id), buffer_table_(table) {}
    uint64_t get_operator_list_id() const { return operator_list_id_; }
    uint64_t get_executable_operator_list_id() const { return executable_id_; }
    const BufferTable &get_buffer_table() const { return buffer_table_; }

private:
    uint64_t operator_list_id_, executable_id_;
    BufferTable buffer_table_;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
