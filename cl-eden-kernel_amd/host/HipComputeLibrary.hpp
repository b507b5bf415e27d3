// The compute library of the HIP userdriver backend: owns the device runtime (stream, buffer manager), makes the
// tensors the operator constructor asks for, and makes the operators.  It is what the reference's userdriver hands
// to its constructor and executor (src/userdriver/gpu/gpu_userdriver.cc:42-54 builds a CLComputeLibrary(0) and passes
// it to both), so swapping the OpenCL backend for this one is swapping that one object.
//
// Mirrors CLComputeLibrary (src/userdriver/gpu/common/CLComputeLibrary.hpp:23-107, CLComputeLibrary.cpp:10-186):
// the IComputeLibrary virtuals, initialize_queue(), tensor_type_2_data_type() and one create<Operator>(precision)
// per operator this backend has.  Texture storage and CPU-side tensors (use_cpu_for_gpu) do not exist here and give
// a null tensor.
#pragma once

#include <map>
#include <memory>

#include "HipOperators.hpp"
#include "IComputeLibrary.hpp"

namespace enn {
namespace ud {
namespace hip {

#define HIP_OP_CREATOR(CLASS_NAME, OP_NAME) \
    std::shared_ptr<CLASS_NAME> create##OP_NAME(const PrecisionType &precision) { return std::make_shared<CLASS_NAME>(runtime_, precision); }

class HipComputeLibrary : public IComputeLibrary {
public:
    explicit HipComputeLibrary(const uint32_t &device_id) : runtime_(std::make_shared<HipRuntime>()) {
        initialized_ = runtime_->initialize(device_id) == Status::SUCCESS;
    }
    ~HipComputeLibrary() override = default;

    // false when the device could not be initialised (no gfx950 device, library missing): nothing will work then
    bool valid() const { return initialized_; }

    void assignBuffers() override { (void)runtime_->assignBufferPool(); }
    void flush() override { runtime_->flush(); }
    void synchronize() override { (void)runtime_->synchronize(); }
    Status setPublicKernels(NnApiType, StorageType storage_type) override {
        // kernels are compiled into the library; only buffer storage exists
        return storage_type == StorageType::BUFFER ? Status::SUCCESS : Status::FAILURE;
    }

    // a list that could not be built: forget the pooled buffers its tensors asked for
    void abandonBuffers() { (void)runtime_->abandonPendingBuffers(); }

    Status initialize_queue() {
        CHECK_EXPR_RETURN_FAILURE(initialized_, "HipComputeLibrary: the device was not initialised");
        return runtime_->initializeQueue();
    }

    std::shared_ptr<ITensor> create_tensor(const TFlite::TensorType &type, const PrecisionType &precision, const NDims &ndim,
                                           const int32_t &buffer_index = UNDEFINED, const BufferType &buffer_type = BufferType::DEDICATED,
                                           const bool &use_cpu_for_gpu = false, const StorageType &storage_type = StorageType::BUFFER,
                                           const DataOrder &data_order = DataOrder::NCHW, const float &scale = 1.0f,
                                           const int32_t &zero_point = 0) override {
        if (use_cpu_for_gpu || storage_type != StorageType::BUFFER) {
            ERROR_PRINT("HipComputeLibrary::create_tensor: CPU-side tensors and texture storage do not exist on this backend\n");
            return nullptr;
        }
        const DataType data_type = tensor_type_2_data_type(type);
        if (data_type == DataType::SIZE) {
            ERROR_PRINT("HipComputeLibrary::create_tensor: tensor type %d has no device type\n", (int)type);
            return nullptr;
        }
        auto tensor = std::make_shared<HipTensor>(runtime_, precision, data_type, ndim, data_order, scale, zero_point, buffer_type,
                                                  storage_type, static_cast<uint32_t>(type), buffer_index);
        if (tensor->getBuffer() == nullptr) return nullptr;
        return tensor;
    }

    std::shared_ptr<ITensor> create_and_copy_tensor(const TFlite::TensorType &type, DataPtr &data, const PrecisionType &precision,
                                                    const NDims &ndim, const int32_t &buffer_index = UNDEFINED,
                                                    const BufferType &buffer_type = BufferType::DEDICATED,
                                                    const bool &use_cpu_for_gpu = false,
                                                    const StorageType &storage_type = StorageType::BUFFER,
                                                    const DataOrder &data_order = DataOrder::NCHW, const float &scale = 1.0f,
                                                    const int32_t &zero_point = 0) override {
        if (use_cpu_for_gpu || storage_type != StorageType::BUFFER || data == nullptr) {
            ERROR_PRINT("HipComputeLibrary::create_and_copy_tensor: no data, or a storage this backend does not have\n");
            return nullptr;
        }
        switch (type) {
            case TFlite::TensorType_FLOAT32: return copied(type, reinterpret_cast<float *>(data), precision, ndim, buffer_index, buffer_type, data_order, scale, zero_point);
            case TFlite::TensorType_INT8: return copied(type, reinterpret_cast<int8_t *>(data), precision, ndim, buffer_index, buffer_type, data_order, scale, zero_point);
            case TFlite::TensorType_INT32: return copied(type, reinterpret_cast<int32_t *>(data), precision, ndim, buffer_index, buffer_type, data_order, scale, zero_point);
            case TFlite::TensorType_UINT8: return copied(type, reinterpret_cast<uint8_t *>(data), precision, ndim, buffer_index, buffer_type, data_order, scale, zero_point);
            default: ERROR_PRINT("HipComputeLibrary::create_and_copy_tensor: tensor type %d is not offered\n", (int)type);
        }
        return nullptr;
    }

    // a tensor of the same type, precision, shape and buffer index with storage of its own (CLComputeLibrary.cpp:183-186)
    std::shared_ptr<ITensor> clone_tensor(const std::shared_ptr<ITensor> base) override {
        return create_tensor((TFlite::TensorType)base->get_buffer_type(), base->getPrecisionType(), base->getDims(), base->get_buffer_index());
    }

    DataType tensor_type_2_data_type(const TFlite::TensorType &type) {
        const auto it = tensor_type_2_data_type_map_.find(type);
        return it == tensor_type_2_data_type_map_.end() ? DataType::SIZE : it->second;
    }

    HIP_OP_CREATOR(HipAdd, Add);
    HIP_OP_CREATOR(HipAveragepool, Averagepool);
    HIP_OP_CREATOR(HipConvolution, Convolution);
    HIP_OP_CREATOR(HipDeconvolution, Deconvolution);
    HIP_OP_CREATOR(HipDepthwiseConvolution, DepthwiseConvolution);
    HIP_OP_CREATOR(HipFullyConnected, FullyConnected);

    // the runtime this library made its tensors and operators on (the executor records and replays on its stream)
    const std::shared_ptr<HipRuntime> &runtime() const { return runtime_; }

private:
    template <typename T>
    std::shared_ptr<ITensor> copied(const TFlite::TensorType &type, T *data, const PrecisionType &precision, const NDims &ndim,
                                    const int32_t buffer_index, const BufferType &buffer_type, const DataOrder &data_order,
                                    const float &scale, const int32_t &zero_point) {
        auto tensor = std::make_shared<HipTensor>(runtime_, precision, data, ndim, data_order, scale, zero_point, buffer_type,
                                                  StorageType::BUFFER, static_cast<uint32_t>(type), buffer_index);
        if (tensor->getNumOfBytes() != 0 && tensor->getDataPtr() == nullptr) return nullptr;
        return tensor;
    }

    std::shared_ptr<HipRuntime> runtime_;
    bool initialized_ = false;
    std::map<TFlite::TensorType, DataType> tensor_type_2_data_type_map_ = {
        {TFlite::TensorType_FLOAT64, DataType::FLOAT}, {TFlite::TensorType_FLOAT32, DataType::FLOAT},
        {TFlite::TensorType_FLOAT16, DataType::HALF},  {TFlite::TensorType_INT32, DataType::INT32},
        {TFlite::TensorType_INT8, DataType::INT8},     {TFlite::TensorType_UINT8, DataType::UINT8},
        {TFlite::TensorType_BOOL, DataType::BOOL},     {TFlite::TensorType_INT16, DataType::INT16},
    };
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
