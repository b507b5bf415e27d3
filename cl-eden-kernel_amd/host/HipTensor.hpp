// Tensor of the HIP userdriver backend: dims, data order, element type and the
// per-tensor quantization parameters (scale, zero point) the operators read at
// execute time, over a HipBuffer.
//
// Mirrors CLTensor (src/userdriver/gpu/common/CLTensor.hpp:40-152 constructors:
// a shape-only tensor is a run-time input/output, a tensor built from host data is
// a constant; CLTensor.cpp:181-225 layout conversion; destructor :268-276).
#pragma once

#include <cstring>
#include <string>
#include <typeinfo>
#include <vector>

#include "HipRuntime.hpp"
#include "ITensor.hpp"

namespace enn {
namespace ud {
namespace hip {

template <typename T> struct data_type_of;
template <> struct data_type_of<uint8_t> { static constexpr DataType value = DataType::UINT8; };
template <> struct data_type_of<int8_t> { static constexpr DataType value = DataType::INT8; };
template <> struct data_type_of<int32_t> { static constexpr DataType value = DataType::INT32; };
template <> struct data_type_of<float> { static constexpr DataType value = DataType::FLOAT; };

class HipTensor : public ITensor {
public:
    // run-time tensor (input, output, intermediate)
    HipTensor(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision, const DataType &data_type,
              const Dim4 &dim, const DataOrder &data_order = DataOrder::NCHW, const float &scale = 1.0f,
              const int32_t &zero_point = 0, const BufferType &buffer_type = BufferType::DEDICATED,
              const StorageType &storage_type = StorageType::BUFFER, const uint32_t buffer_data_type = 0,
              const int32_t buffer_index = UNDEFINED)
        : runtime_(runtime), precision_(precision), data_type_(data_type), dims_(dim), vdims_({dim.n, dim.c, dim.h, dim.w}),
          order_(data_order), scale_(scale), zero_point_(zero_point), buffer_type_(buffer_type), storage_type_(storage_type),
          buffer_data_type_(buffer_data_type), buffer_index_(buffer_index), is_const_(false) {
        buf_ = runtime_->getBuffer(precision_, data_type_, dims_, buffer_type_, storage_type_);
    }

    // the same from a shape of any rank up to four (CLTensor.cpp:29-47): getDims() keeps the rank, getDim() is the
    // shape padded with ones
    HipTensor(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision, const DataType &data_type,
              const NDims &ndim, const DataOrder &data_order = DataOrder::NCHW, const float &scale = 1.0f,
              const int32_t &zero_point = 0, const BufferType &buffer_type = BufferType::DEDICATED,
              const StorageType &storage_type = StorageType::BUFFER, const uint32_t buffer_data_type = 0,
              const int32_t buffer_index = UNDEFINED)
        : HipTensor(runtime, precision, data_type, extendToDim4(ndim), data_order, scale, zero_point, buffer_type, storage_type,
                    buffer_data_type, buffer_index) {
        vdims_ = ndim;
    }

    // constant tensor (weights, bias): uploaded at construction
    template <typename T>
    HipTensor(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision, T *data, const Dim4 &dims,
              const DataOrder &data_order = DataOrder::NCHW, const float &scale = 1.0f, const int32_t &zero_point = 0,
              const BufferType &buffer_type = BufferType::DEDICATED, const StorageType &storage_type = StorageType::BUFFER,
              const uint32_t buffer_data_type = 0, const int32_t buffer_index = UNDEFINED)
        : runtime_(runtime), precision_(precision), data_type_(data_type_of<typename std::remove_const<T>::type>::value),
          dims_(dims), vdims_({dims.n, dims.c, dims.h, dims.w}), order_(data_order), scale_(scale), zero_point_(zero_point),
          buffer_type_(buffer_type), storage_type_(storage_type), buffer_data_type_(buffer_data_type),
          buffer_index_(buffer_index), is_const_(true) {
        buf_ = std::make_shared<HipBuffer>(getNumOfBytes());
        buf_->assignBuffer(runtime_->allocBuffer(getNumOfBytes(), false));
        if (getNumOfBytes())
            (void)runtime_->writeBuffer(buf_->getDataPtr(), data, getTypeBytes(data_type_, precision_), getTotalSizeFromDims(),
                                        true);
    }

    template <typename T>
    HipTensor(const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision, T *data, const NDims &ndim,
              const DataOrder &data_order = DataOrder::NCHW, const float &scale = 1.0f, const int32_t &zero_point = 0,
              const BufferType &buffer_type = BufferType::DEDICATED, const StorageType &storage_type = StorageType::BUFFER,
              const uint32_t buffer_data_type = 0, const int32_t buffer_index = UNDEFINED)
        : HipTensor(runtime, precision, data, extendToDim4(ndim), data_order, scale, zero_point, buffer_type, storage_type,
                    buffer_data_type, buffer_index) {
        vdims_ = ndim;
    }

    // A tensor that is never stored: shape and quantization parameters of a value that only exists inside a fused
    // launch (the operators on either side of it still read its scale and zero point).  No device memory, no pool
    // request; reconfigureDimsAndBuffer() gives it a buffer of its own should it have to be stored after all.
    struct NoStorage {};
    HipTensor(NoStorage, const std::shared_ptr<HipRuntime> runtime, const PrecisionType &precision, const DataType &data_type,
              const NDims &ndim, const DataOrder &data_order, const float &scale, const int32_t &zero_point, const uint32_t buffer_data_type,
              const int32_t buffer_index)
        : runtime_(runtime), precision_(precision), data_type_(data_type), dims_(extendToDim4(ndim)), vdims_(ndim), order_(data_order),
          scale_(scale), zero_point_(zero_point), buffer_type_(BufferType::DEDICATED), storage_type_(StorageType::BUFFER),
          buffer_data_type_(buffer_data_type), buffer_index_(buffer_index), is_const_(false) {}
    bool hasStorage() { return whole_ ? whole_->hasStorage() : (buf_ != nullptr); }

    // A view: `images` of the leading dimension of `whole`, starting at `first_image`, as a tensor of its own shape.
    // It owns no storage (its address follows the whole tensor's, also when that is assigned or moved later) and
    // reads scale and zero point from the whole tensor, which is the one the owner of the list talks to.  The lanes of
    // an operator list see their share of the list's inputs and outputs through such views.  No counterpart in the
    // reference, whose operators always work on whole tensors.
    HipTensor(const std::shared_ptr<HipTensor> &whole, uint32_t first_image, uint32_t images)
        : runtime_(whole->runtime_), precision_(whole->precision_), data_type_(whole->data_type_), dims_(whole->dims_),
          vdims_(whole->vdims_), order_(whole->order_), scale_(whole->scale_), zero_point_(whole->zero_point_),
          buffer_type_(whole->buffer_type_), storage_type_(whole->storage_type_), buffer_data_type_(whole->buffer_data_type_),
          buffer_index_(whole->buffer_index_), is_const_(whole->is_const_), whole_(whole) {
        const uint32_t all = vdims_.empty() ? 1 : vdims_[0];
        const size_t per_image = all ? whole->getNumOfBytes() / all : 0;
        view_offset_ = per_image * first_image;
        if (!vdims_.empty()) vdims_[0] = images;
        dims_ = extendToDim4(vdims_);
    }
    bool isView() const { return whole_ != nullptr; }

    // The device bytes of this tensor, whose shape reads (n, c, h, w), are stored channels-last ([n][h][w][c]).  The
    // operator constructor stores the feature maps inside a planar operator list that way: the kernels of this backend
    // work on channels-last data, and a planar tensor costs every operator a transposition on either side.  Operators
    // ask the tensors they are given; what the owner of the list reads and writes (its inputs and outputs) stays
    // planar.  No counterpart in the reference, whose kernels are planar.
    void storeChannelsLast(bool on) { channels_last_ = on; }
    bool storedChannelsLast() const { return whole_ ? whole_->storedChannelsLast() : channels_last_; }

    ~HipTensor() override {
        if (buf_ && buf_.use_count() == 1 && buf_->getDataPtr() != nullptr) (void)runtime_->releaseBuffer(buf_);
    }

    size_t getNumOfBytes() override { return getTypeBytes(data_type_, precision_) * (size_t)getTotalSizeFromDims(); }
    DataType getDataType() override { return data_type_; }
    PrecisionType getPrecisionType() override { return precision_; }
    const Dim4 &getDim() override { return dims_; }
    const NDims &getDims() override { return vdims_; }
    uint32_t getDims(const int32_t &idx) override { return idx >= 0 && (size_t)idx < vdims_.size() ? vdims_[idx] : 0; }
    uint32_t getNumOfDims() override { return (uint32_t)vdims_.size(); }
    uint32_t getTotalSizeFromDims() override { return getTensorSizeFromDims(vdims_); }
    DataOrder getDataOrder() override { return order_; }
    float getScale() override { return whole_ ? whole_->getScale() : scale_; }
    int32_t getZeroPoint() override { return whole_ ? whole_->getZeroPoint() : zero_point_; }
    void setZeroPoint(int32_t zero_point) override {
        if (whole_) return whole_->setZeroPoint(zero_point);
        zero_point_ = zero_point;
    }
    void setScale(float scale) override {
        if (whole_) return whole_->setScale(scale);
        scale_ = scale;
    }
    void set_buffer_index(int32_t index) override { buffer_index_ = index; }
    int32_t get_buffer_index() override { return buffer_index_; }
    void set_buffer_type(uint32_t type) override { buffer_data_type_ = type; }
    uint32_t get_buffer_type() override { return buffer_data_type_; }
    void set_buffer_ptr(void *addr) override { raw_buffer = addr; }
    bool is_const() override { return is_const_; }

    void *getDataPtr() {
        if (whole_) {
            void *base = whole_->getDataPtr();
            return base ? static_cast<char *>(base) + view_offset_ : nullptr;
        }
        return buf_ ? buf_->getDataPtr() : nullptr;
    }
    std::shared_ptr<HipBuffer> getBuffer() { return buf_; }
    BufferType getBufferType() const { return buffer_type_; }

    // Host -> device, converting the element order on the way when asked to
    // (the reference reorders host NHWC data into its planar device tensors).
    Status writeData(DataPtr data, bool blocking = true, DataOrderChangeType type = DataOrderChangeType::OTHER) override {
        CHECK_EXPR_RETURN_FAILURE(getDataPtr() != nullptr || getNumOfBytes() == 0, "HipTensor::writeData: no device buffer");
        if (getNumOfBytes() == 0) return Status::SUCCESS;
        if (type == DataOrderChangeType::OTHER)
            return runtime_->writeBuffer(getDataPtr(), data, getTypeBytes(data_type_, precision_), getTotalSizeFromDims(),
                                         blocking);
        CHECK_EXPR_RETURN_FAILURE(getTypeBytes(data_type_, precision_) == 1, "layout conversion is byte tensors only");
        CHECK_EXPR_RETURN_FAILURE(type == DataOrderChangeType::NHWC2NCHW || type == DataOrderChangeType::NCHW2NHWC,
                                  "HipTensor::writeData: unsupported order change");
        void *tmp = runtime_->allocBuffer(getNumOfBytes(), false);
        CHECK_EXPR_RETURN_FAILURE(tmp != nullptr, "HipTensor::writeData: staging allocation failed");
        Status st = runtime_->writeBuffer(tmp, data, 1, getTotalSizeFromDims(), true);
        if (st == Status::SUCCESS)
            st = type == DataOrderChangeType::NHWC2NCHW ? runtime_->NHWC2NCHW(tmp, getDataPtr(), dims_)
                                                        : runtime_->NCHW2NHWC(tmp, getDataPtr(), dims_);
        auto holder = std::make_shared<HipBuffer>(getNumOfBytes());
        holder->assignBuffer(tmp);
        (void)runtime_->releaseBuffer(holder);  // synchronises first
        return st;
    }

    // Device -> host.  blocking == false only queues the copy: the host bytes are defined after the runtime's
    // synchronize() (or a later blocking call on the same runtime), as with clEnqueueReadBuffer(CL_FALSE); reads that
    // change the element order always block.
    Status readData(DataPtr data, bool blocking = true, DataOrderChangeType type = DataOrderChangeType::OTHER,
                    void *event = nullptr) override {
        (void)event;
        if (getNumOfBytes() == 0) return Status::SUCCESS;
        CHECK_EXPR_RETURN_FAILURE(getDataPtr() != nullptr, "HipTensor::readData: no device buffer");
        if (type == DataOrderChangeType::OTHER)
            return runtime_->readBuffer(data, getDataPtr(), getTypeBytes(data_type_, precision_), getTotalSizeFromDims(), blocking);
        CHECK_EXPR_RETURN_FAILURE(getTypeBytes(data_type_, precision_) == 1, "layout conversion is byte tensors only");
        CHECK_EXPR_RETURN_FAILURE(type == DataOrderChangeType::NHWC2NCHW || type == DataOrderChangeType::NCHW2NHWC,
                                  "HipTensor::readData: unsupported order change");
        void *tmp = runtime_->allocBuffer(getNumOfBytes(), false);
        CHECK_EXPR_RETURN_FAILURE(tmp != nullptr, "HipTensor::readData: staging allocation failed");
        Status st = type == DataOrderChangeType::NHWC2NCHW ? runtime_->NHWC2NCHW(getDataPtr(), tmp, dims_)
                                                           : runtime_->NCHW2NHWC(getDataPtr(), tmp, dims_);
        if (st == Status::SUCCESS) st = runtime_->readBuffer(data, tmp, 1, getTotalSizeFromDims(), true);
        auto holder = std::make_shared<HipBuffer>(getNumOfBytes());
        holder->assignBuffer(tmp);
        (void)runtime_->releaseBuffer(holder);
        return st;
    }

    Status reconfigure(const PrecisionType &precision, const DataOrder &order, const Dim4 &dims, const float &scale,
                       const int32_t &offset) override {
        precision_ = precision;
        order_ = order;
        scale_ = scale;
        zero_point_ = offset;
        return reconfigureDim(dims);
    }
    Status reconfigure(const PrecisionType &precision, const DataOrder &order, const NDims &ndim, const float &scale,
                       const int32_t &offset) override {
        precision_ = precision;
        order_ = order;
        scale_ = scale;
        zero_point_ = offset;
        return reconfigureDims(ndim);
    }
    Status reconfigureDim(const Dim4 &dims) override {
        dims_ = dims;
        vdims_ = {dims.n, dims.c, dims.h, dims.w};
        return Status::SUCCESS;
    }
    Status reconfigureDims(const NDims &ndim) override {
        vdims_ = ndim;
        dims_ = extendToDim4(ndim);
        return Status::SUCCESS;
    }
    Status reconfigureDimAndBuffer(const Dim4 &dims) override {
        reconfigureDim(dims);
        return growBuffer();
    }
    Status reconfigureDimsAndBuffer(const NDims &dims) override {
        reconfigureDims(dims);
        return growBuffer();
    }
    Status reorder(const DataOrder &order) override {
        order_ = order;
        return Status::SUCCESS;
    }
    void queryTensorInfo() override {
        std::fprintf(stderr, "HipTensor dims [%u %u %u %u] order %d type %d scale %g zp %d const %d\n", dims_.n, dims_.c, dims_.h,
                     dims_.w, (int)order_, (int)data_type_, (double)scale_, zero_point_, (int)is_const_);
    }
    void dumpTensorData(std::string file_name) override {
        std::vector<char> host(getNumOfBytes());
        if (readData(host.data()) != Status::SUCCESS) return;
        if (FILE *f = std::fopen(file_name.c_str(), "wb")) {
            std::fwrite(host.data(), 1, host.size(), f);
            std::fclose(f);
        }
    }
    Status resetInterBuffer() override { return whole_ || !buf_ ? Status::SUCCESS : runtime_->resetInterBuffer(buf_); }

private:
    Status growBuffer() {
        CHECK_EXPR_RETURN_FAILURE(!whole_, "HipTensor: a view cannot be given storage of its own");
        if (buf_ && buf_->getDataPtr() && buf_->getBytes() >= getNumOfBytes()) return Status::SUCCESS;
        if (buf_ && buf_->getDataPtr()) (void)runtime_->releaseBuffer(buf_);
        buf_ = std::make_shared<HipBuffer>(getNumOfBytes());
        buf_->assignBuffer(runtime_->allocBuffer(getNumOfBytes(), true));
        return buf_->getDataPtr() || getNumOfBytes() == 0 ? Status::SUCCESS : Status::FAILURE;
    }

    std::shared_ptr<HipRuntime> runtime_;
    PrecisionType precision_;
    DataType data_type_;
    Dim4 dims_;
    NDims vdims_;
    DataOrder order_;
    float scale_;
    int32_t zero_point_;
    BufferType buffer_type_;
    StorageType storage_type_;
    uint32_t buffer_data_type_;
    int32_t buffer_index_;
    bool is_const_;
    bool channels_last_ = false;
    std::shared_ptr<HipBuffer> buf_;
    std::shared_ptr<HipTensor> whole_;  // views only
    size_t view_offset_ = 0;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
