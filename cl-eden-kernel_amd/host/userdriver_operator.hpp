// Operator-list wrappers of the userdriver protocol: an ordered list of
// type-erased operators that the executor runs one after the other
// (reference: src/userdriver/common/operator_interfaces/userdriver_operator.h:31-142,
// executed by src/userdriver/gpu/gpu_op_executor.cc:56-103).
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "ITensor.hpp"

namespace enn {
namespace ud {

typedef enum { ENN_RET_SUCCESS = 0, ENN_RET_FAILED = 1 } EnnReturn;

class UDBuffer {
public:
    std::vector<std::shared_ptr<ITensor>> in, out, data;
    void set_id(uint64_t id) { execution_id = id; }
    uint64_t get_id() { return execution_id; }

private:
    uint64_t execution_id = 0;
};

class UDOperator {
public:
    UDOperator(const std::string name, const uint64_t id, const std::vector<std::shared_ptr<ITensor>> &in,
               const std::vector<std::shared_ptr<ITensor>> &out, const std::vector<std::shared_ptr<ITensor>> &data)
        : name_(name), id_(id), in_(in), out_(out), data_(data) {}
    virtual ~UDOperator() {}
    virtual EnnReturn execute(const std::shared_ptr<UDBuffer> &buffer) = 0;
    virtual EnnReturn release() = 0;
    // Whether execute() does nothing but enqueue kernels whose arguments follow from the operator's tensors (their
    // device addresses, scales and zero points): such an execution can be recorded once and replayed.  Not part of the
    // reference's UDOperator; the list executor of this backend asks it.
    virtual bool replayable() const { return false; }
    // The lane of its list this operator belongs to (0 unless the constructor cut the list's images into lanes, each
    // with operators of its own that share nothing with the other lanes' but read-only parameters).  Not part of the
    // reference's UDOperator either.
    int lane() const { return lane_; }
    void setLane(int lane) { lane_ = lane; }
    std::string getName() { return name_; }
    uint64_t getId() { return id_; }
    std::vector<std::shared_ptr<ITensor>> getInTensors() { return in_; }
    std::vector<std::shared_ptr<ITensor>> getOutTensors() { return out_; }
    std::vector<std::shared_ptr<ITensor>> getDataTensors() { return data_; }
    // the same lists without a copy, for the executor's per-execution walk over every tensor of every operator
    const std::vector<std::shared_ptr<ITensor>> &inTensors() const { return in_; }
    const std::vector<std::shared_ptr<ITensor>> &outTensors() const { return out_; }

protected:
    std::string name_;
    uint64_t id_;
    std::vector<std::shared_ptr<ITensor>> in_, out_, data_;
    int lane_ = 0;
};

// The reference stamps execute() per operator type with a macro; the operators of
// this backend all take no arguments, so one template body serves them.
template <typename T>
class EnnUDOperator : public UDOperator {
public:
    EnnUDOperator(const std::string name, const uint64_t id, const std::vector<std::shared_ptr<ITensor>> &in,
                  const std::vector<std::shared_ptr<ITensor>> &out, const std::vector<std::shared_ptr<ITensor>> &data,
                  const std::shared_ptr<T> &op)
        : UDOperator(name, id, in, out, data), op_(op) {}
    EnnReturn execute(const std::shared_ptr<UDBuffer> &) override {
        return op_->execute() == Status::SUCCESS ? ENN_RET_SUCCESS : ENN_RET_FAILED;
    }
    EnnReturn release() override { return op_->release() == Status::SUCCESS ? ENN_RET_SUCCESS : ENN_RET_FAILED; }
    bool replayable() const override { return op_->launchesOnly(); }
    std::shared_ptr<T> getOp() { return op_; }

private:
    std::shared_ptr<T> op_;
};

using UDOperators = std::shared_ptr<std::vector<std::shared_ptr<UDOperator>>>;
using UDBuffers = std::vector<std::shared_ptr<UDBuffer>>;
using UDTensors = std::vector<std::shared_ptr<ITensor>>;

}  // namespace ud
}  // namespace enn
