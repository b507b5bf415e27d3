// The userdriver of the HIP backend: opens operator lists (builds their operators once), executes them on host
// buffers named by a buffer table, closes them.
//
// Mirrors GpuUserDriver (src/userdriver/gpu/gpu_userdriver.h:34-94, gpu_userdriver.cc:36-248), the implementation of
// the abstract UserDriver (src/userdriver/common/UserDriver.h:52-122) the runtime's dispatchers call: the same six
// entry points, the same two mutexes (one serialising open / execute / close, one guarding the id -> operators map),
// host bytes written into the list's input tensors without blocking, one flush per execution, outputs read back
// blocking.  The reference is a process-wide singleton over device 0; this class is an ordinary object constructed
// for a device, and get_instance() offers the singleton for callers that want the reference's shape.
// OperatorList / ExecutableOperatorList / OperatorListExecuteRequest of the reference's model and runtime layers are
// the plain descriptions of ModelDesc.hpp.
#pragma once

#include <mutex>
#include <tuple>
#include <unordered_map>

#include "HipOpConstructor.hpp"

namespace enn {
namespace ud {
namespace hip {

class HipUserDriver {
public:
    explicit HipUserDriver(uint32_t device_id = 0) : device_id_(device_id) {}
    ~HipUserDriver() { Deinitialize(); }
    HipUserDriver(const HipUserDriver &) = delete;
    HipUserDriver &operator=(const HipUserDriver &) = delete;

    static HipUserDriver &get_instance() {
        static HipUserDriver instance(0);
        return instance;
    }

    EnnReturn Initialize() {
        std::lock_guard<std::mutex> lock_guard_operators_map(mutex_operators_map);
        ud_operators_map.clear();
        compute_library = std::make_shared<HipComputeLibrary>(device_id_);
        if (!compute_library->valid()) {
            compute_library.reset();
            return ENN_RET_FAILED;
        }
        op_constructor = std::make_unique<OperationConstructor>(compute_library);
        op_executor = std::make_unique<OperationExecutor>(compute_library);
        return ENN_RET_SUCCESS;
    }

    EnnReturn OpenSubGraph(const OperatorListDesc &operator_list) {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor);
        if (!compute_library || compute_library->initialize_queue() != Status::SUCCESS) return ENN_RET_FAILED;
        {
            std::lock_guard<std::mutex> lock_guard_map(mutex_operators_map);
            if (ud_operators_map.find(operator_list.id) != ud_operators_map.end()) {
                ERROR_PRINT("HipUserDriver: operator list 0x%llx is open already\n", (unsigned long long)operator_list.id);
                return ENN_RET_FAILED;
            }
        }
        op_constructor->initialize_ud_operators();
        const EnnReturn ret = op_constructor->open_oplist(operator_list);
        if (ret != ENN_RET_SUCCESS) {
            op_constructor->close_oplist(operator_list.id);
            op_constructor->initialize_ud_operators();  // drop the half-built list
            return ret;
        }
        return add_ud_operators(operator_list.id, op_constructor->get_ud_operators(), op_constructor->get_in_tensors(),
                                op_constructor->get_out_tensors());
    }

    // nothing to prepare: buffers are bound at execution (gpu_userdriver.cc:72-76)
    EnnReturn PrepareSubGraph(uint64_t) { return ENN_RET_SUCCESS; }

    EnnReturn ExecuteSubGraph(const OperatorListExecuteRequest &request) {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor);
        UDOperators operators;
        UDTensors in_tensors, out_tensors;
        if (get_ud_operators(request.get_operator_list_id(), operators, in_tensors, out_tensors) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        UDBuffers buffer;
        const BufferTable &buffer_table = request.get_buffer_table();
        if (set_input_data(in_tensors, buffer_table) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        if (op_executor->execute(operators, buffer, buffer_table) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        compute_library->flush();
        return set_output_data(out_tensors, buffer_table);
    }

    EnnReturn CloseSubGraph(uint64_t operator_list_id) {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor);
        EnnReturn ret = ENN_RET_SUCCESS;
        UDOperators operators;
        UDTensors in_tensors, out_tensors;
        if (get_ud_operators(operator_list_id, operators, in_tensors, out_tensors) == ENN_RET_SUCCESS) op_executor->forget(operators);
        if (remove_ud_operators(operator_list_id) != ENN_RET_SUCCESS) ret = ENN_RET_FAILED;
        op_constructor->close_oplist(operator_list_id);
        return ret;
    }

    EnnReturn Deinitialize() {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor);
        std::lock_guard<std::mutex> lock_guard_operators_map(mutex_operators_map);
        if (op_executor)
            for (auto &kv : ud_operators_map) op_executor->forget(std::get<0>(kv.second));
        ud_operators_map.clear();
        op_executor.reset();
        op_constructor.reset();
        compute_library.reset();
        return ENN_RET_SUCCESS;
    }

    // the built list, for tests and harnesses (get_graph_for_TC in the reference, gpu_userdriver.h:49-52)
    EnnReturn get_graph_for_TC(uint64_t id, UDOperators &out_graph) {
        UDTensors in, out;
        return get_ud_operators(id, out_graph, in, out);
    }
    EnnReturn get_ud_operators(uint64_t id, UDOperators &out_ud_operators, UDTensors &in_tensors, UDTensors &out_tensors) {
        std::lock_guard<std::mutex> lock_guard(mutex_operators_map);
        auto it = ud_operators_map.find(id);
        if (it == ud_operators_map.end()) {
            ERROR_PRINT("HipUserDriver: operator list 0x%llx is not open\n", (unsigned long long)id);
            return ENN_RET_FAILED;
        }
        std::tie(out_ud_operators, in_tensors, out_tensors) = it->second;
        return ENN_RET_SUCCESS;
    }

    // Runs the list's operators `times` times on the tensors as they stand (no host copies): what a caller whose
    // data already lives on the device executes, and what a throughput measurement times.  Asynchronous.
    EnnReturn ExecuteOperators(uint64_t operator_list_id, int times = 1) {
        std::lock_guard<std::mutex> lock_guard(mutex_constructor);
        UDOperators operators;
        UDTensors in_tensors, out_tensors;
        if (get_ud_operators(operator_list_id, operators, in_tensors, out_tensors) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        UDBuffers buffer;
        BufferTable none;
        if (op_executor->execute_times(operators, buffer, none, times) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
        compute_library->flush();
        return ENN_RET_SUCCESS;
    }

    const std::shared_ptr<HipComputeLibrary> &computeLibrary() const { return compute_library; }
    OperationExecutor *executor() { return op_executor.get(); }
    OperationConstructor *constructor() { return op_constructor.get(); }

private:
    EnnReturn add_ud_operators(uint64_t id, UDOperators ud_operators, UDTensors in_tensors, UDTensors out_tensors) {
        std::lock_guard<std::mutex> lock_guard(mutex_operators_map);
        if (ud_operators_map.find(id) != ud_operators_map.end()) return ENN_RET_FAILED;
        ud_operators_map[id] = std::make_tuple(ud_operators, in_tensors, out_tensors);
        return ENN_RET_SUCCESS;
    }
    EnnReturn remove_ud_operators(uint64_t id) {
        std::lock_guard<std::mutex> lock_guard(mutex_operators_map);
        return ud_operators_map.erase(id) == 1 ? ENN_RET_SUCCESS : ENN_RET_FAILED;
    }

    // A list input whose buffer index the table holds is written from that host memory, without blocking; a tensor
    // that keeps its data channels-last while the operators compute planar is converted on the way (gpu_userdriver.cc:188-220).
    EnnReturn set_input_data(UDTensors &in_tensors, const BufferTable &buffer_table) {
        for (auto &in : in_tensors) {
            const int32_t in_index = in->get_buffer_index();
            if (!buffer_table.exist(in_index)) continue;
            if (buffer_table[in_index].get_size() < in->getNumOfBytes()) {
                ERROR_PRINT("HipUserDriver: input buffer %d holds %zu bytes, the tensor needs %zu\n", in_index, buffer_table[in_index].get_size(),
                            in->getNumOfBytes());
                return ENN_RET_FAILED;
            }
            const DataOrderChangeType order_type = in->getDataOrder() == DataOrder::NHWC ? DataOrderChangeType::NHWC2NCHW : DataOrderChangeType::OTHER;
            if (in->writeData(const_cast<DataPtr>(buffer_table[in_index].get_addr()), false, order_type) != Status::SUCCESS) return ENN_RET_FAILED;
        }
        return ENN_RET_SUCCESS;
    }

    // blocking, so the host bytes are there when ExecuteSubGraph returns (gpu_userdriver.cc:222-248)
    EnnReturn set_output_data(UDTensors &out_tensors, const BufferTable &buffer_table) {
        for (auto &out : out_tensors) {
            const int32_t out_index = out->get_buffer_index();
            if (!buffer_table.exist(out_index)) continue;
            if (buffer_table[out_index].get_size() < out->getNumOfBytes()) {
                ERROR_PRINT("HipUserDriver: output buffer %d holds %zu bytes, the tensor needs %zu\n", out_index,
                            buffer_table[out_index].get_size(), out->getNumOfBytes());
                return ENN_RET_FAILED;
            }
            // the same constant as on the input side: the reference converts NHWC2NCHW here too
            const DataOrderChangeType order_type = out->getDataOrder() == DataOrder::NHWC ? DataOrderChangeType::NHWC2NCHW : DataOrderChangeType::OTHER;
            if (out->readData(const_cast<DataPtr>(buffer_table[out_index].get_addr()), true, order_type) != Status::SUCCESS) return ENN_RET_FAILED;
        }
        return ENN_RET_SUCCESS;
    }

    uint32_t device_id_;
    std::shared_ptr<HipComputeLibrary> compute_library;
    std::unique_ptr<OperationConstructor> op_constructor;
    std::unique_ptr<OperationExecutor> op_executor;
    std::mutex mutex_constructor;
    std::mutex mutex_operators_map;
    std::unordered_map<uint64_t, std::tuple<UDOperators, UDTensors, UDTensors>> ud_operators_map;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
