// C ABI of the userdriver level (include/eden_ud.h) over the C++ host classes: HipUserDriver and the plain model
// descriptions.  Built as libedenud.so, linked against libedenhip.so.
#include "eden_ud.h"

#include <cstdarg>
#include <cstring>
#include <exception>
#include <new>

#include "HipUserDriver.hpp"

using namespace enn::ud;
using namespace enn::ud::hip;

namespace {

thread_local char g_error[512] = "";

int fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return 1;
}

// the last error of the layer below, when it left one
int fail_below(const char *what) {
    const char *below = eh_last_error();
    return fail("%s%s%s", what, below && *below ? ": " : "", below ? below : "");
}

template <typename F>
int guarded(F &&body) {
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return fail("out of host memory");
    } catch (const std::exception &e) {
        return fail("%s", e.what());
    } catch (...) {
        return fail("unknown exception");
    }
}

}  // namespace

struct eud_driver {
    HipUserDriver ud;
    explicit eud_driver(uint32_t device) : ud(device) {}
};

struct eud_oplist {
    OperatorListDesc desc;
    std::vector<std::shared_ptr<TensorDesc>> tensors;
    std::vector<std::shared_ptr<std::vector<uint8_t>>> data;  // parameter bytes, owned here
};

extern "C" {

const char *eud_last_error(void) { return g_error; }

int eud_initialize(eud_driver **driver, int device) {
    return guarded([&] {
        if (driver == nullptr || device < 0) return fail("eud_initialize: bad argument");
        *driver = nullptr;
        auto *d = new eud_driver((uint32_t)device);
        if (d->ud.Initialize() != ENN_RET_SUCCESS) {
            delete d;
            return fail_below("eud_initialize");
        }
        *driver = d;
        return 0;
    });
}

int eud_deinitialize(eud_driver *driver) {
    return guarded([&] {
        if (driver) {
            driver->ud.Deinitialize();
            delete driver;
        }
        return 0;
    });
}

int eud_oplist_create(eud_oplist **list, uint64_t id, int32_t legacy_model) {
    return guarded([&] {
        if (list == nullptr || legacy_model < 0 || legacy_model > TFlite::LegacyModel_ANDROID_NN) return fail("eud_oplist_create: bad argument");
        *list = new eud_oplist();
        (*list)->desc.id = id;
        (*list)->desc.legacy_model = (TFlite::LegacyModel)legacy_model;
        return 0;
    });
}

static int32_t add_tensor(eud_oplist *list, const uint32_t *shape, int32_t rank, int32_t tensor_type, float scale, int32_t zero_point,
                          std::shared_ptr<TensorDesc> *made) {
    if (list == nullptr || shape == nullptr || rank < 1 || rank > 4) return -fail("tensor: bad shape");
    if (tensor_type != EUD_TENSOR_INT32 && tensor_type != EUD_TENSOR_UINT8 && tensor_type != EUD_TENSOR_INT8) return -fail("tensor: type %d is not offered", tensor_type);
    auto t = std::make_shared<TensorDesc>();
    t->name = "t" + std::to_string(list->tensors.size());
    t->shape.assign(shape, shape + rank);
    t->data_type = (TFlite::TensorType)tensor_type;
    t->scale = scale;
    t->zero_point = zero_point;
    list->tensors.push_back(t);
    *made = t;
    return (int32_t)list->tensors.size() - 1;
}

int32_t eud_oplist_feature_map(eud_oplist *list, int32_t buffer_index, const uint32_t *shape, int32_t rank, int32_t tensor_type,
                               float scale, int32_t zero_point) {
    int32_t id = -1;
    (void)guarded([&] {
        std::shared_ptr<TensorDesc> t;
        id = add_tensor(list, shape, rank, tensor_type, scale, zero_point, &t);
        if (id >= 0) t->buffer_index = buffer_index;
        return 0;
    });
    return id;
}

int32_t eud_oplist_parameter(eud_oplist *list, const uint32_t *shape, int32_t rank, int32_t tensor_type, float scale, int32_t zero_point,
                             const void *data, size_t bytes, const float *scales, int32_t scale_count) {
    int32_t id = -1;
    (void)guarded([&] {
        if (data == nullptr || bytes == 0) return fail("parameter: no data");
        if (list && shape && rank >= 1 && rank <= 4) {
            size_t count = 1;
            for (int32_t i = 0; i < rank; ++i) count *= shape[i];
            if (count * (tensor_type == EUD_TENSOR_INT32 ? 4 : 1) != bytes) return fail("parameter: %zu bytes given, the shape holds %zu", bytes, count * (tensor_type == EUD_TENSOR_INT32 ? 4 : 1));
        }
        std::shared_ptr<TensorDesc> t;
        id = add_tensor(list, shape, rank, tensor_type, scale, zero_point, &t);
        if (id < 0) return 1;
        auto copy = std::make_shared<std::vector<uint8_t>>((const uint8_t *)data, (const uint8_t *)data + bytes);
        list->data.push_back(copy);
        t->is_const = true;
        t->data = copy->data();
        if (scales && scale_count > 0) t->per_channel_scales.assign(scales, scales + scale_count);
        return 0;
    });
    return id;
}

int eud_oplist_operator(eud_oplist *list, const char *name, int32_t builtin_code, const int32_t *inputs, int32_t input_count,
                        const int32_t *outputs, int32_t output_count, const eud_options *o) {
    return guarded([&] {
        if (list == nullptr || o == nullptr || inputs == nullptr || outputs == nullptr || input_count < 1 || output_count < 1)
            return fail("eud_oplist_operator: bad argument");
        OperatorDesc d;
        d.name = name ? name : "";
        d.id = list->desc.operators.size() + 1;
        d.code = (TFlite::BuiltinOperator)builtin_code;
        auto pick = [&](const int32_t *ids, int32_t n, std::vector<std::shared_ptr<TensorDesc>> *dst) {
            for (int32_t i = 0; i < n; ++i) {
                if (ids[i] < 0 || (size_t)ids[i] >= list->tensors.size()) return false;
                dst->push_back(list->tensors[ids[i]]);
            }
            return true;
        };
        if (!pick(inputs, input_count, &d.in_tensors) || !pick(outputs, output_count, &d.out_tensors)) return fail("eud_oplist_operator: unknown tensor number");
        const auto act = (TFlite::ActivationFunctionType)o->fused_activation_function;
        const std::vector<int32_t> pads = o->has_padding_value ? std::vector<int32_t>(o->padding_value, o->padding_value + 4) : std::vector<int32_t>();
        switch (builtin_code) {
            case EUD_OP_CONV_2D: {
                auto t = std::make_shared<TFlite::Conv2DOptions>();
                t->padding = (TFlite::Padding)o->padding;
                t->stride_w = o->stride_w;
                t->stride_h = o->stride_h;
                t->dilation_w_factor = o->dilation_w_factor;
                t->dilation_h_factor = o->dilation_h_factor;
                t->fused_activation_function = act;
                t->padding_value = pads;
                t->use_nchw = o->use_nchw != 0;
                d.option = t;
                break;
            }
            case EUD_OP_DEPTHWISE_CONV_2D: {
                auto t = std::make_shared<TFlite::DepthwiseConv2DOptions>();
                t->padding = (TFlite::Padding)o->padding;
                t->stride_w = o->stride_w;
                t->stride_h = o->stride_h;
                t->depth_multiplier = o->depth_multiplier;
                t->dilation_w_factor = o->dilation_w_factor;
                t->dilation_h_factor = o->dilation_h_factor;
                t->fused_activation_function = act;
                t->padding_value = pads;
                t->use_nchw = o->use_nchw != 0;
                d.option = t;
                break;
            }
            case EUD_OP_TRANSPOSE_CONV: {
                auto t = std::make_shared<TFlite::TransposeConvOptions>();
                t->padding = (TFlite::Padding)o->padding;
                t->stride_w = o->stride_w;
                t->stride_h = o->stride_h;
                t->group = o->group;
                t->fused_activation_function = act;
                t->padding_value = pads;
                t->use_nchw = o->use_nchw != 0;
                d.option = t;
                break;
            }
            case EUD_OP_AVERAGE_POOL_2D: {
                auto t = std::make_shared<TFlite::Pool2DOptions>();
                t->padding = (TFlite::Padding)o->padding;
                t->stride_w = o->stride_w;
                t->stride_h = o->stride_h;
                t->filter_width = o->filter_width;
                t->filter_height = o->filter_height;
                t->fused_activation_function = act;
                t->padding_value = pads;
                t->use_nchw = o->use_nchw != 0;
                d.option = t;
                break;
            }
            case EUD_OP_FULLY_CONNECTED: {
                auto t = std::make_shared<TFlite::FullyConnectedOptions>();
                t->fused_activation_function = act;
                d.option = t;
                break;
            }
            case EUD_OP_ADD: {
                auto t = std::make_shared<TFlite::AddOptions>();
                t->fused_activation_function = act;
                d.option = t;
                break;
            }
            default: return fail("eud_oplist_operator: operator code %d is not offered", builtin_code);
        }
        list->desc.operators.push_back(d);
        return 0;
    });
}

int eud_oplist_destroy(eud_oplist *list) {
    delete list;
    return 0;
}

int eud_open_subgraph(eud_driver *driver, const eud_oplist *list, int32_t fuse_residual_adds) {
    return guarded([&] {
        if (driver == nullptr || list == nullptr) return fail("eud_open_subgraph: null argument");
        driver->ud.constructor()->fuse_residual_adds = fuse_residual_adds != 0;
        return driver->ud.OpenSubGraph(list->desc) == ENN_RET_SUCCESS ? 0 : fail_below("eud_open_subgraph");
    });
}

int eud_prepare_subgraph(eud_driver *driver, uint64_t list_id) {
    return driver && driver->ud.PrepareSubGraph(list_id) == ENN_RET_SUCCESS ? 0 : fail("eud_prepare_subgraph failed");
}

int eud_execute_subgraph(eud_driver *driver, uint64_t list_id, const int32_t *buffer_indices, void *const *addresses, const size_t *sizes,
                         int32_t buffer_count) {
    return guarded([&] {
        if (driver == nullptr || buffer_count < 0 || (buffer_count > 0 && (!buffer_indices || !addresses || !sizes)))
            return fail("eud_execute_subgraph: bad argument");
        BufferTable table;
        for (int32_t i = 0; i < buffer_count; ++i) table.add(buffer_indices[i], addresses[i], sizes[i]);
        const OperatorListExecuteRequest request(list_id, 0, table);
        return driver->ud.ExecuteSubGraph(request) == ENN_RET_SUCCESS ? 0 : fail_below("eud_execute_subgraph");
    });
}

int eud_close_subgraph(eud_driver *driver, uint64_t list_id) {
    return guarded([&] { return driver && driver->ud.CloseSubGraph(list_id) == ENN_RET_SUCCESS ? 0 : fail("eud_close_subgraph: list is not open"); });
}

int eud_execute_operators(eud_driver *driver, uint64_t list_id, int32_t times) {
    return guarded([&] {
        if (driver == nullptr || times < 1) return fail("eud_execute_operators: bad argument");
        return driver->ud.ExecuteOperators(list_id, times) == ENN_RET_SUCCESS ? 0 : fail_below("eud_execute_operators");
    });
}

int eud_set_replay(eud_driver *driver, int32_t replay) {
    if (driver == nullptr || driver->ud.executor() == nullptr) return fail("eud_set_replay: no driver");
    driver->ud.executor()->replay = replay != 0;
    return 0;
}

int eud_set_image_lanes(eud_driver *driver, int32_t lanes, int32_t min_lane_images) {
    if (driver == nullptr || driver->ud.constructor() == nullptr) return fail("eud_set_image_lanes: no driver");
    if (lanes < 1 || min_lane_images < 1) return fail("eud_set_image_lanes: lanes and min_lane_images start at 1");
    driver->ud.constructor()->image_lanes = lanes;
    driver->ud.constructor()->min_lane_images = min_lane_images;
    return 0;
}

int eud_set_fuse_expansions(eud_driver *driver, int32_t mode) {
    if (driver == nullptr || driver->ud.constructor() == nullptr) return fail("eud_set_fuse_expansions: no driver");
    if (mode < 0 || mode > 2) return fail("eud_set_fuse_expansions: mode is 0, 1 or 2");
    driver->ud.constructor()->fuse_expansions = mode != 0;
    driver->ud.constructor()->fuse_unlisted_expansions = mode == 2;
    return 0;
}

int eud_set_store_channels_last(eud_driver *driver, int32_t on) {
    if (driver == nullptr || driver->ud.constructor() == nullptr) return fail("eud_set_store_channels_last: no driver");
    driver->ud.constructor()->store_channels_last = on != 0;
    return 0;
}

int eud_synchronize(eud_driver *driver) {
    if (driver == nullptr || !driver->ud.computeLibrary()) return fail("eud_synchronize: no driver");
    return driver->ud.computeLibrary()->runtime()->synchronize() == Status::SUCCESS ? 0 : fail_below("eud_synchronize");
}

void *eud_stream(eud_driver *driver) {
    return driver && driver->ud.computeLibrary() ? driver->ud.computeLibrary()->runtime()->stream() : nullptr;
}

int eud_stats(eud_driver *driver, uint64_t list_id, int32_t *operator_count, uint64_t *direct, uint64_t *recordings, uint64_t *replays,
              size_t *pool_bytes) {
    return guarded([&] {
        if (driver == nullptr || driver->ud.executor() == nullptr) return fail("eud_stats: no driver");
        UDOperators ops;
        if (driver->ud.get_graph_for_TC(list_id, ops) != ENN_RET_SUCCESS) return fail("eud_stats: list is not open");
        const auto &c = driver->ud.executor()->counters();
        if (operator_count) *operator_count = (int32_t)ops->size();
        if (direct) *direct = c.direct;
        if (recordings) *recordings = c.recordings;
        if (replays) *replays = c.replays;
        if (pool_bytes) *pool_bytes = driver->ud.computeLibrary()->runtime()->lastPoolAllocationBytes();
        return 0;
    });
}

static int list_tensor(eud_driver *driver, uint64_t list_id, bool output, int32_t i, std::shared_ptr<ITensor> *t) {
    if (driver == nullptr) return fail("no driver");
    UDOperators ops;
    UDTensors in, out;
    if (driver->ud.get_ud_operators(list_id, ops, in, out) != ENN_RET_SUCCESS) return fail("list is not open");
    const UDTensors &v = output ? out : in;
    if (i < 0 || (size_t)i >= v.size()) return fail("the list has %zu such tensors", v.size());
    *t = v[i];
    return 0;
}

int eud_write_input(eud_driver *driver, uint64_t list_id, int32_t i, const void *host, size_t bytes) {
    return guarded([&] {
        std::shared_ptr<ITensor> t;
        if (list_tensor(driver, list_id, false, i, &t)) return 1;
        if (host == nullptr || bytes != t->getNumOfBytes()) return fail("eud_write_input: %zu bytes given, the tensor holds %zu", bytes, t->getNumOfBytes());
        return t->writeData(const_cast<void *>(host), true) == Status::SUCCESS ? 0 : fail_below("eud_write_input");
    });
}

int eud_read_output(eud_driver *driver, uint64_t list_id, int32_t i, void *host, size_t bytes) {
    return guarded([&] {
        std::shared_ptr<ITensor> t;
        if (list_tensor(driver, list_id, true, i, &t)) return 1;
        if (host == nullptr || bytes != t->getNumOfBytes()) return fail("eud_read_output: %zu bytes given, the tensor holds %zu", bytes, t->getNumOfBytes());
        return t->readData(host, true) == Status::SUCCESS ? 0 : fail_below("eud_read_output");
    });
}

int eud_set_quant(eud_driver *driver, uint64_t list_id, int32_t is_output, int32_t i, float scale, int32_t zero_point) {
    return guarded([&] {
        std::shared_ptr<ITensor> t;
        if (list_tensor(driver, list_id, is_output != 0, i, &t)) return 1;
        t->setScale(scale);
        t->setZeroPoint(zero_point);
        return 0;
    });
}

}  // extern "C"
