// Types shared by the operator interface of the HIP userdriver backend.
// Mirrors the names, enumerator values and field order of the reference's
// src/userdriver/common/operator_interfaces/common/Common.hpp:12-260 for the
// subset the quantized convolution / depthwise / fully-connected / deconvolution
// path touches, so that code written against the reference compiles against this.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <numeric>
#include <vector>

typedef void *DataPtr;
constexpr int32_t UNDEFINED = -1;
typedef std::vector<uint32_t> NDims;

enum class DataOrder { NCHW = 0, NHWC = 1, OTHER = 2, SIZE };

enum class DataOrderChangeType {
    NHWC2NCHW = 0, NCHW2NHWC = 1, NHWC2DHWC4 = 2, NCHW2DHWC4 = 3, DHWC42NHWC = 4, DHWC42NCHW = 5, OTHER = 6, SIZE
};

enum class DataType {
    UNKNOWN = -1, FLOAT = 0, HALF = 1, INT32 = 2, INT8 = 3, UINT8 = 4, BOOL = 5, INT16 = 6, UINT16 = 7, FLOAT16 = 8, SIZE
};

enum class PrecisionType { FP32 = 0, FP16 = 1, INT32 = 2, INT16 = 3, INT8 = 4, UINT8 = 5, SIZE };

enum class Status { SUCCESS = 0, FAILURE = 1, CL_FAILURE = 2, INVALID_PARAMS = 3, SIZE };

enum class BufferType {
    DEDICATED = 0,           // constant tensor of an operator: allocated at once, zero filled
    INTER_SHARED_REUSE = 1,  // output of an operator: may take over a released inter-operator buffer
    INTER_SHARED_NEW = 2,    // input of an operator: a fresh inter-operator buffer
    INTRA_SHARED = 3,        // scratch inside an operator: pooled, sized to the largest request
    SIZE
};

enum class StorageType { BUFFER = 0, TEXTURE = 1, SIZE };
enum class ComputeType { TFLite = 0, Caffe, SIZE };

enum { N_NCHW = 0, C_NCHW = 1, H_NCHW = 2, W_NCHW = 3 };
enum { N_NHWC = 0, H_NHWC = 1, W_NHWC = 2, C_NHWC = 3 };

typedef struct QuantInfo {
    float scale;
    int32_t zeroPoint;
} QuantInfo;

typedef struct Dim4 {
    uint32_t n, c, h, w;
} Dim4;

typedef struct Dim2 {
    uint32_t h, w;
} Dim2;

typedef struct Pad4 {
    uint32_t t, r, b, l;
} Pad4;

// A Dim4 that holds channels-last extents positionally (n, h, w, c) read as planar (n, c, h, w).
inline Dim4 convertDimToNCHW(const Dim4 &nhwc) { return Dim4{nhwc.n, nhwc.w, nhwc.c, nhwc.h}; }
inline Dim4 convertDimToNHWC(const Dim4 &nchw) { return Dim4{nchw.n, nchw.h, nchw.w, nchw.c}; }

inline uint32_t getTensorSizeFromDims(const Dim4 &d) { return d.n * d.c * d.h * d.w; }
inline uint32_t getTensorSizeFromDims(const NDims &nd) {
    return std::accumulate(nd.begin(), nd.end(), 1u, std::multiplies<uint32_t>());
}

inline Dim4 extendToDim4(const std::vector<uint32_t> &from) {
    if (from.empty()) return Dim4{0, 0, 0, 0};
    uint32_t v[4] = {1, 1, 1, 1};
    for (size_t i = 0; i < from.size() && i < 4; ++i) v[i] = from[i];
    return Dim4{v[0], v[1], v[2], v[3]};
}

inline size_t alignTo(size_t value, size_t alignment) { return (value + alignment - 1) / alignment * alignment; }

inline size_t getTypeBytes(const DataType &data_type, const PrecisionType &precision) {
    switch (data_type) {
        case DataType::FLOAT: return precision == PrecisionType::FP16 ? 2 : 4;
        case DataType::HALF:
        case DataType::FLOAT16: return precision == PrecisionType::FP32 ? 4 : 2;
        case DataType::INT32: return 4;
        case DataType::INT8:
        case DataType::UINT8:
        case DataType::BOOL: return 1;
        case DataType::UINT16:
        case DataType::INT16: return 2;
        default: return 0;
    }
}

inline bool isDimsSame(const Dim4 &a, const Dim4 &b) { return a.n == b.n && a.c == b.c && a.h == b.h && a.w == b.w; }

template <typename T>
std::shared_ptr<T> make_shared_array(size_t size) {
    return std::shared_ptr<T>(new T[size], std::default_delete<T[]>());
}
