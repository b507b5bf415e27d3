// Device runtime and buffer manager of the HIP userdriver backend: hipMalloc-backed
// buffers on one GPU behind the reference's pooling protocol.
//
// Mirrors CLRuntime's buffer manager (src/userdriver/gpu/common/CLRuntime.cpp:34-157
// getBuffer / assignBufferPool / resetIntraBuffer / resetInterBuffer, :1339-1372
// allocBuffer with its 1024-byte head and 32-byte tail slack, :1409-1416
// releaseBuffer) and its copy / layout entry points (CLRuntime.hpp:59-110,
// CLRuntime.cpp:1477-1619).  One in-order stream stands in for the reference's
// single in-order command queue (CLRuntime.cpp:920-928).
#pragma once

#include <algorithm>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <utility>
#include <vector>

#include "Common.hpp"
#include "Error.hpp"
#include "eden_hip.h"

namespace enn {
namespace ud {
namespace hip {

// A device allocation that may not exist yet (pooled buffers materialise in assignBufferPool).
class HipBuffer {
public:
    explicit HipBuffer(size_t byte) : byte_(byte), buffer_(nullptr) {}
    void assignBuffer(void *buffer) { buffer_ = buffer; }
    void setBytes(size_t byte) { byte_ = byte; }
    size_t getBytes() { return byte_; }
    void *getDataPtr() { return buffer_; }

private:
    size_t byte_;
    void *buffer_;
};

class HipRuntime {
public:
    HipRuntime() = default;
    ~HipRuntime() {
        for (auto &kv : allocations_) eh_free(kv.second);
        if (stream_) eh_stream_destroy(stream_);
    }
    HipRuntime(const HipRuntime &) = delete;
    HipRuntime &operator=(const HipRuntime &) = delete;

    Status initialize(const uint32_t &target_device_id) {
        CHECK_EXPR_RETURN_FAILURE(eh_init((int)target_device_id) == EH_OK, "HipRuntime::initialize: %s", eh_last_error());
        return Status::SUCCESS;
    }
    Status initializeQueue() {
        if (!stream_) CHECK_EXPR_RETURN_FAILURE(eh_stream_create(&stream_) == EH_OK, "stream: %s", eh_last_error());
        return Status::SUCCESS;
    }
    void *stream() { return stream_; }

    // BufferType protocol, as CLRuntime::getBuffer.
    std::shared_ptr<HipBuffer> getBuffer(const PrecisionType &precision, const DataType &data_type, const Dim4 &dims,
                                         const BufferType &buffer_type,
                                         const StorageType &storage_type = StorageType::BUFFER) {
        if (storage_type != StorageType::BUFFER) {
            ERROR_PRINT("HipRuntime::getBuffer: texture storage does not exist on this backend\n");
            return nullptr;
        }
        const size_t bytes = getTypeBytes(data_type, precision) * (size_t)dims.n * dims.c * dims.h * dims.w;
        switch (buffer_type) {
            case BufferType::DEDICATED: {
                auto buffer = std::make_shared<HipBuffer>(bytes);
                buffer->assignBuffer(allocBuffer(bytes, true));
                return buffer;
            }
            case BufferType::INTER_SHARED_NEW: {
                auto buffer = std::make_shared<HipBuffer>(bytes);
                inter_buffers_.push_back(std::make_pair(buffer, true));
                return buffer;
            }
            case BufferType::INTER_SHARED_REUSE: {
                for (auto &entry : inter_buffers_) {
                    if (!entry.second) {  // released by resetInterBuffer: take it over, grown if needed
                        if (entry.first->getBytes() < bytes) entry.first->setBytes(bytes);
                        entry.second = true;
                        return entry.first;
                    }
                }
                auto buffer = std::make_shared<HipBuffer>(bytes);
                inter_buffers_.push_back(std::make_pair(buffer, true));
                return buffer;
            }
            case BufferType::INTRA_SHARED: {
                for (auto &entry : intra_buffers_) {  // a free one that is already large enough
                    if (!std::get<1>(entry) && std::get<0>(entry) >= bytes) {
                        std::get<1>(entry) = true;
                        return std::get<2>(entry);
                    }
                }
                for (auto it = intra_buffers_.rbegin(); it != intra_buffers_.rend(); ++it) {  // the largest free one, grown
                    if (!std::get<1>(*it)) {
                        std::get<0>(*it) = bytes;
                        std::get<1>(*it) = true;
                        auto mem = std::get<2>(*it);
                        sortIntra();
                        return mem;
                    }
                }
                auto buffer = std::make_shared<HipBuffer>(0);
                intra_buffers_.push_back(std::make_tuple(bytes, true, buffer));
                sortIntra();
                return buffer;
            }
            default: ERROR_PRINT("HipRuntime::getBuffer: unknown buffer type\n");
        }
        return nullptr;
    }

    // Materialises every pooled buffer at its final size (intra: zero filled), then forgets the pools.
    Status assignBufferPool() {
        for (auto &entry : intra_buffers_) {
            std::get<2>(entry)->setBytes(std::get<0>(entry));
            std::get<2>(entry)->assignBuffer(allocBuffer(std::get<0>(entry), true));
        }
        intra_buffers_.clear();
        for (auto &entry : inter_buffers_) entry.first->assignBuffer(allocBuffer(entry.first->getBytes(), false));
        inter_buffers_.clear();
        return Status::SUCCESS;
    }

    Status resetIntraBuffer() {
        for (auto &entry : intra_buffers_) std::get<1>(entry) = false;
        return Status::SUCCESS;
    }

    Status resetInterBuffer(const std::shared_ptr<HipBuffer> buffer) {
        for (auto &entry : inter_buffers_) {
            if (entry.first == buffer) {
                entry.second = false;
                return Status::SUCCESS;
            }
        }
        ERROR_PRINT("HipRuntime::resetInterBuffer: buffer not found\n");
        return Status::FAILURE;
    }

    size_t interPoolSize() const { return inter_buffers_.size(); }
    size_t intraPoolSize() const { return intra_buffers_.size(); }

    // 1024 bytes of slack in front, 32 behind, total rounded to 1024, as the reference pads every
    // allocation; the returned pointer is 1024-byte aligned.
    void *allocBuffer(const size_t &bytes, const bool &zero_init) {
        if (bytes == 0) return nullptr;
        const size_t head = 1024, tail = 32;
        const size_t total = alignTo(head + tail + bytes, 1024);
        void *base = nullptr;
        if (eh_malloc(&base, total) != EH_OK) {  // eh_malloc zero-fills, which covers zero_init
            ERROR_PRINT("HipRuntime::allocBuffer: %s\n", eh_last_error());
            return nullptr;
        }
        (void)zero_init;
        void *user = static_cast<char *>(base) + head;
        std::lock_guard<std::mutex> lock(mutex_);
        allocations_[user] = base;
        return user;
    }

    Status releaseBuffer(std::shared_ptr<HipBuffer> buffer) {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = allocations_.find(buffer->getDataPtr());
        CHECK_EXPR_RETURN_FAILURE(it != allocations_.end(), "HipRuntime::releaseBuffer: unknown buffer");
        synchronizeLocked();
        const int rc = eh_free(it->second);
        allocations_.erase(it);
        buffer->assignBuffer(nullptr);
        return rc == EH_OK ? Status::SUCCESS : Status::CL_FAILURE;
    }

    Status writeBuffer(void *dst, const void *src, size_t type_bytes, uint32_t num, bool blocking) {
        std::lock_guard<std::mutex> lock(mutex_);
        CHECK_EXPR_RETURN_FAILURE(eh_h2d(dst, src, type_bytes * (size_t)num, stream_) == EH_OK, "writeBuffer: %s",
                                  eh_last_error());
        // the source is pageable host memory the caller may reuse at once: always wait
        (void)blocking;
        return synchronizeLocked();
    }

    Status readBuffer(void *dst, const void *src, size_t type_bytes, uint32_t num, bool blocking) {
        std::lock_guard<std::mutex> lock(mutex_);
        CHECK_EXPR_RETURN_FAILURE(eh_d2h(dst, src, type_bytes * (size_t)num, stream_) == EH_OK, "readBuffer: %s",
                                  eh_last_error());
        (void)blocking;
        return synchronizeLocked();
    }

    Status copyBuffer(void *dst, const void *src, size_t bytes) {
        CHECK_EXPR_RETURN_FAILURE(eh_d2d(dst, src, bytes, stream_) == EH_OK, "copyBuffer: %s", eh_last_error());
        return Status::SUCCESS;
    }

    Status NCHW2NHWC(const void *src, void *dst, const Dim4 &nchw) {
        CHECK_EXPR_RETURN_FAILURE(eh_transpose_u8_nchw2nhwc(src, dst, nchw.n, nchw.c, nchw.h, nchw.w, stream_) == EH_OK,
                                  "NCHW2NHWC: %s", eh_last_error());
        return Status::SUCCESS;
    }
    Status NHWC2NCHW(const void *src, void *dst, const Dim4 &nchw) {
        CHECK_EXPR_RETURN_FAILURE(eh_transpose_u8_nhwc2nchw(src, dst, nchw.n, nchw.c, nchw.h, nchw.w, stream_) == EH_OK,
                                  "NHWC2NCHW: %s", eh_last_error());
        return Status::SUCCESS;
    }

    void flush() {}  // launches are submitted as they are made
    Status synchronize() {
        std::lock_guard<std::mutex> lock(mutex_);
        return synchronizeLocked();
    }

private:
    Status synchronizeLocked() {
        CHECK_EXPR_RETURN_FAILURE(eh_stream_sync(stream_) == EH_OK, "synchronize: %s", eh_last_error());
        return Status::SUCCESS;
    }
    void sortIntra() {
        std::sort(intra_buffers_.begin(), intra_buffers_.end(),
                  [](const IntraEntry &a, const IntraEntry &b) { return std::get<0>(a) < std::get<0>(b); });
    }

    typedef std::tuple<size_t, bool, std::shared_ptr<HipBuffer>> IntraEntry;
    std::vector<std::pair<std::shared_ptr<HipBuffer>, bool>> inter_buffers_;
    std::vector<IntraEntry> intra_buffers_;
    std::map<void *, void *> allocations_;  // user pointer -> hipMalloc base
    std::mutex mutex_;
    void *stream_ = nullptr;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
