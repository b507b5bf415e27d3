// Device runtime and buffer manager of the HIP userdriver backend: hipMalloc-backed
// buffers on one GPU behind the reference's pooling protocol.
//
// Same protocol as CLRuntime's buffer manager (src/userdriver/gpu/common/CLRuntime.cpp:34-157
// getBuffer / assignBufferPool / resetIntraBuffer / resetInterBuffer, :1339-1372
// allocBuffer with its 1024-byte head and 32-byte tail slack, :1409-1416
// releaseBuffer) and its copy / layout entry points (CLRuntime.hpp:59-110,
// CLRuntime.cpp:1477-1619), built differently: the pooled buffers of an operator list
// (INTER_SHARED_*, INTRA_SHARED) are slots of the library's eh_pool, which
// assignBufferPool() lays out in one device allocation, so an operator list costs one
// hipMalloc and none after it is built; DEDICATED buffers are allocations of their own.
// One in-order stream stands in for the reference's single in-order command queue
// (CLRuntime.cpp:920-928).
#pragma once

#include <map>
#include <memory>
#include <mutex>
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
    explicit HipBuffer(size_t byte, int32_t pool_slot = -1, int32_t arena = 0)
        : byte_(byte), buffer_(nullptr), pool_slot_(pool_slot), arena_(arena) {}
    void assignBuffer(void *buffer) { buffer_ = buffer; }
    void setBytes(size_t byte) { byte_ = byte; }
    size_t getBytes() { return byte_; }
    void *getDataPtr() { return buffer_; }
    int32_t poolSlot() const { return pool_slot_; }  // >= 0: lives in one of the runtime's pooled allocations
    int32_t arena() const { return arena_; }         // which one

private:
    size_t byte_;
    void *buffer_;
    int32_t pool_slot_;
    int32_t arena_;
};

class HipRuntime {
public:
    HipRuntime() = default;
    ~HipRuntime() {
        for (auto &kv : allocations_) eh_free(kv.second);
        for (auto &a : arenas_)
            if (a.pool) eh_pool_destroy(a.pool);
        for (void *e : events_) eh_event_destroy(e);
        for (void *s : lane_streams_) eh_stream_destroy(s);
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
    // The stream operators launch on: the runtime's own, unless the list executor has pointed the launches of a lane
    // at that lane's stream for the moment (launchOn).
    void *stream() { return launch_stream_ ? launch_stream_ : stream_; }
    void *mainStream() { return stream_; }
    void launchOn(void *stream) { launch_stream_ = stream; }

    // Streams for the lanes of an operator list beyond the first (default priority, made on first use), and events to
    // fork them from the main stream and join them to it.
    void *laneStream(size_t lane) {
        while (lane_streams_.size() <= lane) {
            void *s = nullptr;
            if (eh_stream_create(&s) != EH_OK) return nullptr;
            lane_streams_.push_back(s);
        }
        return lane_streams_[lane];
    }
    void *event(size_t index) {
        while (events_.size() <= index) {
            void *e = nullptr;
            if (eh_event_create(&e) != EH_OK) return nullptr;
            events_.push_back(e);
        }
        return events_[index];
    }

    // Pooled buffers are requested from the arena selected at the time.  Arenas are separate pools, each laid out in
    // an allocation of its own: a buffer never takes over storage from another arena's buffers, which is what the
    // lanes of an operator list need (they are at different operators at any moment, so one lane's liveness says
    // nothing about when another lane's buffer is free).
    void selectArena(int32_t arena) {
        if (arena < 0) arena = 0;
        if ((size_t)arena >= arenas_.size()) arenas_.resize((size_t)arena + 1);
        arena_ = arena;
    }

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
            case BufferType::INTER_SHARED_NEW: return pooled(EH_POOL_INTER_NEW, bytes);
            case BufferType::INTER_SHARED_REUSE: return pooled(EH_POOL_INTER_REUSE, bytes);
            case BufferType::INTRA_SHARED: return pooled(EH_POOL_INTRA, bytes);
            default: ERROR_PRINT("HipRuntime::getBuffer: unknown buffer type\n");
        }
        return nullptr;
    }

    // Materialises every pooled buffer at its final size, all of them in ONE device allocation (the reference
    // allocates each: CLRuntime.cpp:120-137), then forgets the pools.
    Status assignBufferPool() {
        last_arena_bytes_ = 0;
        for (auto &a : arenas_) {
            if (!a.pool) continue;
            size_t arena = 0;
            CHECK_EXPR_RETURN_FAILURE(eh_pool_assign(a.pool, &arena) == EH_OK, "assignBufferPool: %s", eh_last_error());
            last_arena_bytes_ += arena;
            for (auto &kv : a.pending) {
                void *ptr = nullptr;
                size_t bytes = 0;
                CHECK_EXPR_RETURN_FAILURE(eh_pool_slot(a.pool, kv.first, &ptr, &bytes) == EH_OK, "assignBufferPool: %s", eh_last_error());
                kv.second.first->setBytes(bytes);
                kv.second.first->assignBuffer(bytes ? ptr : nullptr);
            }
            a.pending.clear();
        }
        return Status::SUCCESS;
    }

    // Gives up the pooled buffers requested since the last assignment (a list whose construction failed half way):
    // they take no part in the next assignment and get no memory.
    Status abandonPendingBuffers() {
        Status st = Status::SUCCESS;
        for (auto &a : arenas_) {
            for (auto &kv : a.pending)
                if (a.pool && eh_pool_release(a.pool, kv.first) != EH_OK) st = Status::FAILURE;
            a.pending.clear();
        }
        return st;
    }

    Status resetIntraBuffer() {
        Arena &a = arenas_[(size_t)arena_];
        if (a.pool) CHECK_EXPR_RETURN_FAILURE(eh_pool_reset_intra(a.pool) == EH_OK, "resetIntraBuffer: %s", eh_last_error());
        return Status::SUCCESS;
    }

    Status resetInterBuffer(const std::shared_ptr<HipBuffer> buffer) {
        Arena *a = buffer && buffer->arena() >= 0 && (size_t)buffer->arena() < arenas_.size() ? &arenas_[(size_t)buffer->arena()] : nullptr;
        auto it = a ? a->pending.find(buffer->poolSlot()) : std::map<int32_t, std::pair<std::shared_ptr<HipBuffer>, int>>::iterator();
        if (!a || it == a->pending.end() || it->second.first != buffer || it->second.second == EH_POOL_INTRA || !a->pool ||
            eh_pool_reset_inter(a->pool, it->first) != EH_OK) {
            ERROR_PRINT("HipRuntime::resetInterBuffer: buffer not found\n");
            return Status::FAILURE;
        }
        return Status::SUCCESS;
    }

    // bytes of the allocations (one per arena in use) the last assignBufferPool() made for its pooled buffers
    size_t lastPoolAllocationBytes() const { return last_arena_bytes_; }

    size_t interPoolSize() const { return countPending(false); }
    size_t intraPoolSize() const { return countPending(true); }

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
        if (buffer->poolSlot() >= 0) {  // a pooled buffer: its allocation goes when the last buffer in it is released
            eh_pool *pool = buffer->arena() >= 0 && (size_t)buffer->arena() < arenas_.size() ? arenas_[(size_t)buffer->arena()].pool : nullptr;
            CHECK_EXPR_RETURN_FAILURE(pool != nullptr, "HipRuntime::releaseBuffer: no pool");
            synchronizeLocked();
            const int rc = eh_pool_release(pool, buffer->poolSlot());
            buffer->assignBuffer(nullptr);
            return rc == EH_OK ? Status::SUCCESS : Status::CL_FAILURE;
        }
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
        // The source is ordinary pageable memory that the caller may reuse as soon as this returns (the contract of
        // clEnqueueWriteBuffer(blocking = CL_FALSE) is that the caller waits for the event; callers of the reference's
        // writeData(false) do not, gpu_userdriver.cc:188-220).  That hipMemcpyAsync has staged a pageable source by the
        // time it returns is what the runtime does today, not what the API promises, so both modes wait for the copy.
        (void)blocking;
        return synchronizeLocked();
    }

    Status readBuffer(void *dst, const void *src, size_t type_bytes, uint32_t num, bool blocking) {
        std::lock_guard<std::mutex> lock(mutex_);
        CHECK_EXPR_RETURN_FAILURE(eh_d2h(dst, src, type_bytes * (size_t)num, stream_) == EH_OK, "readBuffer: %s",
                                  eh_last_error());
        // the destination is pageable host memory: the copy is complete only after the stream has drained, and a
        // caller that asks for a non-blocking read must synchronize() before it looks (as with clEnqueueReadBuffer)
        return blocking ? synchronizeLocked() : Status::SUCCESS;
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
    // One pooled request: the library keeps the protocol's books (which slot a REUSE takes over, how large it has
    // to be in the end); a slot that is taken over keeps its HipBuffer object, as the reference hands back the same
    // CLBuffer.
    std::shared_ptr<HipBuffer> pooled(int kind, size_t bytes) {
        Arena &a = arenas_[(size_t)arena_];
        if (!a.pool && eh_pool_create(&a.pool) != EH_OK) {
            ERROR_PRINT("HipRuntime::getBuffer: %s\n", eh_last_error());
            return nullptr;
        }
        int32_t slot = -1;
        if (eh_pool_request(a.pool, kind, bytes, &slot) != EH_OK) {
            ERROR_PRINT("HipRuntime::getBuffer: %s\n", eh_last_error());
            return nullptr;
        }
        size_t final_bytes = bytes;
        (void)eh_pool_slot(a.pool, slot, nullptr, &final_bytes);
        auto it = a.pending.find(slot);
        if (it != a.pending.end()) {
            it->second.first->setBytes(final_bytes);
            return it->second.first;
        }
        auto buffer = std::make_shared<HipBuffer>(final_bytes, slot, arena_);
        a.pending[slot] = std::make_pair(buffer, kind);
        return buffer;
    }
    size_t countPending(bool intra) const {
        size_t n = 0;
        for (auto &a : arenas_)
            for (auto &kv : a.pending) n += (kv.second.second == EH_POOL_INTRA) == intra ? 1 : 0;
        return n;
    }

    struct Arena {
        eh_pool *pool = nullptr;
        std::map<int32_t, std::pair<std::shared_ptr<HipBuffer>, int>> pending;  // slots requested since the last assignment
    };
    std::vector<Arena> arenas_ = std::vector<Arena>(1);
    int32_t arena_ = 0;
    std::vector<void *> lane_streams_, events_;
    void *launch_stream_ = nullptr;
    size_t last_arena_bytes_ = 0;
    std::map<void *, void *> allocations_;  // user pointer -> hipMalloc base
    std::mutex mutex_;
    void *stream_ = nullptr;
};

}  // namespace hip
}  // namespace ud
}  // namespace enn
