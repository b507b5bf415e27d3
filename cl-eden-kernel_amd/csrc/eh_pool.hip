// Pooled device buffers of an operator list: the reference's buffer manager protocol
// (CLRuntime::getBuffer / resetInterBuffer / resetIntraBuffer / assignBufferPool,
// src/userdriver/gpu/common/CLRuntime.cpp:34-157) with one difference in how it ends.  The reference sizes its
// pooled buffers while the operators are built and then allocates each of them (:120-137, allocBuffer :1339-1372);
// here assignment lays all of them out in ONE device allocation, every buffer at its own 1024-byte aligned offset
// with the reference's 1024 bytes of slack in front and 32 behind (its kernels over-read with vector loads, and so
// do these).  An operator list therefore costs one hipMalloc however many feature maps it has, nothing is allocated
// after assignment (a captured graph never meets an allocator), and the feature maps that take over each other's
// storage (liveness reuse, gpu_op_constructor.cc:2157-2191) sit next to each other in memory.
#include <new>
#include <vector>

#include "eh_internal.h"

namespace {

constexpr size_t kHead = 1024, kTail = 32, kAlign = 1024;

struct Slot {
    size_t bytes = 0;
    int kind = 0;          // EH_POOL_INTER_* or EH_POOL_INTRA as first requested
    bool live = false;     // inter: not yet handed back; intra: taken by the operator being built
    int generation = 0;    // which assignment materialises it
    size_t offset = 0;     // of the user pointer within the generation's allocation, once laid out
    bool released = false; // eh_pool_release called
};

struct Arena {
    void *base = nullptr;
    size_t bytes = 0;
    int live_slots = 0;
};

size_t padded(size_t bytes) { return (kHead + bytes + kTail + kAlign - 1) / kAlign * kAlign; }

}  // namespace

struct eh_pool {
    std::vector<Slot> slots;
    std::vector<Arena> arenas;  // one per assignment
    int generation = 0;         // of the slots being collected now

    // offsets of the current generation's slots in request order; returns the allocation size
    size_t layout() {
        size_t at = 0;
        for (auto &s : slots) {
            if (s.generation != generation || s.released) continue;  // a buffer released before assignment gets no memory
            s.offset = at + kHead;
            at += padded(s.bytes);
        }
        return at;
    }
};

extern "C" {

int eh_pool_create(eh_pool **pool) {
    EH_REQUIRE(pool != nullptr, "null result pointer");
    *pool = new (std::nothrow) eh_pool();
    EH_REQUIRE(*pool != nullptr, "out of host memory");
    return EH_OK;
}

int eh_pool_request(eh_pool *pool, int kind, size_t bytes, int32_t *slot) {
    EH_REQUIRE(pool != nullptr && slot != nullptr, "null argument");
    EH_REQUIRE(kind == EH_POOL_INTER_NEW || kind == EH_POOL_INTER_REUSE || kind == EH_POOL_INTRA, "unknown pool kind %d", kind);
    auto &slots = pool->slots;
    const int gen = pool->generation;
    auto fresh = [&](bool intra) {
        Slot s;
        s.bytes = bytes;
        s.kind = kind;
        s.live = true;
        s.generation = gen;
        (void)intra;
        try {
            slots.push_back(s);
        } catch (const std::bad_alloc &) {
            {
            eh::set_error("out of host memory");
            return EH_FAILURE;
        }
        }
        *slot = (int32_t)slots.size() - 1;
        return EH_OK;
    };
    if (kind == EH_POOL_INTER_NEW) return fresh(false);
    if (kind == EH_POOL_INTER_REUSE) {
        // the first buffer handed back by resetInterBuffer, grown if it is too small (CLRuntime.cpp:52-72)
        for (size_t i = 0; i < slots.size(); ++i) {
            Slot &s = slots[i];
            if (s.generation == gen && s.kind != EH_POOL_INTRA && !s.live && !s.released) {
                if (s.bytes < bytes) s.bytes = bytes;
                s.live = true;
                *slot = (int32_t)i;
                return EH_OK;
            }
        }
        return fresh(false);
    }
    // intra-operator scratch (CLRuntime.cpp:73-113): the smallest free one that is large enough, else the largest
    // free one grown, else a new one
    int best = -1;
    for (size_t i = 0; i < slots.size(); ++i) {
        const Slot &s = slots[i];
        if (s.generation == gen && s.kind == EH_POOL_INTRA && !s.live && !s.released && s.bytes >= bytes && (best < 0 || s.bytes < slots[best].bytes))
            best = (int)i;
    }
    if (best < 0) {
        for (size_t i = 0; i < slots.size(); ++i) {
            const Slot &s = slots[i];
            if (s.generation == gen && s.kind == EH_POOL_INTRA && !s.live && !s.released && (best < 0 || s.bytes > slots[best].bytes)) best = (int)i;
        }
        if (best >= 0) slots[best].bytes = bytes;
    }
    if (best < 0) return fresh(true);
    slots[best].live = true;
    *slot = best;
    return EH_OK;
}

int eh_pool_reset_inter(eh_pool *pool, int32_t slot) {
    EH_REQUIRE(pool != nullptr, "null pool");
    EH_REQUIRE(slot >= 0 && (size_t)slot < pool->slots.size() && pool->slots[slot].generation == pool->generation &&
                   pool->slots[slot].kind != EH_POOL_INTRA && !pool->slots[slot].released,
               "resetInterBuffer: slot %d is not a pooled feature map of the list being built", slot);
    pool->slots[slot].live = false;
    return EH_OK;
}

int eh_pool_reset_intra(eh_pool *pool) {
    EH_REQUIRE(pool != nullptr, "null pool");
    for (auto &s : pool->slots)
        if (s.generation == pool->generation && s.kind == EH_POOL_INTRA) s.live = false;
    return EH_OK;
}

int eh_pool_layout(eh_pool *pool, size_t *arena_bytes, int32_t *slot_count) {
    EH_REQUIRE(pool != nullptr, "null pool");
    const size_t total = pool->layout();
    int32_t count = 0;
    for (auto &s : pool->slots) count += (s.generation == pool->generation && !s.released) ? 1 : 0;
    if (arena_bytes) *arena_bytes = total;
    if (slot_count) *slot_count = count;
    return EH_OK;
}

int eh_pool_assign(eh_pool *pool, size_t *arena_bytes) {
    EH_REQUIRE(pool != nullptr, "null pool");
    const size_t total = pool->layout();
    Arena arena;
    arena.bytes = total;
    // slots released before this assignment were left out of the layout and do not keep the allocation alive
    for (auto &s : pool->slots) arena.live_slots += (s.generation == pool->generation && !s.released) ? 1 : 0;
    try {
        pool->arenas.resize((size_t)pool->generation + 1);
    } catch (const std::bad_alloc &) {
        {
            eh::set_error("out of host memory");
            return EH_FAILURE;
        }
    }
    if (total > 0 && arena.live_slots > 0) {
        int rc = eh_malloc(&arena.base, total);  // zero-filled: the reference zero-fills its intra buffers (:124-129)
        if (rc) return rc;
    }
    pool->arenas[pool->generation] = arena;
    ++pool->generation;  // the pools are forgotten: later requests start another list (:131-135)
    if (arena_bytes) *arena_bytes = total;
    return EH_OK;
}

int eh_pool_slot(const eh_pool *pool, int32_t slot, void **ptr, size_t *bytes) {
    EH_REQUIRE(pool != nullptr, "null pool");
    EH_REQUIRE(slot >= 0 && (size_t)slot < pool->slots.size(), "pool slot %d does not exist", slot);
    const Slot &s = pool->slots[slot];
    if (bytes) *bytes = s.bytes;
    if (ptr) {
        const bool assigned = s.generation < pool->generation && !s.released && pool->arenas[s.generation].base != nullptr;
        *ptr = assigned ? static_cast<char *>(pool->arenas[s.generation].base) + s.offset : nullptr;  // null until assigned
    }
    return EH_OK;
}

int eh_pool_release(eh_pool *pool, int32_t slot) {
    EH_REQUIRE(pool != nullptr, "null pool");
    EH_REQUIRE(slot >= 0 && (size_t)slot < pool->slots.size(), "pool slot %d does not exist", slot);
    Slot &s = pool->slots[slot];
    EH_REQUIRE(!s.released, "pool slot %d released twice", slot);
    s.released = true;
    if (s.generation < pool->generation) {
        Arena &a = pool->arenas[s.generation];
        if (--a.live_slots == 0 && a.base) {  // the allocation goes with its last buffer
            int rc = eh_free(a.base);
            a.base = nullptr;
            return rc;
        }
    }
    return EH_OK;
}

int eh_pool_destroy(eh_pool *pool) {
    if (!pool) return EH_OK;
    int rc = EH_OK;
    for (auto &a : pool->arenas)
        if (a.base) {
            const int r = eh_free(a.base);
            rc = rc ? rc : r;
        }
    delete pool;
    return rc;
}

}  // extern "C"
