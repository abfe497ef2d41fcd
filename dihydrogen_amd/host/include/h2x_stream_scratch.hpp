// Device scratch memory shared by the calls made on one stream: the workspaces
// of the overloads that keep the reference's exact signatures (which have no
// workspace argument) and of the h2 operators.  Used by both header trees
// (distconv/ and h2/).
//
// Lifetime.  The table lives on the heap and is never destroyed: no destructor
// of static storage duration ever calls into the HIP runtime, whose own exit
// handlers may already have run by then (the reference frees device memory per
// object, never at static destruction:
// legacy/include/distconv/tensor/halo_exchange_cuda.hpp:259-303).  Buffers stay
// allocated until the process ends or the caller releases them with release()
// (one stream: call it before hipStreamDestroy, because the runtime may hand the
// same handle to a later stream) or release_all().
//
// Threads.  The table is guarded by a mutex, so calls on different streams may
// come from different host threads.  Calls on ONE stream share one buffer per
// slot by design (their kernels are ordered by the stream); two host threads
// that enqueue on the same stream at the same time must serialise themselves,
// as with any other use of a stream.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <map>
#include <mutex>
#include <tuple>

namespace h2x_host
{

class StreamScratch
{
public:
    // Slots keep the users apart: a call may hold several buffers at once.
    enum Slot
    {
        BN_PARTIALS = 0,     // fp64 partial sums of the batch-norm reductions
        REDUCE_PARTIALS = 1, // tensor reduce_sum
        SOFTMAX_PARTIALS = 2,
        SOFTMAX_SCALARS = 3,
        GENERIC = 4
    };

    // At least `bytes` of device memory for (current device, stream, slot); grows
    // by synchronising the stream and reallocating.  Returns nullptr and sets
    // *err when the runtime refuses.
    static void* get(hipStream_t stream, int slot, size_t bytes, hipError_t* err)
    {
        int device = 0;
        if ((*err = hipGetDevice(&device)) != hipSuccess)
            return nullptr;
        Table& t = table();
        std::lock_guard<std::mutex> lock(t.mutex);
        Entry& e = t.entries[Key{device, stream, slot}];
        if (bytes > e.bytes || e.ptr == nullptr)
        {
            if (e.ptr)
            {
                if ((*err = hipStreamSynchronize(stream)) != hipSuccess)
                    return nullptr;
                void* old = e.ptr;
                e.ptr = nullptr;
                e.bytes = 0;
                if ((*err = hipFree(old)) != hipSuccess)
                    return nullptr;
            }
            void* p = nullptr;
            if ((*err = hipMalloc(&p, bytes ? bytes : 1)) != hipSuccess)
                return nullptr;
            e.ptr = p;
            e.bytes = bytes ? bytes : 1;
        }
        return e.ptr;
    }

    // Waits for `stream` and frees every buffer held for it on the current device.
    static hipError_t release(hipStream_t stream)
    {
        int device = 0;
        if (hipError_t e = hipGetDevice(&device))
            return e;
        Table& t = table();
        std::lock_guard<std::mutex> lock(t.mutex);
        hipError_t first = hipSuccess;
        bool synced = false;
        for (auto it = t.entries.begin(); it != t.entries.end();)
        {
            if (it->first.device != device || it->first.stream != stream)
            {
                ++it;
                continue;
            }
            if (it->second.ptr)
            {
                if (!synced)
                {
                    keep_first(first, hipStreamSynchronize(stream));
                    synced = true;
                }
                keep_first(first, hipFree(it->second.ptr));
            }
            it = t.entries.erase(it);
        }
        return first;
    }

    // Waits for the current device and frees every buffer of every stream on it.
    static hipError_t release_all()
    {
        int device = 0;
        if (hipError_t e = hipGetDevice(&device))
            return e;
        Table& t = table();
        std::lock_guard<std::mutex> lock(t.mutex);
        hipError_t first = hipSuccess;
        bool synced = false;
        for (auto it = t.entries.begin(); it != t.entries.end();)
        {
            if (it->first.device != device)
            {
                ++it;
                continue;
            }
            if (it->second.ptr)
            {
                if (!synced)
                {
                    keep_first(first, hipDeviceSynchronize());
                    synced = true;
                }
                keep_first(first, hipFree(it->second.ptr));
            }
            it = t.entries.erase(it);
        }
        return first;
    }

    // Buffers currently held (for tests and diagnostics).
    static size_t held_buffers()
    {
        Table& t = table();
        std::lock_guard<std::mutex> lock(t.mutex);
        size_t n = 0;
        for (auto& kv : t.entries)
            n += kv.second.ptr != nullptr;
        return n;
    }

private:
    struct Entry
    {
        void* ptr = nullptr;
        size_t bytes = 0;
    };
    struct Key
    {
        int device;
        hipStream_t stream;
        int slot;
        bool operator<(const Key& o) const
        {
            return std::tie(device, stream, slot) < std::tie(o.device, o.stream, o.slot);
        }
    };
    struct Table
    {
        std::mutex mutex;
        std::map<Key, Entry> entries;
    };
    static Table& table()
    {
        static Table* const t = new Table; // leaked on purpose, see the head of this file
        return *t;
    }
    static void keep_first(hipError_t& first, hipError_t e)
    {
        if (first == hipSuccess)
            first = e;
    }
};

} // namespace h2x_host
