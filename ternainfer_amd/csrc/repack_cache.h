// Bookkeeping of the repack cache behind the reference-format entry points: which device-side P2 copy belongs to which
// weight, how much memory the copies take, which one goes when the limit is reached, and what happens to a copy that was
// found stale.  Host-only and free of HIP (the owner passes the function that releases device memory), so the policy
// can be exercised on a machine without a GPU.
//
// Rules:
//   - a weight is identified by device, the bitmap / sign / offset pointers and the shape;
//   - copies are kept in order of last use; when a new copy would take the total past the limit, the least recently
//     used copies go first -- except pinned ones;
//   - a copy is pinned once a launch on it was recorded during stream capture: a captured graph holds its address, so
//     it is never released to make room, and when it is found stale its memory is parked (kept allocated, out of the
//     map) instead of released.  Only clear() releases pinned and parked copies;
//   - every copy has an id (1, 2, ...); the device-side check reports a stale copy by that id.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <list>
#include <unordered_map>
#include <vector>

namespace terna {

struct RepackKey {
    int device;
    const void* bitmap;
    const void* signs;
    const void* offsets;
    int n, k;
    bool operator==(const RepackKey& o) const
    {
        return device == o.device && bitmap == o.bitmap && signs == o.signs && offsets == o.offsets && n == o.n && k == o.k;
    }
};
struct RepackKeyHash {
    size_t operator()(const RepackKey& key) const
    {
        size_t h = std::hash<const void*>()(key.bitmap);
        h = h * 1000003u ^ std::hash<const void*>()(key.signs);
        h = h * 1000003u ^ std::hash<const void*>()(key.offsets);
        return h * 1000003u ^ (static_cast<size_t>(key.n) << 20) ^ static_cast<size_t>(key.k) ^ (static_cast<size_t>(key.device) << 40);
    }
};

template <class Payload>
class RepackCachePolicy {
public:
    struct Slot {
        RepackKey key;
        Payload payload;     // what a launch on the copy needs
        void* mem;           // the allocation (released through the owner's function)
        size_t bytes;
        uint32_t id;
        bool pinned;
    };
    using Release = void (*)(void*);

    RepackCachePolicy(Release release, size_t limit_bytes) : release_(release), limit_(limit_bytes) {}
    ~RepackCachePolicy() = default;      // device memory outlives the process's static destructors: nothing is released here

    // The copy of `key`, now the most recently used one, or NULL.
    Slot* find(const RepackKey& key)
    {
        const auto it = index_.find(key);
        if (it == index_.end()) return nullptr;
        order_.splice(order_.begin(), order_, it->second);
        return &*it->second;
    }

    // Room for `bytes` more under the limit, releasing least recently used copies that are not pinned.  False when
    // that is impossible (the new copy alone exceeds the limit, or what remains is pinned): nothing was released then.
    bool make_room(size_t bytes)
    {
        if (bytes > limit_) return false;
        size_t freeable = 0;
        for (const Slot& s : order_)
            if (!s.pinned) freeable += s.bytes;
        if (used_ + bytes > limit_ + freeable) return false;
        auto it = order_.end();
        while (used_ + bytes > limit_ && it != order_.begin()) {
            --it;
            if (it->pinned) continue;
            index_.erase(it->key);
            release_(it->mem);
            used_ -= it->bytes;
            ++evicted_;
            it = order_.erase(it);
        }
        return used_ + bytes <= limit_;
    }

    Slot* insert(const RepackKey& key, void* mem, size_t bytes, const Payload& payload)
    {
        order_.push_front(Slot{key, payload, mem, bytes, next_id_, false});
        next_id_ = next_id_ == UINT32_MAX ? 1u : next_id_ + 1u;
        index_[key] = order_.begin();
        used_ += bytes;
        return &order_.front();
    }

    // The id the next insert() will hand out (the copy's fingerprint check is set up before the copy is registered).
    uint32_t next_id() const { return next_id_; }

    // The copy with this id was found stale: it leaves the map; its memory is released, or parked when it is pinned.
    // False when no copy has that id (already gone).
    bool retire(uint32_t id)
    {
        for (auto it = order_.begin(); it != order_.end(); ++it) {
            if (it->id != id) continue;
            index_.erase(it->key);
            used_ -= it->bytes;
            if (it->pinned) {
                parked_.push_back(it->mem);
                parked_bytes_ += it->bytes;
            } else {
                release_(it->mem);
            }
            order_.erase(it);
            ++retired_;
            return true;
        }
        return false;
    }

    void clear()
    {
        for (const Slot& s : order_) release_(s.mem);
        for (void* p : parked_) release_(p);
        order_.clear();
        index_.clear();
        parked_.clear();
        used_ = parked_bytes_ = 0;
    }

    void set_limit(size_t bytes) { limit_ = bytes; }
    size_t limit() const { return limit_; }
    size_t used() const { return used_; }
    size_t entries() const { return order_.size(); }
    size_t parked_bytes() const { return parked_bytes_; }
    uint64_t retired() const { return retired_; }
    uint64_t evicted() const { return evicted_; }

private:
    Release release_;
    size_t limit_;
    size_t used_ = 0, parked_bytes_ = 0;
    uint64_t retired_ = 0, evicted_ = 0;
    uint32_t next_id_ = 1;
    std::list<Slot> order_;                                                      // most recently used first
    std::unordered_map<RepackKey, typename std::list<Slot>::iterator, RepackKeyHash> index_;
    std::vector<void*> parked_;
};

// ---- how much of the caller's `workspace` a call may use -----------------------------------------------------------
// The reference's own use of that buffer is the contract (the caller sizes it for the reference, model.py:34-42,
// tests/test_kernel.cu:331): its decode path writes SPLIT_K planes of M x N int32 partial sums
// (TernaSpMM_API.cuh:66-136), its prefill path a dense int8 copy of the N x K matrix (SpMM_Kernel.cuh:263-269,
// TernaSpMM_API.cuh:279-282).  `prefill_path`: the call is one the reference would serve by its prefill path
// (M > 64 on the plain symbol, or the _prefill symbol).
inline size_t reference_workspace_bytes(bool prefill_path, int M, int N, int K, int split_k)
{
    if (prefill_path) return static_cast<size_t>(N) * static_cast<size_t>(K);
    return split_k > 0 ? static_cast<size_t>(4) * M * N * static_cast<size_t>(split_k) : 0;
}

}  // namespace terna
