// Least-recently-used cache and the metadata key of the operator adaptors. Host-only, no device code.
//
// Behaviour follows the reference's include/infinicore/common/LRUCache.hpp:12-139 (capacity 0 = unbounded,
// get() refreshes an entry, put() on a full cache evicts the least recently used one, setCapacity() evicts
// down to the new size) and include/infinicore/common/hash.hpp:11-31 (dtype, extents, strides folded in
// order). Differences: the key keeps the metadata words themselves and compares them, so two tensors'
// metadata that collide in the 64-bit hash do not share an entry; values are released by their own
// destructors (the adaptors store shared pointers) instead of through a destructor callback.
#ifndef INFINICORE_AMD_LRU_CACHE_H
#define INFINICORE_AMD_LRU_CACHE_H

#include <cstddef>
#include <cstdint>
#include <limits>
#include <list>
#include <optional>
#include <unordered_map>
#include <utility>
#include <vector>

namespace infinicore_amd {

// The words a descriptor depends on, with the reference's fold as the hash.
struct MetaKey {
    std::vector<int64_t> words;

    void add(int64_t w) { words.push_back(w); }
    // dtype, rank, then every extent, then every stride (hash.hpp:24-30, with the rank added: the word runs
    // of the tensors are concatenated, and without it two argument lists whose ranks differ could spell the
    // same words); an absent optional tensor is a single 0 after its presence flag (hash.hpp:35-40).
    void addTensor(int dtype, size_t ndim, const size_t *shape, const ptrdiff_t *strides) {
        add(dtype);
        add(static_cast<int64_t>(ndim));
        for (size_t i = 0; i < ndim; ++i) {
            add(static_cast<int64_t>(shape[i]));
        }
        // contiguous strides spelled out, so that NULL strides and explicit contiguous ones are one key
        ptrdiff_t running = 1;
        std::vector<int64_t> s(ndim);
        for (size_t i = ndim; i-- > 0;) {
            s[i] = strides ? static_cast<int64_t>(strides[i]) : static_cast<int64_t>(running);
            running *= static_cast<ptrdiff_t>(shape[i]);
        }
        words.insert(words.end(), s.begin(), s.end());
    }
    bool operator==(const MetaKey &other) const { return words == other.words; }
    size_t hash() const {
        size_t seed = 0;
        for (int64_t w : words) {
            seed ^= std::hash<int64_t>{}(w) + 0x9e3779b9 + (seed << 6) + (seed >> 2);
        }
        return seed;
    }
};

struct MetaKeyHash {
    size_t operator()(const MetaKey &k) const { return k.hash(); }
};

template <typename Key, typename Value, typename Hash = std::hash<Key>>
class LruCache {
public:
    explicit LruCache(size_t capacity = 100) { setCapacityOnly(capacity); }

    std::optional<Value> get(const Key &key) {
        auto it = map_.find(key);
        if (it == map_.end()) {
            ++misses_;
            return std::nullopt;
        }
        ++hits_;
        items_.splice(items_.begin(), items_, it->second); // most recent at the front
        return it->second->second;
    }

    void put(const Key &key, Value value) {
        auto it = map_.find(key);
        if (it != map_.end()) {
            it->second->second = std::move(value);
            items_.splice(items_.begin(), items_, it->second);
            return;
        }
        while (items_.size() >= capacity_) {
            evictOldest();
        }
        items_.emplace_front(key, std::move(value));
        map_[key] = items_.begin();
    }

    void setCapacity(size_t capacity) {
        setCapacityOnly(capacity);
        while (items_.size() > capacity_) {
            evictOldest();
        }
    }

    void clear() {
        map_.clear();
        items_.clear();
    }

    bool contains(const Key &key) const { return map_.find(key) != map_.end(); }
    size_t size() const { return items_.size(); }
    uint64_t hits() const { return hits_; }
    uint64_t misses() const { return misses_; }

private:
    void setCapacityOnly(size_t capacity) {
        capacity_ = capacity == 0 ? std::numeric_limits<size_t>::max() : capacity;
    }
    void evictOldest() {
        if (!items_.empty()) {
            map_.erase(items_.back().first);
            items_.pop_back();
        }
    }

    using Item = std::pair<Key, Value>;
    std::list<Item> items_;
    std::unordered_map<Key, typename std::list<Item>::iterator, Hash> map_;
    size_t capacity_;
    uint64_t hits_ = 0, misses_ = 0;
};

} // namespace infinicore_amd

#endif
