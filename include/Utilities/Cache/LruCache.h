// Thread-safe least-recently-used map (reference: Utilities/Cache/LruCache.h:11-146).  Holds compiled kernels
// (10 000 entries) and per-equation plans (128 entries).
#pragma once

#include <cstddef>
#include <functional>
#include <list>
#include <mutex>
#include <optional>
#include <unordered_map>
#include <utility>

template <typename Key, typename Value, typename Hash = std::hash<Key>>
class LruCacheThreadSafe {
   public:
    explicit LruCacheThreadSafe(size_t capacity) : capacity(capacity ? capacity : 1) {}

    std::optional<Value> get(const Key& key) {
        std::lock_guard<std::mutex> lock(mutex);
        auto it = index.find(key);
        if (it == index.end()) return std::nullopt;
        order.splice(order.begin(), order, it->second);
        return it->second->second;
    }

    void put(const Key& key, Value value) {
        std::lock_guard<std::mutex> lock(mutex);
        auto it = index.find(key);
        if (it != index.end()) {
            it->second->second = std::move(value);
            order.splice(order.begin(), order, it->second);
            return;
        }
        order.emplace_front(key, std::move(value));
        index[key] = order.begin();
        while (index.size() > capacity) {
            index.erase(order.back().first);
            order.pop_back();
        }
    }

    // Returns the cached value or stores and returns make().  make() runs outside the lock, so two threads may both
    // build the value; the first one stored wins and both get that one.
    template <typename Make>
    Value getOrCreate(const Key& key, Make&& make) {
        if (auto hit = get(key)) return *hit;
        Value built = make();
        std::lock_guard<std::mutex> lock(mutex);
        auto it = index.find(key);
        if (it != index.end()) return it->second->second;
        order.emplace_front(key, built);
        index[key] = order.begin();
        while (index.size() > capacity) {
            index.erase(order.back().first);
            order.pop_back();
        }
        return built;
    }

    size_t size() const {
        std::lock_guard<std::mutex> lock(mutex);
        return index.size();
    }

    void clear() {
        std::lock_guard<std::mutex> lock(mutex);
        index.clear();
        order.clear();
    }

   private:
    const size_t capacity;
    mutable std::mutex mutex;
    std::list<std::pair<Key, Value>> order;
    std::unordered_map<Key, typename std::list<std::pair<Key, Value>>::iterator, Hash> index;
};
