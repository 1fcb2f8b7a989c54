// Page-id allocator of the cache manager (control plane only: it owns no tensor memory).
//
// Same contract as the reference's pool (core/include/distie/block_pool.h:16-44,
// core/src/block_pool.cpp:46-114): ids 0..n-1, a fresh pool hands out 0,1,2,..., a freed id
// is the next one handed out (LIFO), allocate and free are all-or-nothing, a free of an id
// that is out of range, not in use, or named twice changes nothing and reports an error.
// The same class serves pages of a cache group and per-request state slots.
//
// Exposed as a C interface for ctypes: no Python headers are needed to build it.

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

namespace {

class IdPool {
 public:
  explicit IdPool(int64_t n) : size_(n), held_(static_cast<size_t>(n), 0) {
    stack_.resize(static_cast<size_t>(n));
    for (int64_t i = 0; i < n; ++i) stack_[static_cast<size_t>(i)] = static_cast<int32_t>(n - 1 - i);
    log_ = [] {
      const char* e = std::getenv("DISTIE_MEMORY_LOG");
      return e != nullptr && std::strcmp(e, "1") == 0;
    }();
    note("pool of " + std::to_string(n) + " ids");
  }

  // 0 = done; 1 = fewer than `count` ids are free (nothing taken).
  int take(int64_t count, int32_t* out) {
    std::lock_guard<std::mutex> guard(lock_);
    if (count < 0 || static_cast<size_t>(count) > stack_.size()) {
      note("take " + std::to_string(count) + " refused, free " + std::to_string(stack_.size()));
      return 1;
    }
    for (int64_t i = 0; i < count; ++i) {
      const int32_t id = stack_.back();
      stack_.pop_back();
      held_[static_cast<size_t>(id)] = 1;
      out[i] = id;
    }
    return 0;
  }

  // 0 = done; 2 = some id is invalid (nothing given back), `why` says which.
  int give(const int32_t* ids, int64_t count, std::string* why) {
    std::lock_guard<std::mutex> guard(lock_);
    // marks: 1 = held, 2 = held and named in this call
    int64_t checked = 0;
    int status = 0;
    for (; checked < count; ++checked) {
      const int32_t id = ids[checked];
      if (id < 0 || id >= size_) {
        *why = "id out of range: " + std::to_string(id);
        status = 2;
        break;
      }
      uint8_t& mark = held_[static_cast<size_t>(id)];
      if (mark == 0) {
        *why = "id is not in use (double free): " + std::to_string(id);
        status = 2;
        break;
      }
      if (mark == 2) {
        *why = "id named twice: " + std::to_string(id);
        status = 2;
        break;
      }
      mark = 2;
    }
    if (status != 0) {
      for (int64_t i = 0; i < checked; ++i) held_[static_cast<size_t>(ids[i])] = 1;
      return status;
    }
    for (int64_t i = 0; i < count; ++i) {
      held_[static_cast<size_t>(ids[i])] = 0;
      stack_.push_back(ids[i]);
    }
    return 0;
  }

  int64_t size() const { return size_; }
  int64_t free_count() {
    std::lock_guard<std::mutex> guard(lock_);
    return static_cast<int64_t>(stack_.size());
  }
  int is_held(int32_t id) {
    std::lock_guard<std::mutex> guard(lock_);
    return (id >= 0 && id < size_) ? (held_[static_cast<size_t>(id)] != 0) : -1;
  }

 private:
  void note(const std::string& text) const {
    if (log_) std::fprintf(stderr, "[distie_amd.memory] %s\n", text.c_str());
  }
  std::mutex lock_;
  int64_t size_;
  std::vector<int32_t> stack_;   // free ids; the back is handed out next
  std::vector<uint8_t> held_;
  bool log_ = false;
};

}  // namespace

extern "C" {

void* distie_pool_create(int64_t n) {
  if (n < 1 || n > INT32_MAX) return nullptr;
  return new (std::nothrow) IdPool(n);
}

void distie_pool_destroy(void* pool) { delete static_cast<IdPool*>(pool); }

int distie_pool_take(void* pool, int64_t count, int32_t* out) {
  return static_cast<IdPool*>(pool)->take(count, out);
}

int distie_pool_give(void* pool, const int32_t* ids, int64_t count, char* why, int64_t why_len) {
  std::string text;
  const int status = static_cast<IdPool*>(pool)->give(ids, count, &text);
  if (status != 0 && why != nullptr && why_len > 0) {
    std::strncpy(why, text.c_str(), static_cast<size_t>(why_len - 1));
    why[why_len - 1] = '\0';
  }
  return status;
}

int64_t distie_pool_size(void* pool) { return static_cast<IdPool*>(pool)->size(); }
int64_t distie_pool_free_count(void* pool) { return static_cast<IdPool*>(pool)->free_count(); }
int distie_pool_is_held(void* pool, int32_t id) { return static_cast<IdPool*>(pool)->is_held(id); }

}  // extern "C"
