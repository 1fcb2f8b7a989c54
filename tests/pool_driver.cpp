// Exercises the id pool of the cache manager through its C interface from eight threads; built and run by
// tests/test_cache_manager.py under the address, undefined-behaviour and thread sanitizers.
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <thread>
#include <vector>

extern "C" {
void* distie_pool_create(int64_t n);
void distie_pool_destroy(void* pool);
int distie_pool_take(void* pool, int64_t count, int32_t* out);
int distie_pool_give(void* pool, const int32_t* ids, int64_t count, char* why, int64_t why_len);
int64_t distie_pool_size(void* pool);
int64_t distie_pool_free_count(void* pool);
int distie_pool_is_held(void* pool, int32_t id);
}

int main() {
  const int64_t n = 96;
  void* pool = distie_pool_create(n);
  if (pool == nullptr || distie_pool_size(pool) != n || distie_pool_free_count(pool) != n) return 1;
  std::atomic<int> wrong{0};
  std::vector<std::thread> threads;
  for (int t = 0; t < 8; ++t)
    threads.emplace_back([&, t] {
      int32_t ids[5];
      char why[128];
      for (int round = 0; round < 2000; ++round) {
        const int64_t count = 1 + (round + t) % 5;
        if (distie_pool_take(pool, count, ids) != 0) continue;           // the pool was empty: all or nothing
        for (int64_t i = 0; i < count; ++i)
          if (ids[i] < 0 || ids[i] >= n || !distie_pool_is_held(pool, ids[i])) ++wrong;
        if (distie_pool_give(pool, ids, count, why, sizeof(why)) != 0) ++wrong;
      }
    });
  for (auto& th : threads) th.join();
  if (wrong.load() != 0 || distie_pool_free_count(pool) != n) return 2;
  // giving back twice, or an id that was never handed out, is refused with a reason and changes nothing
  int32_t one[1];
  char why[128] = {0};
  if (distie_pool_take(pool, 1, one) != 0) return 3;
  if (distie_pool_give(pool, one, 1, why, sizeof(why)) != 0) return 4;
  if (distie_pool_give(pool, one, 1, why, sizeof(why)) == 0 || why[0] == '\0') return 5;
  const int32_t outside[1] = {static_cast<int32_t>(n)};
  if (distie_pool_give(pool, outside, 1, why, sizeof(why)) == 0) return 6;
  if (distie_pool_free_count(pool) != n) return 7;
  distie_pool_destroy(pool);
  std::puts("pool driver: fine");
  return 0;
}
