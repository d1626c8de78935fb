// Several threads drive one engine through the C ABI at once: every thread
// registers its own source and destination instance in a shared namespace,
// then saves, queries and loads blocks drawn from a common universe of hashes
// while the pinned pool is too small for that universe, so saves of one thread
// evict what another thread queried a moment ago.  The bytes of a block are a
// pure function of (hash, layer, segment), so whichever thread stored the block
// that a lease pins, the loader can check every byte.  This follows the
// reference's concurrency contract: one engine shared by all connections,
// leases pin blocks against eviction until their load is done
// (pegaflow-core/src/lease.rs, storage/mod.rs:294-330).
// Built by `make -C pegaflow_amd/csrc native-tests`; run by
// tests/test_gpu_native.py.  Exit status 0 and a last line "all ok" = pass.
#include "../../include/pegahip.h"
#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <thread>
#include <vector>

namespace {

constexpr int kThreads = 4;
constexpr int kRounds = 120;
constexpr int kLayers = 3;
constexpr int kSegments = 2;
constexpr uint64_t kBlocks = 128;      // blocks per layer of every cache
constexpr uint64_t kSeg = 4096;        // bytes per (block, segment)
constexpr uint64_t kPerRound = 24;     // blocks saved per round
constexpr uint64_t kUniverse = 1536;   // distinct hashes: 36 MiB of blocks over a 16 MiB pool
constexpr uint64_t kLayerBytes = kSegments * kBlocks * kSeg;

std::atomic<int> failures{0};
std::atomic<uint64_t> blocks_loaded{0}, blocks_missed{0}, saves_refused{0};

void fill_block(uint8_t* out, uint64_t hash, int layer, int seg) {
  uint32_t x = static_cast<uint32_t>(hash * 2654435761u) ^ (layer * 40503u) ^ (seg * 977u);
  for (uint64_t j = 0; j < kSeg; j += 4) {
    x = x * 1664525u + 1013904223u;
    std::memcpy(out + j, &x, 4);
  }
}

#define CHECK(x)                                                                          \
  do {                                                                                    \
    int st_ = (x);                                                                        \
    if (st_ != 0) {                                                                       \
      printf("thread %d FAIL line %d: %s -> %d %s\n", tid, __LINE__, #x, st_, pf_last_error()); \
      fflush(stdout);                                                                     \
      failures++;                                                                         \
      return;                                                                             \
    }                                                                                     \
  } while (0)

void worker(pf_engine_t e, int tid) {
  if (hipSetDevice(0) != hipSuccess) { failures++; return; }
  std::mt19937_64 rng(1000 + tid);
  const std::string src_name = "src" + std::to_string(tid), dst_name = "dst" + std::to_string(tid);
  std::vector<void*> src(kLayers), dst(kLayers);
  std::vector<std::string> names(kLayers);
  std::vector<const char*> cn(kLayers);
  for (int l = 0; l < kLayers; ++l) {
    if (hipMalloc(&src[l], kLayerBytes) || hipMalloc(&dst[l], kLayerBytes)) { failures++; return; }
    names[l] = "model.layers." + std::to_string(l) + ".attn";
    cn[l] = names[l].c_str();
  }
  std::vector<uint64_t> sz(kLayers, kLayerBytes), nbs(kLayers, kBlocks), bpb(kLayers, kSeg),
      kvs(kLayers, kBlocks * kSeg), sg(kLayers, kSegments);
  for (int which = 0; which < 2; ++which) {
    std::vector<uint64_t> ptrs(kLayers);
    for (int l = 0; l < kLayers; ++l) ptrs[l] = reinterpret_cast<uint64_t>(which ? dst[l] : src[l]);
    CHECK(pf_engine_register_context_layer_batch(
        e, which ? dst_name.c_str() : src_name.c_str(), "ns", 0, 0, 0, 1, 1, kLayers, cn.data(),
        ptrs.data(), sz.data(), nbs.data(), bpb.data(), kvs.data(), sg.data(), nullptr, nullptr,
        tid % 2 /* direct and kernel instances side by side */, 0));
  }
  std::vector<uint8_t> image(kLayerBytes), got(kLayerBytes);
  std::vector<uint64_t> slots(kBlocks);
  for (int round = 0; round < kRounds; ++round) {
    // A run of consecutive hashes from the universe, so prefixes overlap between threads.
    const uint64_t first = rng() % (kUniverse - kPerRound);
    std::vector<uint64_t> hashes(kPerRound);
    for (uint64_t i = 0; i < kPerRound; ++i) hashes[i] = first + i;
    for (uint64_t i = 0; i < kBlocks; ++i) slots[i] = i;
    std::shuffle(slots.begin(), slots.end(), rng);
    std::vector<uint64_t> ids(slots.begin(), slots.begin() + kPerRound);
    for (int l = 0; l < kLayers; ++l) {
      for (uint64_t i = 0; i < kPerRound; ++i) {
        for (int s = 0; s < kSegments; ++s) {
          fill_block(&image[s * kBlocks * kSeg + ids[i] * kSeg], hashes[i], l, s);
        }
      }
      if (hipMemcpy(src[l], image.data(), kLayerBytes, hipMemcpyHostToDevice)) { failures++; return; }
    }
    // The engine's workers use streams of their own, which do not wait for the
    // null stream: everything written above has to be in place before the save.
    if (hipDeviceSynchronize()) { failures++; return; }
    std::vector<const uint8_t*> hp(kPerRound);
    std::vector<uint32_t> hl(kPerRound, 8);
    for (uint64_t i = 0; i < kPerRound; ++i) hp[i] = reinterpret_cast<const uint8_t*>(&hashes[i]);
    std::vector<pf_layer_save> saves(kLayers);
    for (int l = 0; l < kLayers; ++l) saves[l] = {cn[l], ids.data(), hp.data(), hl.data(), kPerRound};
    int st = pf_engine_batch_save(e, src_name.c_str(), 0, 0, 0, saves.data(), kLayers);
    if (st != 0) {
      // Every other block may be pinned by the leases of the other threads for
      // a moment: a refused allocation is a legal outcome, anything else is not.
      if (st != PF_ERR_STORAGE || std::strstr(pf_last_error(), "pinned pool exhausted") == nullptr) {
        printf("thread %d round %d: save -> %d %s\n", tid, round, st, pf_last_error());
        failures++;
        return;
      }
      saves_refused++;
    }
    uint64_t hits = 0, lease = 0;
    CHECK(pf_engine_query_prefix(e, dst_name.c_str(), hp.data(), hl.data(), kPerRound, &hits, &lease));
    blocks_missed += kPerRound - hits;
    if (hits == 0) continue;
    if (round % 7 == 3) {  // sometimes give the lease back unused
      CHECK(pf_engine_release_lease(e, lease));
      continue;
    }
    std::shuffle(slots.begin(), slots.end(), rng);
    std::vector<int64_t> dest(slots.begin(), slots.begin() + hits);
    for (int l = 0; l < kLayers; ++l) {
      if (hipMemset(dst[l], 0xEE, kLayerBytes)) { failures++; return; }
    }
    if (hipDeviceSynchronize()) { failures++; return; }  // hipMemset returns before it has run
    const char* const* groups[1] = {cn.data()};
    uint64_t group_sizes[1] = {kLayers};
    const int64_t* dd[1] = {dest.data()};
    pf_task_t task = nullptr;
    CHECK(pf_engine_batch_load(e, dst_name.c_str(), 0, 0, 1, groups, group_sizes, lease, dd, hits,
                               nullptr, &task));
    pf_task_result result;
    CHECK(pf_task_wait(task, -1, &result));
    CHECK(pf_task_destroy(task));
    std::vector<uint8_t> want(kSeg);
    std::vector<bool> written(kBlocks, false);
    for (uint64_t i = 0; i < hits; ++i) written[dest[i]] = true;
    for (int l = 0; l < kLayers; ++l) {
      if (hipMemcpy(got.data(), dst[l], kLayerBytes, hipMemcpyDeviceToHost)) { failures++; return; }
      for (int s = 0; s < kSegments; ++s) {
        for (uint64_t i = 0; i < hits; ++i) {
          fill_block(want.data(), hashes[i], l, s);
          if (std::memcmp(&got[s * kBlocks * kSeg + dest[i] * kSeg], want.data(), kSeg) != 0) {
            const uint8_t* g = &got[s * kBlocks * kSeg + dest[i] * kSeg];
            uint64_t at = 0;
            while (g[at] == want[at]) ++at;
            printf("thread %d round %d: MISMATCH layer %d segment %d hash %llu position %llu of %llu "
                   "at byte %llu: got %02x %02x %02x %02x want %02x %02x %02x %02x\n",
                   tid, round, l, s, static_cast<unsigned long long>(hashes[i]),
                   static_cast<unsigned long long>(i), static_cast<unsigned long long>(hits),
                   static_cast<unsigned long long>(at), g[at], g[at + 1], g[at + 2], g[at + 3],
                   want[at], want[at + 1], want[at + 2], want[at + 3]);
            failures++;
            return;
          }
        }
        for (uint64_t b = 0; b < kBlocks; ++b) {
          if (written[b]) continue;
          const uint8_t* p = &got[s * kBlocks * kSeg + b * kSeg];
          for (uint64_t j = 0; j < kSeg; ++j) {
            if (p[j] != 0xEE) {
              printf("thread %d round %d: block %llu outside the load was written\n", tid, round,
                     static_cast<unsigned long long>(b));
              failures++;
              return;
            }
          }
        }
      }
    }
    blocks_loaded += hits;
  }
  CHECK(pf_engine_unregister_instance(e, src_name.c_str()));
  CHECK(pf_engine_unregister_instance(e, dst_name.c_str()));
  for (int l = 0; l < kLayers; ++l) {
    (void)hipFree(src[l]);
    (void)hipFree(dst[l]);
  }
}

}  // namespace

int main() {
  pf_engine_config cfg;
  std::memset(&cfg, 0, sizeof cfg);
  cfg.pool_size = 16ull << 20;
  cfg.pool_shards = 2;
  pf_engine_t e = nullptr;
  if (pf_engine_create(&cfg, &e) != 0) {
    printf("engine: %s\n", pf_last_error());
    return 1;
  }
  std::vector<std::thread> threads;
  for (int t = 0; t < kThreads; ++t) threads.emplace_back(worker, e, t);
  for (auto& t : threads) t.join();
  if (pf_engine_destroy(e) != 0) failures++;
  printf("threads=%d rounds=%d loaded=%llu missed=%llu saves_refused=%llu failures=%d\n", kThreads,
         kRounds, static_cast<unsigned long long>(blocks_loaded.load()),
         static_cast<unsigned long long>(blocks_missed.load()),
         static_cast<unsigned long long>(saves_refused.load()), failures.load());
  printf(failures.load() ? "FAILED\n" : "all ok\n");
  return failures.load() ? 1 : 0;
}
