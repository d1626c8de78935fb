// The engine's CPU path on long block lists, from C++ through the C ABI: the
// groups of the reference's pegaflow-core/benches/cpu_path.rs that sit on the
// save -> query -> load path (save_flush_unique :389-420, save_flush_cpu_
// multilayer_61 :457-492, save_flush_dtoh_multilayer_61 :570-606, save_flush_
// transfer_fragmentation :608-657, load_transfer_fragmentation :659-709,
// query_prefetch_lease :711-740, load_submit_wait :742-774), with its shapes:
// block counts 128 / 1024 / 8192 / 32768, 1 KiB blocks (1-byte blocks in the
// 61-layer CPU group, whose layers all name one source buffer), one layer
// "layer_0" or 61 layers "layer_{i}", block ids 0..n or every other slot,
// 16-byte hashes (salt, index), block i filled with (i % 251) + 1, a pool of
// four times the payload + 64 MiB, fresh hashes and an untimed cache clean-up
// per save iteration.  The groups around the MetaServer and the two that time
// internal stages of the reference's asynchronous save are left out: a save
// here returns when its blocks are queryable, so "save + flush" is one call.
// 3 warm-up and 10 timed iterations per case; the mean is reported.  Every load
// case checks the bytes that arrived.  Prints one JSON line; a last line
// "all ok" and exit status 0 = pass.  Argument "quick" runs the two smaller
// block counts only.
#include "../../include/pegahip.h"

#include <chrono>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#define OK(x)                                                                          \
  do {                                                                                 \
    int st_ = (x);                                                                     \
    if (st_ != 0) {                                                                    \
      printf("FAIL line %d: %s -> %d %s\n", __LINE__, #x, st_, pf_last_error());       \
      return 1;                                                                        \
    }                                                                                  \
  } while (0)

namespace {

constexpr int kWarm = 3, kIters = 10;
constexpr int kLayers61 = 61;

struct Row {
  std::string group, param;
  double mean_us;
  uint64_t bytes, elements;
  bool has_profile = false;
  pf_save_profile profile{};  // phases of the last timed save
};
std::vector<Row> g_rows;

double now_us() {
  return std::chrono::duration<double, std::micro>(
             std::chrono::steady_clock::now().time_since_epoch())
      .count();
}

struct Hashes {
  std::vector<uint8_t> bytes;
  std::vector<const uint8_t*> ptr;
  std::vector<uint32_t> len;
  void make(uint64_t n, uint64_t salt) {  // cpu_path.rs:786-795
    bytes.resize(n * 16);
    ptr.resize(n);
    len.assign(n, 16);
    for (uint64_t i = 0; i < n; ++i) {
      memcpy(&bytes[i * 16], &salt, 8);
      memcpy(&bytes[i * 16 + 8], &i, 8);
      ptr[i] = &bytes[i * 16];
    }
  }
};

struct Fixture {
  pf_engine_t e = nullptr;
  uint64_t dev = 0, dev_bytes = 0, block = 0, n = 0;
  int layers = 1;
  std::vector<std::string> names;
  std::vector<const char*> cnames;
  std::vector<uint64_t> ids;
  std::vector<int64_t> dest;
  std::vector<uint8_t> pattern;

  // registered: slots per layer; distinct: every layer its own slice of the buffer.
  int init(uint64_t registered, uint64_t bytes_per_block, int n_layers, bool distinct, int mode,
           bool strided, uint64_t n_blocks) {
    block = bytes_per_block;
    n = n_blocks;
    layers = n_layers;
    const uint64_t layer_bytes = registered * block;
    dev_bytes = distinct ? layer_bytes * n_layers : layer_bytes;
    OK(pf_set_device(0));
    OK(pf_dev_malloc(dev_bytes, &dev));
    pattern.resize(dev_bytes);
    for (uint64_t i = 0; i < dev_bytes / block; ++i) {  // cpu_path.rs:810-815
      memset(&pattern[i * block], static_cast<int>(i % 251) + 1, block);
    }
    OK(pf_dev_copy_from_host(dev, pattern.data(), dev_bytes));
    pf_engine_config cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.pool_size = n * block * n_layers * 4 + (64ull << 20);
    cfg.pool_shards = 1;
    cfg.unit_size_hint = block;
    OK(pf_engine_create(&cfg, &e));
    names.resize(n_layers);
    cnames.resize(n_layers);
    for (int l = 0; l < n_layers; ++l) {
      names[l] = "layer_" + std::to_string(l);
      cnames[l] = names[l].c_str();
    }
    std::vector<uint64_t> ptrs(n_layers), sizes(n_layers, layer_bytes), nbs(n_layers, registered),
        bpb(n_layers, block), kvs(n_layers, 0), segs(n_layers, 1);
    for (int l = 0; l < n_layers; ++l) ptrs[l] = dev + (distinct ? l * layer_bytes : 0);
    OK(pf_engine_register_context_layer_batch(e, "cpu-path-bench", "cpu-path", 0, 0, 0, 1, 1,
                                              n_layers, cnames.data(), ptrs.data(), sizes.data(),
                                              nbs.data(), bpb.data(), kvs.data(), segs.data(),
                                              nullptr, nullptr, mode, 0));
    ids.resize(n);
    dest.resize(n);
    for (uint64_t i = 0; i < n; ++i) {
      ids[i] = strided ? 2 * i : i;
      dest[i] = static_cast<int64_t>(ids[i]);
    }
    return 0;
  }
  int save(const Hashes& h) {
    std::vector<pf_layer_save> saves(layers);
    for (int l = 0; l < layers; ++l) saves[l] = {cnames[l], ids.data(), h.ptr.data(), h.len.data(), n};
    OK(pf_engine_batch_save(e, "cpu-path-bench", 0, 0, 0, saves.data(), layers));
    return 0;
  }
  int query(const Hashes& h, uint64_t* lease) {
    uint64_t hits = 0;
    OK(pf_engine_query_prefix(e, "cpu-path-bench", h.ptr.data(), h.len.data(), n, &hits, lease));
    if (hits != n) {
      printf("FAIL: %llu of %llu blocks hit\n", (unsigned long long)hits, (unsigned long long)n);
      return 1;
    }
    return 0;
  }
  int load(uint64_t lease) {
    const char* const* groups[1] = {cnames.data()};
    const uint64_t sizes[1] = {static_cast<uint64_t>(layers)};
    const int64_t* dd[1] = {dest.data()};
    pf_task_t t = nullptr;
    OK(pf_engine_batch_load(e, "cpu-path-bench", 0, 0, 1, groups, sizes, lease, dd, n, nullptr, &t));
    pf_task_result r;
    OK(pf_task_wait(t, -1, &r));
    OK(pf_task_destroy(t));
    return r.status;
  }
  // The device buffer holds the pattern in every slot the ids name.
  int check_device(const char* what) {
    std::vector<uint8_t> got(dev_bytes);
    OK(pf_dev_copy_to_host(got.data(), dev, dev_bytes));
    const uint64_t per_layer = dev_bytes / block;
    for (uint64_t i = 0; i < n; ++i) {
      if (ids[i] >= per_layer) continue;
      if (memcmp(&got[ids[i] * block], &pattern[ids[i] * block], block)) {
        printf("MISMATCH %s: block id %llu\n", what, (unsigned long long)ids[i]);
        return 2;
      }
    }
    return 0;
  }
  void close() {
    if (e) {
      (void)pf_engine_unregister_instance(e, "cpu-path-bench");
      (void)pf_engine_destroy(e);
    }
    if (dev) (void)pf_dev_free(dev);
    e = nullptr;
    dev = 0;
  }
};

int save_group(const char* group, const std::string& param, Fixture& f, uint64_t bytes,
               uint64_t elements) {
  double total = 0;
  Hashes h;
  pf_save_profile profile{};
  for (int it = 0; it < kWarm + kIters; ++it) {
    h.make(f.n, static_cast<uint64_t>(it) + 1);
    const double t0 = now_us();
    if (f.save(h)) return 1;
    if (it >= kWarm) total += now_us() - t0;
    OK(pf_engine_last_save_profile(f.e, &profile));
    if (it + 1 == kWarm + kIters) {  // what the last save stored is what a load brings back
      uint64_t lease = 0;
      if (f.query(h, &lease)) return 1;
      OK(pf_dev_memset(f.dev, 0, f.dev_bytes));
      if (f.load(lease)) return 1;
      if (f.check_device(group)) return 2;
    }
    (void)pf_engine_evict_all(f.e);  // cleanup_memory_cache, untimed
  }
  g_rows.push_back({group, param, total / kIters, bytes, elements, true, profile});
  return 0;
}

int primed(Fixture& f, Hashes* h) {
  h->make(f.n, 0);
  return f.save(*h);
}

}  // namespace

int main(int argc, char** argv) {
  const bool quick = argc > 1 && !strcmp(argv[1], "quick");
  std::vector<uint64_t> cases = {128, 1024, 8192, 32768};
  std::vector<uint64_t> dtoh_cases = {128, 1024, 8192};
  std::vector<uint64_t> frag_cases = {1024, 8192};
  if (quick) cases = {128, 1024}, dtoh_cases = {128, 1024}, frag_cases = {1024};
  const uint64_t kBlock = 1024;

  for (uint64_t n : cases) {
    printf("save_flush_unique %llu\n", (unsigned long long)n);
    fflush(stdout);
    Fixture f;
    if (f.init(n, kBlock, 1, false, PF_MODE_DIRECT, false, n)) return 1;
    if (save_group("save_flush_unique", std::to_string(n), f, n * kBlock, n)) return 1;
    f.close();
  }
  for (uint64_t n : cases) {
    printf("save_flush_cpu_multilayer_61 %llu\n", (unsigned long long)n);
    fflush(stdout);
    Fixture f;
    if (f.init(n, 1, kLayers61, false, PF_MODE_DIRECT, false, n)) return 1;
    if (save_group("save_flush_cpu_multilayer_61", std::to_string(n), f, n * kLayers61,
                   n * kLayers61)) {
      return 1;
    }
    f.close();
  }
  for (uint64_t n : dtoh_cases) {
    printf("save_flush_dtoh_multilayer_61 %llu\n", (unsigned long long)n);
    fflush(stdout);
    Fixture f;
    if (f.init(n, kBlock, kLayers61, true, PF_MODE_DIRECT, false, n)) return 1;
    if (save_group("save_flush_dtoh_multilayer_61", std::to_string(n), f, n * kLayers61 * kBlock,
                   n * kLayers61)) {
      return 1;
    }
    f.close();
  }
  for (uint64_t n : frag_cases) {
    for (int mode : {PF_MODE_DIRECT, PF_MODE_KERNEL}) {
      for (bool strided : {false, true}) {
        const std::string param = std::string(mode == PF_MODE_DIRECT ? "direct" : "kernel") +
                                  (strided ? "_strided_device/" : "_contiguous/") +
                                  std::to_string(n);
        printf("transfer_fragmentation %s\n", param.c_str());
        fflush(stdout);
        {
          Fixture f;
          if (f.init(strided ? 2 * n : n, kBlock, 1, false, mode, strided, n)) return 1;
          if (save_group("save_flush_transfer_fragmentation", param, f, n * kBlock, n)) return 1;
          f.close();
        }
        Fixture f;
        if (f.init(strided ? 2 * n : n, kBlock, 1, false, mode, strided, n)) return 1;
        Hashes h;
        if (primed(f, &h)) return 1;
        OK(pf_dev_memset(f.dev, 0, f.dev_bytes));
        double total = 0;
        for (int it = 0; it < kWarm + kIters; ++it) {
          uint64_t lease = 0;
          if (f.query(h, &lease)) return 1;
          const double t0 = now_us();
          if (f.load(lease)) return 1;
          if (it >= kWarm) total += now_us() - t0;
        }
        if (f.check_device("load_transfer_fragmentation")) return 2;
        g_rows.push_back({"load_transfer_fragmentation", param, total / kIters, n * kBlock, n});
        f.close();
      }
    }
  }
  for (uint64_t n : cases) {
    printf("query_prefetch_lease / load_submit_wait %llu\n", (unsigned long long)n);
    fflush(stdout);
    Fixture f;
    if (f.init(n, kBlock, 1, false, PF_MODE_DIRECT, false, n)) return 1;
    Hashes h;
    if (primed(f, &h)) return 1;
    double total = 0;
    for (int it = 0; it < kWarm + kIters; ++it) {
      uint64_t lease = 0;
      const double t0 = now_us();
      if (f.query(h, &lease)) return 1;
      if (it >= kWarm) total += now_us() - t0;
      OK(pf_engine_release_lease(f.e, lease));
    }
    g_rows.push_back({"query_prefetch_lease", std::to_string(n), total / kIters, 0, n});
    OK(pf_dev_memset(f.dev, 0, f.dev_bytes));
    total = 0;
    for (int it = 0; it < kWarm + kIters; ++it) {
      uint64_t lease = 0;
      if (f.query(h, &lease)) return 1;
      const double t0 = now_us();
      if (f.load(lease)) return 1;
      if (it >= kWarm) total += now_us() - t0;
    }
    if (f.check_device("load_submit_wait")) return 2;
    g_rows.push_back({"load_submit_wait", std::to_string(n), total / kIters, n * kBlock, n});
    f.close();
  }

  printf("{\"rows\": [");
  for (size_t i = 0; i < g_rows.size(); ++i) {
    const Row& r = g_rows[i];
    printf("%s{\"group\": \"%s\", \"case\": \"%s\", \"mean_us\": %.1f, \"ns_per_block\": %.1f, "
           "\"MiB_per_s\": %.1f",
           i ? ", " : "", r.group.c_str(), r.param.c_str(), r.mean_us,
           r.mean_us * 1e3 / static_cast<double>(r.elements),
           r.bytes ? static_cast<double>(r.bytes) / r.mean_us * 1e6 / (1 << 20) : 0.0);
    if (r.has_profile) {
      const pf_save_profile& q = r.profile;
      printf(", \"last_save_us\": {\"validate\": %.1f, \"filter\": %.1f, \"alloc\": %.1f, "
             "\"assemble_during_transfer\": %.1f, \"transfer\": %.1f, \"publish\": %.1f}",
             q.validate_ms * 1e3, q.filter_ms * 1e3, q.alloc_ms * 1e3, q.assemble_ms * 1e3,
             q.transfer_ms * 1e3, q.publish_ms * 1e3);
    }
    printf("}");
  }
  printf("]}\nall ok\n");
  return 0;
}
