// Small transfers through the C ABI, timed from C++: wall time of one call
// followed by a stream synchronise, the shape of the reference's own transfer
// bench (pegaflow-core/benches/transfer_h2d.rs:62-109,317-339: submit +
// synchronise per iteration, 3 warm-up + 20 timed iterations of each case; here
// 20 warm-up and 200 timed, median reported).  Cases: one K/V-split layer of
// 32 KiB fragments moved by block id (1, 4 and 16 MiB), and 1024 shuffled 4 KiB
// fragments (the reference bench's smallest row) by block id, through the
// kernel backend, through the direct backend and through pf_desc_copy_noalloc;
// next to them one plain hipMemcpyAsync of the same size as the yardstick.
// Every case checks the bytes it moved.  Prints one JSON line; exit status 0 = ok.
#include "../../include/pegahip.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <random>
#include <string>
#include <vector>

#define OK(x)                                                                             \
  do {                                                                                    \
    int st_ = (x);                                                                        \
    if (st_ != 0) {                                                                       \
      fprintf(stderr, "FAIL line %d: %s -> %d %s\n", __LINE__, #x, st_, pf_last_error()); \
      return 1;                                                                           \
    }                                                                                     \
  } while (0)

namespace {

struct Row {
  std::string name;
  uint64_t bytes;
  double median_us;
};

template <typename F>
int timed(const char* name, uint64_t bytes, pf_stream_t s, std::vector<Row>* rows, F&& call) {
  for (int i = 0; i < 20; ++i) {
    int st = call();
    if (st != 0) return st;
    if (pf_stream_synchronize(s) != 0) return -1;
  }
  std::vector<double> us;
  for (int i = 0; i < 200; ++i) {
    const auto t0 = std::chrono::steady_clock::now();
    int st = call();
    if (st != 0) return st;
    if (pf_stream_synchronize(s) != 0) return -1;
    us.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
  }
  std::sort(us.begin(), us.end());
  rows->push_back({name, bytes, us[us.size() / 2]});
  return 0;
}

}  // namespace

int main() {
  OK(pf_set_device(0));
  pf_stream_t s = nullptr;
  OK(pf_stream_create(&s));
  const uint64_t kBuf = 64ull << 20;
  uint64_t dev = 0;
  OK(pf_dev_malloc(kBuf, &dev));
  pf_host_mem host;
  OK(pf_host_alloc(kBuf, PF_HOST_HIP_ALLOC, -1, &host));
  std::vector<uint8_t> pattern(kBuf);
  std::mt19937_64 rng(3);
  for (uint64_t i = 0; i < kBuf; i += 8) {
    const uint64_t v = rng();
    memcpy(&pattern[i], &v, 8);
  }
  OK(pf_dev_copy_from_host(dev, pattern.data(), kBuf));
  std::vector<Row> rows;
  std::vector<uint8_t> back(kBuf);

  // ---- one split layer by block id: [2, 1024 blocks, 32 KiB] ---------------
  pf_xfer_t x = nullptr;
  OK(pf_xfer_create(nullptr, &x));
  const uint64_t nb = 1024, seg = 32768;
  pf_kv_layout layout;
  OK(pf_layout_new(dev, 2 * nb * seg, nb, seg, nb * seg, 2, &layout));
  std::vector<uint32_t> perm(nb);
  std::iota(perm.begin(), perm.end(), 0u);
  std::shuffle(perm.begin(), perm.end(), rng);
  for (uint64_t n : {16ull, 64ull, 256ull}) {
    pf_layer_blocks lb;
    memset(&lb, 0, sizeof lb);
    lb.layout = layout;
    lb.block_ids = perm.data();
    lb.n_blocks = n;
    for (int g = 0; g < 2; ++g) {
      lb.host[g] = static_cast<uint8_t*>(host.host) + g * n * seg;
      lb.host_device[g] = host.device + g * n * seg;
      lb.host_len[g] = n * seg;
    }
    lb.host_stride = seg;
    const uint64_t bytes = 2 * n * seg;
    char name[96];
    snprintf(name, sizeof name, "block_ids_save_%lluMiB", (unsigned long long)(bytes >> 20));
    memset(host.host, 0, bytes);
    OK(timed(name, bytes, s, &rows, [&] { return pf_xfer_save(x, &lb, 1, PF_PATH_ZEROCOPY, s); }));
    for (uint64_t i = 0; i < n; ++i) {
      for (int g = 0; g < 2; ++g) {
        if (memcmp(static_cast<uint8_t*>(host.host) + g * n * seg + i * seg,
                   &pattern[g * nb * seg + perm[i] * seg], seg)) {
          fprintf(stderr, "MISMATCH save n=%llu pos %llu seg %d\n", (unsigned long long)n,
                  (unsigned long long)i, g);
          return 2;
        }
      }
    }
    OK(pf_dev_memset(dev, 0, 2 * nb * seg));
    snprintf(name, sizeof name, "block_ids_load_%lluMiB", (unsigned long long)(bytes >> 20));
    OK(timed(name, bytes, s, &rows, [&] { return pf_xfer_load(x, &lb, 1, PF_PATH_ZEROCOPY, s); }));
    OK(pf_dev_copy_to_host(back.data(), dev, 2 * nb * seg));
    for (uint64_t i = 0; i < n; ++i) {
      for (int g = 0; g < 2; ++g) {
        if (memcmp(&back[g * nb * seg + perm[i] * seg], &pattern[g * nb * seg + perm[i] * seg], seg)) {
          fprintf(stderr, "MISMATCH load n=%llu pos %llu seg %d\n", (unsigned long long)n,
                  (unsigned long long)i, g);
          return 2;
        }
      }
    }
    OK(pf_dev_copy_from_host(dev, pattern.data(), kBuf));
    snprintf(name, sizeof name, "hipMemcpyAsync_d2h_%lluMiB", (unsigned long long)(bytes >> 20));
    OK(timed(name, bytes, s, &rows, [&] { return pf_memcpy_d2h_async(host.host, dev, bytes, s); }));
    snprintf(name, sizeof name, "hipMemcpyAsync_h2d_%lluMiB", (unsigned long long)(bytes >> 20));
    OK(timed(name, bytes, s, &rows,
             [&] { return pf_memcpy_h2d_async(dev + 32 * (1ull << 20), host.host, bytes, s); }));
    OK(pf_dev_copy_from_host(dev, pattern.data(), kBuf));
  }

  // ---- 1024 x 4 KiB, shuffled, device slots of 8 KiB -----------------------
  const uint64_t n = 1024, frag = 4096;
  std::vector<uint32_t> slot(n);
  std::iota(slot.begin(), slot.end(), 0u);
  std::shuffle(slot.begin(), slot.end(), rng);
  for (auto& v : slot) v *= 2;
  pf_kv_layout small;
  OK(pf_layout_new(dev, 2 * n * frag, 2 * n, frag, 0, 1, &small));
  pf_layer_blocks lb;
  memset(&lb, 0, sizeof lb);
  lb.layout = small;
  lb.block_ids = slot.data();
  lb.n_blocks = n;
  lb.host[0] = host.host;
  lb.host_device[0] = host.device;
  lb.host_len[0] = n * frag;
  lb.host_stride = frag;
  std::vector<pf_copy_desc> descs(n);
  for (uint64_t i = 0; i < n; ++i) {
    descs[i] = {dev + slot[i] * frag, static_cast<uint8_t*>(host.host) + i * frag,
                host.device + i * frag, frag, 0, 1};
  }
  auto check_host = [&](const char* what) -> int {
    for (uint64_t i = 0; i < n; ++i) {
      if (memcmp(static_cast<uint8_t*>(host.host) + i * frag, &pattern[slot[i] * frag], frag)) {
        fprintf(stderr, "MISMATCH %s fragment %llu\n", what, (unsigned long long)i);
        return 2;
      }
    }
    memset(host.host, 0, n * frag);
    return 0;
  };
  pf_backend_t kernel = nullptr, direct = nullptr;
  OK(pf_backend_create(PF_MODE_KERNEL, &kernel));
  OK(pf_backend_create(PF_MODE_DIRECT, &direct));
  memset(host.host, 0, n * frag);
  OK(timed("block_ids_d2h_1024x4KiB", n * frag, s, &rows, [&] { return pf_xfer_save(x, &lb, 1, PF_PATH_AUTO, s); }));
  if (check_host("block ids")) return 2;
  OK(timed("kernel_backend_d2h_1024x4KiB", n * frag, s, &rows, [&] { return pf_backend_d2h(kernel, descs.data(), n, s); }));
  if (check_host("kernel backend")) return 2;
  OK(timed("direct_backend_d2h_1024x4KiB", n * frag, s, &rows, [&] { return pf_backend_d2h(direct, descs.data(), n, s); }));
  if (check_host("direct backend")) return 2;
  OK(timed("noalloc_d2h_1024x4KiB", n * frag, s, &rows, [&] { return pf_desc_copy_noalloc(descs.data(), n, 0, s); }));
  if (check_host("noalloc")) return 2;
  OK(pf_xfer_save(x, &lb, 1, PF_PATH_AUTO, s));
  OK(pf_stream_synchronize(s));
  OK(timed("block_ids_h2d_1024x4KiB", n * frag, s, &rows, [&] { return pf_xfer_load(x, &lb, 1, PF_PATH_AUTO, s); }));
  OK(timed("kernel_backend_h2d_1024x4KiB", n * frag, s, &rows, [&] { return pf_backend_h2d(kernel, descs.data(), n, s); }));
  OK(timed("direct_backend_h2d_1024x4KiB", n * frag, s, &rows, [&] { return pf_backend_h2d(direct, descs.data(), n, s); }));
  OK(timed("noalloc_h2d_1024x4KiB", n * frag, s, &rows, [&] { return pf_desc_copy_noalloc(descs.data(), n, 1, s); }));
  OK(pf_dev_copy_to_host(back.data(), dev, 2 * n * frag));
  if (memcmp(back.data(), pattern.data(), 2 * n * frag)) {
    fprintf(stderr, "MISMATCH after the 4 KiB loads\n");
    return 2;
  }

  printf("{\"unit\": \"median microseconds of call + synchronise over 200 iterations\", \"rows\": [");
  for (size_t i = 0; i < rows.size(); ++i) {
    printf("%s{\"case\": \"%s\", \"bytes\": %llu, \"us\": %.1f, \"GBps\": %.2f, \"GiBps\": %.2f}",
           i ? ", " : "", rows[i].name.c_str(), (unsigned long long)rows[i].bytes, rows[i].median_us,
           rows[i].bytes / rows[i].median_us / 1e3, rows[i].bytes / rows[i].median_us / 1e3 / 1.073741824);
  }
  printf("]}\n");
  OK(pf_backend_destroy(kernel));
  OK(pf_backend_destroy(direct));
  OK(pf_xfer_destroy(x));
  OK(pf_host_free(&host));
  OK(pf_dev_free(dev));
  OK(pf_stream_destroy(s));
  printf("all ok\n");
  return 0;
}
