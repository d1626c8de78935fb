// NUMA helpers of the pinned pool and the GPU workers: cpulist parsing,
// thread pinning, running a closure on a node, GPU -> node lookup.
// Follows pegaflow-common/src/numa.rs:17-257,340-497 of the reference; the
// GPU -> node source is the PCI device's sysfs entry, not nvidia-smi.
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <vector>

namespace pf {

// numa.rs:17-45.  UNKNOWN is u32::MAX.
struct NumaNode {
  static constexpr uint32_t kUnknown = 0xFFFFFFFFu;
  uint32_t id = kUnknown;
  NumaNode() = default;
  explicit NumaNode(uint32_t v) : id(v) {}
  static NumaNode from_int(int v) { return v < 0 ? NumaNode() : NumaNode(static_cast<uint32_t>(v)); }
  bool is_unknown() const { return id == kUnknown; }
  bool is_valid() const { return id != kUnknown; }
  int as_int() const { return is_unknown() ? -1 : static_cast<int>(id); }
  std::string to_string() const;  // "NUMA3" / "UNKNOWN"
  bool operator==(const NumaNode& o) const { return id == o.id; }
  bool operator<(const NumaNode& o) const { return id < o.id; }
};

// numa.rs:49-78: [0,1,2,4] -> "0-2,4".
std::string format_cpu_list(const std::vector<size_t>& cpus);

// numa.rs:132-172: "0-3,8" -> [0,1,2,3,8], sorted and de-duplicated.
// Returns false and sets *err on malformed input.
bool parse_cpulist(const std::string& cpulist, std::vector<size_t>* out, std::string* err);

// numa.rs:88-129: node id -> cpus from /sys/devices/system/node (or `root`
// when given, for tests).
bool read_cpu_topology_from_sysfs(std::map<uint32_t, std::vector<size_t>>* out, std::string* err,
                                  const char* root = nullptr);

// numa.rs:178-217.
bool pin_thread_to_numa_node(NumaNode node, std::string* err);

// numa.rs:224-257: run `f` on a fresh thread pinned to `node`.
bool run_on_numa(NumaNode node, const std::function<void()>& f, std::string* err);

// NUMA node of a PCI device ("0000:c1:00.0") from sysfs; -1 when unknown.
int numa_node_of_pci_device(const char* bdf, const char* sysfs_root = nullptr);

// numa.rs:448-497: node of the page holding each address (move_pages query).
std::vector<NumaNode> query_pages_numa(const std::vector<const void*>& addrs);

// numa.rs:340-430.
class NumaTopology {
 public:
  static NumaTopology detect();
  NumaTopology() = default;
  NumaTopology(std::map<int, NumaNode> gpu_map, std::vector<NumaNode> nodes)
      : gpu_numa_map_(std::move(gpu_map)), numa_nodes_(std::move(nodes)) {}
  NumaNode numa_for_gpu(int device_id) const;
  const std::vector<NumaNode>& numa_nodes() const { return numa_nodes_; }
  std::vector<NumaNode> gpu_numa_nodes() const;
  size_t num_nodes() const { return numa_nodes_.size(); }
  bool is_multi_numa() const { return numa_nodes_.size() > 1; }

 private:
  std::map<int, NumaNode> gpu_numa_map_;
  std::vector<NumaNode> numa_nodes_;
};

}  // namespace pf
