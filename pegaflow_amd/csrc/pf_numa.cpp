#include "pf_numa.hpp"

#include <dirent.h>
#include <sched.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>
#include <fstream>
#include <sstream>
#include <thread>

#include "pf_common.hpp"

namespace pf {

std::string NumaNode::to_string() const {
  if (is_unknown()) return "UNKNOWN";
  return "NUMA" + std::to_string(id);
}

std::string format_cpu_list(const std::vector<size_t>& cpus) {
  std::string out;
  size_t i = 0;
  while (i < cpus.size()) {
    size_t j = i;
    while (j + 1 < cpus.size() && cpus[j + 1] == cpus[j] + 1) ++j;
    if (!out.empty()) out += ",";
    out += std::to_string(cpus[i]);
    if (j > i) out += "-" + std::to_string(cpus[j]);
    i = j + 1;
  }
  return out;
}

static bool parse_cpu_id(const std::string& s, size_t* out) {
  if (s.empty()) return false;
  size_t v = 0;
  for (char c : s) {
    if (c < '0' || c > '9') return false;
    v = v * 10 + static_cast<size_t>(c - '0');
  }
  *out = v;
  return true;
}

bool parse_cpulist(const std::string& cpulist, std::vector<size_t>* out, std::string* err) {
  out->clear();
  if (cpulist.empty()) return true;
  std::stringstream ss(cpulist);
  std::string part;
  while (std::getline(ss, part, ',')) {
    size_t dash = part.find('-');
    if (dash != std::string::npos) {
      std::string lo = part.substr(0, dash), hi = part.substr(dash + 1);
      if (hi.find('-') != std::string::npos) {
        if (err) *err = "Invalid CPU range format: " + part;
        return false;
      }
      size_t a = 0, b = 0;
      if (!parse_cpu_id(lo, &a)) {
        if (err) *err = "Invalid CPU ID: " + lo;
        return false;
      }
      if (!parse_cpu_id(hi, &b)) {
        if (err) *err = "Invalid CPU ID: " + hi;
        return false;
      }
      for (size_t c = a; c <= b; ++c) out->push_back(c);
    } else {
      size_t a = 0;
      if (!parse_cpu_id(part, &a)) {
        if (err) *err = "Invalid CPU ID: " + part;
        return false;
      }
      out->push_back(a);
    }
  }
  std::sort(out->begin(), out->end());
  out->erase(std::unique(out->begin(), out->end()), out->end());
  return true;
}

static std::string trim(const std::string& s) {
  size_t a = s.find_first_not_of(" \t\r\n");
  if (a == std::string::npos) return "";
  size_t b = s.find_last_not_of(" \t\r\n");
  return s.substr(a, b - a + 1);
}

bool read_cpu_topology_from_sysfs(std::map<uint32_t, std::vector<size_t>>* out, std::string* err,
                                  const char* root) {
  out->clear();
  std::string dir = root ? root : "/sys/devices/system/node";
  DIR* d = opendir(dir.c_str());
  if (!d) {
    if (err) *err = "NUMA not supported: " + dir + " not found";
    return false;
  }
  bool ok = true;
  while (struct dirent* ent = readdir(d)) {
    std::string name = ent->d_name;
    if (name.rfind("node", 0) != 0) continue;
    size_t id = 0;
    if (!parse_cpu_id(name.substr(4), &id)) {
      if (err) *err = "Invalid node directory name: " + name;
      ok = false;
      break;
    }
    std::ifstream f(dir + "/" + name + "/cpulist");
    if (!f) continue;
    std::string line;
    std::getline(f, line);
    std::vector<size_t> cpus;
    if (!parse_cpulist(trim(line), &cpus, err)) {
      ok = false;
      break;
    }
    (*out)[static_cast<uint32_t>(id)] = std::move(cpus);
  }
  closedir(d);
  if (!ok) return false;
  if (out->empty()) {
    if (err) *err = "No NUMA nodes found";
    return false;
  }
  return true;
}

bool pin_thread_to_numa_node(NumaNode node, std::string* err) {
  if (node.is_unknown()) {
    if (err) *err = "Cannot pin to unknown NUMA node";
    return false;
  }
  std::map<uint32_t, std::vector<size_t>> topo;
  std::string e;
  if (!read_cpu_topology_from_sysfs(&topo, &e)) {
    if (err) *err = "Failed to get NUMA topology: " + e;
    return false;
  }
  auto it = topo.find(node.id);
  if (it == topo.end()) {
    if (err) *err = "No CPUs found for NUMA node " + std::to_string(node.id);
    return false;
  }
  if (it->second.empty()) {
    if (err) *err = "CPU list is empty for NUMA node " + std::to_string(node.id);
    return false;
  }
  cpu_set_t set;
  CPU_ZERO(&set);
  for (size_t c : it->second) {
    if (c < CPU_SETSIZE) CPU_SET(c, &set);
  }
  if (sched_setaffinity(0, sizeof(set), &set) != 0) {
    if (err) *err = std::string("sched_setaffinity failed: ") + strerror(errno);
    return false;
  }
  return true;
}

bool run_on_numa(NumaNode node, const std::function<void()>& f, std::string* err) {
  if (node.is_unknown()) {
    if (err) *err = "Cannot run on unknown NUMA node";
    return false;
  }
  bool ok = false;
  std::string thread_err;
  std::thread t([&] {
    if (!pin_thread_to_numa_node(node, &thread_err)) return;
    f();
    ok = true;
  });
  t.join();
  if (!ok && err) *err = thread_err;
  return ok;
}

int numa_node_of_pci_device(const char* bdf, const char* sysfs_root) {
  if (!bdf || !*bdf) return -1;
  std::string id = bdf;
  for (char& c : id) {
    if (c >= 'A' && c <= 'F') c = static_cast<char>(c - 'A' + 'a');
  }
  std::string root = sysfs_root ? sysfs_root : "/sys/bus/pci/devices";
  std::ifstream f(root + "/" + id + "/numa_node");
  if (!f) return -1;
  int node = -1;
  f >> node;
  if (!f) return -1;
  return node < 0 ? -1 : node;
}

std::vector<NumaNode> query_pages_numa(const std::vector<const void*>& addrs) {
  std::vector<NumaNode> out;
  if (addrs.empty()) return out;
  long page = sysconf(_SC_PAGESIZE);
  if (page <= 0) page = 4096;
  std::vector<void*> pages(addrs.size());
  for (size_t i = 0; i < addrs.size(); ++i) {
    pages[i] = reinterpret_cast<void*>(reinterpret_cast<uintptr_t>(addrs[i]) &
                                       ~static_cast<uintptr_t>(page - 1));
  }
  std::vector<int> status(addrs.size(), 0);
  long ret = syscall(SYS_move_pages, 0, addrs.size(), pages.data(), nullptr, status.data(), 0);
  out.resize(addrs.size());
  if (ret != 0) return out;  // all UNKNOWN
  for (size_t i = 0; i < addrs.size(); ++i) {
    if (status[i] >= 0) out[i] = NumaNode(static_cast<uint32_t>(status[i]));
  }
  return out;
}

NumaTopology NumaTopology::detect() {
  std::map<int, NumaNode> gpu_map;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess) {
    (void)hipGetLastError();
    count = 0;
  }
  for (int d = 0; d < count; ++d) {
    char bdf[64] = {0};
    if (hipDeviceGetPCIBusId(bdf, sizeof(bdf), d) != hipSuccess) {
      (void)hipGetLastError();
      gpu_map[d] = NumaNode();
      continue;
    }
    gpu_map[d] = NumaNode::from_int(numa_node_of_pci_device(bdf));
  }
  std::vector<NumaNode> nodes;
  std::map<uint32_t, std::vector<size_t>> topo;
  std::string err;
  if (read_cpu_topology_from_sysfs(&topo, &err)) {
    for (auto& kv : topo) nodes.push_back(NumaNode(kv.first));
  } else {
    nodes.push_back(NumaNode(0));
  }
  return NumaTopology(std::move(gpu_map), std::move(nodes));
}

NumaNode NumaTopology::numa_for_gpu(int device_id) const {
  auto it = gpu_numa_map_.find(device_id);
  return it == gpu_numa_map_.end() ? NumaNode() : it->second;
}

std::vector<NumaNode> NumaTopology::gpu_numa_nodes() const {
  std::vector<NumaNode> nodes;
  for (auto& kv : gpu_numa_map_) {
    if (kv.second.is_valid()) nodes.push_back(kv.second);
  }
  std::sort(nodes.begin(), nodes.end());
  nodes.erase(std::unique(nodes.begin(), nodes.end()), nodes.end());
  return nodes;
}

}  // namespace pf
