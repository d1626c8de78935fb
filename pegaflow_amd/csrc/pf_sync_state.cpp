#include "pf_sync_state.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <cstring>
#include <random>

namespace pf {

namespace {

struct Record {
  std::atomic<uint32_t> magic;
  std::atomic<uint32_t> version;
  std::atomic<int64_t> state;
};
static_assert(sizeof(Record) == 16, "LoadState record is 16 bytes");

constexpr size_t kMetaSize = 8;
constexpr size_t kAllocationSize = kMetaSize + sizeof(Record) + alignof(Record);  // 32

std::string shm_path(const std::string& name) { return name.empty() || name[0] == '/' ? name : "/" + name; }

}  // namespace

std::unique_ptr<LoadState> LoadState::create(std::string* err) {
  std::random_device rd;
  char hex[33];
  for (int i = 0; i < 4; ++i) snprintf(hex + 8 * i, 9, "%08x", static_cast<unsigned>(rd()));
  std::unique_ptr<LoadState> s(new LoadState());
  s->name_ = std::string("pega_load_") + hex;
  int fd = shm_open(shm_path(s->name_).c_str(), O_CREAT | O_EXCL | O_RDWR, S_IRUSR | S_IWUSR);
  if (fd < 0) {
    if (err) *err = std::string("failed to create shared memory: ") + strerror(errno);
    return nullptr;
  }
  s->owner_ = true;
  if (ftruncate(fd, static_cast<off_t>(kAllocationSize)) != 0) {
    if (err) *err = std::string("failed to create shared memory: ") + strerror(errno);
    close(fd);
    shm_unlink(shm_path(s->name_).c_str());
    s->owner_ = false;
    return nullptr;
  }
  void* base = mmap(nullptr, kAllocationSize, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (base == MAP_FAILED) {
    if (err) *err = std::string("failed to create shared memory: ") + strerror(errno);
    shm_unlink(shm_path(s->name_).c_str());
    s->owner_ = false;
    return nullptr;
  }
  s->base_ = base;
  s->len_ = kAllocationSize;
  uintptr_t b = reinterpret_cast<uintptr_t>(base);
  uintptr_t aligned = (b + kMetaSize + alignof(Record) - 1) & ~(static_cast<uintptr_t>(alignof(Record)) - 1);
  uint64_t offset = aligned - b;
  std::memcpy(base, &offset, sizeof(offset));
  auto* rec = reinterpret_cast<Record*>(aligned);
  rec->magic.store(kLoadStateMagic, std::memory_order_release);
  rec->version.store(kLoadStateVersion, std::memory_order_release);
  rec->state.store(kLoadStatePending, std::memory_order_release);
  s->record_ = rec;
  return s;
}

std::unique_ptr<LoadState> LoadState::attach(const std::string& shm_name, std::string* err) {
  int fd = shm_open(shm_path(shm_name).c_str(), O_RDWR, 0);
  if (fd < 0) {
    if (err) *err = std::string("failed to open shared memory: ") + strerror(errno);
    return nullptr;
  }
  struct stat st;
  if (fstat(fd, &st) != 0) {
    if (err) *err = std::string("failed to open shared memory: ") + strerror(errno);
    close(fd);
    return nullptr;
  }
  size_t len = static_cast<size_t>(st.st_size);
  if (len < kMetaSize + sizeof(Record)) {
    if (err) {
      *err = "shared memory too small (actual=" + std::to_string(len) +
             " bytes, required=" + std::to_string(kAllocationSize) + " bytes)";
    }
    close(fd);
    return nullptr;
  }
  void* base = mmap(nullptr, len, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (base == MAP_FAILED) {
    if (err) *err = std::string("failed to open shared memory: ") + strerror(errno);
    return nullptr;
  }
  std::unique_ptr<LoadState> s(new LoadState());
  s->name_ = shm_name;
  s->base_ = base;
  s->len_ = len;
  uint64_t offset = 0;
  std::memcpy(&offset, base, sizeof(offset));
  if (offset > len || len - offset < sizeof(Record) || (offset % alignof(Record)) != 0) {
    if (err) {
      *err = "invalid LoadState offset (offset=" + std::to_string(offset) +
             ", len=" + std::to_string(len) + ") recorded in shared memory";
    }
    return nullptr;
  }
  auto* rec = reinterpret_cast<Record*>(static_cast<uint8_t*>(base) + offset);
  uint32_t magic = rec->magic.load(std::memory_order_acquire);
  uint32_t version = rec->version.load(std::memory_order_acquire);
  if (magic != kLoadStateMagic || version != kLoadStateVersion) {
    if (err) {
      char buf[160];
      snprintf(buf, sizeof buf,
               "invalid LoadState header (magic=%#x, version=%u, expected magic=%#x, version=%u)",
               magic, version, kLoadStateMagic, kLoadStateVersion);
      *err = buf;
    }
    return nullptr;
  }
  s->record_ = rec;
  return s;
}

LoadState::~LoadState() {
  if (base_) munmap(base_, len_);
  if (owner_) shm_unlink(shm_path(name_).c_str());
}

int64_t LoadState::get() const {
  return static_cast<Record*>(record_)->state.load(std::memory_order_acquire);
}

void LoadState::set_completed() {
  static_cast<Record*>(record_)->state.store(kLoadStateSuccess, std::memory_order_release);
}

void LoadState::set_error() {
  static_cast<Record*>(record_)->state.store(kLoadStateError, std::memory_order_release);
}

}  // namespace pf
