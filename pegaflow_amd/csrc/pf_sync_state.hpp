// Shared-memory completion flag of an asynchronous load, polled by the
// process that asked for it.  Wire format follows
// pegaflow-core/src/sync_state.rs:23-300 of the reference: a POSIX shm object
// whose first 8 bytes hold the offset of an 8-aligned record
// { u32 magic 'PFLD', u32 version 1, i64 state } with state 0 = pending,
// 1 = success, -1 = error.
#pragma once

#include <cstdint>
#include <memory>
#include <string>

namespace pf {

constexpr int64_t kLoadStatePending = 0;
constexpr int64_t kLoadStateSuccess = 1;
constexpr int64_t kLoadStateError = -1;
constexpr uint32_t kLoadStateMagic = 0x50464c44;  // 'PFLD'
constexpr uint32_t kLoadStateVersion = 1;

class LoadState {
 public:
  // Creates "pega_load_<32 hex digits>" and initialises it to pending.
  static std::unique_ptr<LoadState> create(std::string* err);
  // Opens an existing object and validates its header.
  static std::unique_ptr<LoadState> attach(const std::string& shm_name, std::string* err);
  ~LoadState();
  const std::string& shm_name() const { return name_; }
  int64_t get() const;
  void set_completed();
  void set_error();

 private:
  LoadState() = default;
  std::string name_;
  void* base_ = nullptr;
  size_t len_ = 0;
  void* record_ = nullptr;
  bool owner_ = false;
};

}  // namespace pf
