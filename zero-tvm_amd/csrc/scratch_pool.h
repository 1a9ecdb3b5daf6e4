// Lifetime of the context's scratch buffer.
//
// Kernels of the rows, skinny and tile-GEMM families take the scratch address as an argument, and a
// recorded command buffer keeps that address in its kernel nodes for as long as it lives. So a
// buffer that any live command buffer may reference is never freed when a later dispatch needs a
// larger one: it is retired and freed only when the last command buffer that could hold its address
// is gone (or with the context). Growth at least doubles, so the retired buffers together stay
// smaller than the current one.
//
// The allocator is a template parameter so that the bookkeeping can be exercised on the CPU.
#pragma once
#include <stddef.h>
#include <vector>

namespace ztvm {

template <class Alloc>
class ScratchPool {
 public:
  explicit ScratchPool(Alloc a = Alloc()) : alloc_(a) {}
  ScratchPool(const ScratchPool&) = delete;
  ScratchPool& operator=(const ScratchPool&) = delete;

  void* data() const { return cur_; }
  size_t bytes() const { return bytes_; }
  size_t retired() const { return retired_.size(); }
  int pinned() const { return pins_; }

  // Make at least `need` bytes available; returns false if the allocation fails (the old buffer is
  // kept then). Never invalidates an address handed out while a command buffer was alive.
  bool reserve(size_t need) {
    if (need <= bytes_) return true;
    size_t want = bytes_ * 2 > need ? bytes_ * 2 : need;
    void* p = alloc_.allocate(want);
    if (!p && want != need) { want = need; p = alloc_.allocate(want); }
    if (!p) return false;
    if (cur_) {
      if (pins_ > 0) retired_.push_back(cur_);
      else alloc_.release(cur_);
    }
    cur_ = p;
    bytes_ = want;
    return true;
  }

  // A command buffer that may hold the current (or a retired) address came to life / died.
  void pin() { ++pins_; }
  void unpin() {
    if (pins_ > 0 && --pins_ == 0) {
      for (void* p : retired_) alloc_.release(p);
      retired_.clear();
    }
  }

  void release_all() {
    for (void* p : retired_) alloc_.release(p);
    retired_.clear();
    if (cur_) alloc_.release(cur_);
    cur_ = nullptr;
    bytes_ = 0;
  }

 private:
  Alloc alloc_;
  void* cur_ = nullptr;
  size_t bytes_ = 0;
  std::vector<void*> retired_;
  int pins_ = 0;
};

}  // namespace ztvm
