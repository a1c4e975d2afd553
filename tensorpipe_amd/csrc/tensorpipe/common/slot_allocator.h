// Asynchronous fixed-slot allocator over one slab. alloc() queues a request;
// requests are served first come first served, each with the lowest free slot;
// a granted slot is returned by dropping the shared_ptr; close() fails every
// waiting and future request. Not thread-safe: use from one loop.
// Same observable behaviour as tensorpipe/common/allocator.cc:26-79.
#pragma once

#include <cstdint>
#include <deque>
#include <functional>
#include <memory>
#include <vector>

#include <tensorpipe/common/error.h>

TP_AMD_NAMESPACE_BEGIN

class AllocatorClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "allocator closed";
  }
};

class SlotAllocator {
 public:
  using TSlot = std::shared_ptr<uint8_t>;
  using TCallback = std::function<void(const Error&, TSlot)>;

  SlotAllocator(uint8_t* slab, size_t numSlots, size_t slotSize)
      : state_(std::make_shared<State>()) {
    state_->slab = slab;
    state_->slotSize = slotSize;
    state_->free.assign(numSlots, true);
  }

  ~SlotAllocator() {
    close();
  }

  void alloc(TCallback callback) {
    state_->waiters.push_back(std::move(callback));
    serve(state_);
  }

  size_t slotSize() const {
    return state_->slotSize;
  }

  size_t slotIndex(const uint8_t* ptr) const {
    return static_cast<size_t>(ptr - state_->slab) / state_->slotSize;
  }

  void close() {
    if (state_->closed) {
      return;
    }
    state_->closed = true;
    serve(state_);
  }

 private:
  struct State {
    uint8_t* slab{nullptr};
    size_t slotSize{0};
    std::vector<bool> free;
    std::deque<TCallback> waiters;
    bool closed{false};
    bool serving{false};
  };

  static void serve(const std::shared_ptr<State>& st) {
    if (st->serving) {
      return; // a callback released a slot: the outer call keeps going
    }
    st->serving = true;
    while (!st->waiters.empty()) {
      TSlot slot;
      if (!st->closed) {
        for (size_t i = 0; i < st->free.size(); ++i) {
          if (st->free[i]) {
            st->free[i] = false;
            std::weak_ptr<State> weak = st;
            slot = TSlot(st->slab + i * st->slotSize, [weak, i](uint8_t*) {
              if (auto s = weak.lock()) {
                s->free[i] = true;
                serve(s);
              }
            });
            break;
          }
        }
        if (!slot) {
          break;
        }
      }
      TCallback cb = std::move(st->waiters.front());
      st->waiters.pop_front();
      if (slot) {
        cb(Error::kSuccess, std::move(slot));
      } else {
        cb(TP_CREATE_ERROR(AllocatorClosedError), nullptr);
      }
    }
    st->serving = false;
  }

  std::shared_ptr<State> state_;
};

TP_AMD_NAMESPACE_END
