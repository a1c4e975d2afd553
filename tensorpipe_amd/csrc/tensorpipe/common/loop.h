// Serial executors. Every object in this library mutates its state only from
// inside one loop, so no per-object locks are needed.
//
//  OnDemandLoop : no thread of its own. defer() enqueues; if nobody is
//                 draining the queue the caller drains it (and anything that
//                 gets enqueued meanwhile) before returning. Keeps the send /
//                 recv fast path on the calling thread, without a hop.
//  ThreadLoop   : same queue, drained by a dedicated thread that sleeps on a
//                 condition variable.
#pragma once

#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

using TTask = std::function<void()>;

class OnDemandLoop {
 public:
  void defer(TTask fn) {
    {
      std::unique_lock<std::mutex> lock(mutex_);
      queue_.push_back(std::move(fn));
      if (draining_) {
        return;
      }
      draining_ = true;
    }
    owner_.store(std::this_thread::get_id(), std::memory_order_relaxed);
    for (;;) {
      TTask task;
      {
        std::unique_lock<std::mutex> lock(mutex_);
        if (queue_.empty()) {
          owner_.store(std::thread::id(), std::memory_order_relaxed);
          draining_ = false;
          return;
        }
        task = std::move(queue_.front());
        queue_.pop_front();
      }
      task();
    }
  }

  bool inLoop() const {
    return owner_.load(std::memory_order_relaxed) == std::this_thread::get_id();
  }

 private:
  std::mutex mutex_;
  std::deque<TTask> queue_;
  bool draining_{false};
  std::atomic<std::thread::id> owner_{std::thread::id()};
};

class ThreadLoop {
 public:
  explicit ThreadLoop(std::string name = "tp_loop") : name_(std::move(name)) {
    thread_ = std::thread([this] { run(); });
  }

  ~ThreadLoop() {
    join();
  }

  void defer(TTask fn) {
    {
      std::unique_lock<std::mutex> lock(mutex_);
      queue_.push_back(std::move(fn));
    }
    cv_.notify_one();
  }

  bool inLoop() const {
    return std::this_thread::get_id() == thread_.get_id();
  }

  // Runs what is queued, then stops the thread. Idempotent.
  void join() {
    {
      std::unique_lock<std::mutex> lock(mutex_);
      if (stopping_) {
        return;
      }
      stopping_ = true;
    }
    cv_.notify_one();
    if (thread_.joinable()) {
      thread_.join();
    }
  }

 private:
  void run() {
    std::unique_lock<std::mutex> lock(mutex_);
    for (;;) {
      cv_.wait(lock, [this] { return stopping_ || !queue_.empty(); });
      while (!queue_.empty()) {
        TTask task = std::move(queue_.front());
        queue_.pop_front();
        lock.unlock();
        task();
        lock.lock();
      }
      if (stopping_) {
        return;
      }
    }
  }

  const std::string name_;
  std::mutex mutex_;
  std::condition_variable cv_;
  std::deque<TTask> queue_;
  bool stopping_{false};
  std::thread thread_;
};

TP_AMD_NAMESPACE_END
