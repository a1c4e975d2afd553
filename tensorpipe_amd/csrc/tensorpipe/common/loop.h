// Serial executors. Every object in this library mutates its state only from
// inside one loop, so no per-object locks are needed.
//
//  OnDemandLoop : no thread of its own. defer() enqueues; if nobody is
//                 draining the queue the caller drains it before returning.
//                 Keeps the send / recv fast path on the calling thread,
//                 without a hop.
//  ThreadLoop   : same queue, drained by a dedicated thread that sleeps on a
//                 condition variable.
//
// Whose tasks a draining thread runs depends on whose thread it is. A thread
// the library created (transport reactor, event poller, ThreadLoop) runs
// whatever is queued, also what other threads add meanwhile. A thread of the
// application that entered through send/recv/write/read runs only what it
// queued itself: a completion that a library thread queues at that moment
// would otherwise run the application's callback on the application's own
// stack, inside the very call that started the operation -- and a caller that
// holds a lock its callback also takes would deadlock (the reference checks
// for exactly that: tensorpipe/test/channel/channel_test_cpu.cc:44-109). The
// library thread instead waits the few microseconds until the application's
// thread has left the loop and drains the queue itself.
#pragma once

#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>

#include <sched.h>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

using TTask = std::function<void()>;

// Set once by every thread the library starts.
inline bool& thisIsLibraryThread() {
  static thread_local bool flag = false;
  return flag;
}

// Whether this process has fewer CPUs to run on (affinity mask, pinned
// containers) than a pipe keeps busy at full tilt: the caller, the context's
// loop and the two threads that stay hot after an event (transport reactor,
// event poller). With fewer, a thread that spins keeps the thread it waits for
// off the CPU, so those loops go to sleep at once instead. The threshold can be
// moved with TP_SPIN_MIN_CPUS.
inline bool runsOnFewCpus() {
  static const bool few = [] {
    int need = 4;
    if (const char* e = std::getenv("TP_SPIN_MIN_CPUS")) {
      need = std::atoi(e);
    }
    cpu_set_t set;
    CPU_ZERO(&set);
    return ::sched_getaffinity(0, sizeof(set), &set) == 0 && CPU_COUNT(&set) < need;
  }();
  return few;
}

class OnDemandLoop {
 public:
  void defer(TTask fn) {
    const std::thread::id me = std::this_thread::get_id();
    bool wait = false;
    {
      std::unique_lock<std::mutex> lock(mutex_);
      queue_.push_back(Item{std::move(fn), me});
      if (draining_) {
        if (drainer_ == me || !guestDrainer_) {
          return; // the draining thread will get to it
        }
        // An application thread is draining: it leaves our task alone.
        ++waiters_;
        wait = true;
      } else {
        draining_ = true;
        drainer_ = me;
        guestDrainer_ = !thisIsLibraryThread();
      }
    }
    if (wait) {
      for (unsigned spins = 0;; ++spins) {
        {
          std::unique_lock<std::mutex> lock(mutex_);
          if (!draining_) {
            --waiters_;
            draining_ = true;
            drainer_ = me;
            guestDrainer_ = !thisIsLibraryThread();
            break;
          }
          if (!guestDrainer_) {
            --waiters_;
            return; // a library thread took over and will run it
          }
        }
        if (spins < 2000) {
#if defined(__x86_64__)
          __builtin_ia32_pause();
#endif
        } else {
          std::this_thread::yield();
        }
      }
    }
    owner_.store(me, std::memory_order_relaxed);
    for (;;) {
      TTask task;
      {
        std::unique_lock<std::mutex> lock(mutex_);
        // A guest stops at the first task that is not its own when that task's
        // owner is waiting to take over; with nobody waiting it carries on, so
        // that no task is left behind.
        if (queue_.empty() || (guestDrainer_ && queue_.front().from != me && waiters_ > 0)) {
          owner_.store(std::thread::id(), std::memory_order_relaxed);
          draining_ = false;
          return;
        }
        task = std::move(queue_.front().fn);
        queue_.pop_front();
      }
      task();
    }
  }

  bool inLoop() const {
    return owner_.load(std::memory_order_relaxed) == std::this_thread::get_id();
  }

 private:
  struct Item {
    TTask fn;
    std::thread::id from;
  };
  std::mutex mutex_;
  std::deque<Item> queue_;
  bool draining_{false};
  bool guestDrainer_{false}; // the draining thread belongs to the application
  std::thread::id drainer_;
  unsigned waiters_{0}; // threads waiting for a guest drainer to leave
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
    thisIsLibraryThread() = true;
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
