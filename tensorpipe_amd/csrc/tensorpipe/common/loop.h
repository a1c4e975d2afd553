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
// the library created (transport reactor, event poller, ThreadLoop, helper)
// runs whatever is queued, also what other threads add meanwhile. A thread of
// the application that entered through send/recv/write/read runs only what it
// queued itself: a completion that another thread queues at that moment would
// otherwise run the application's callback on the application's own stack,
// inside the very call that started the operation -- and a caller that holds a
// lock its callback also takes would deadlock (the reference checks for
// exactly that: tensorpipe/test/channel/channel_test_cpu.cc:44-109).
//
// Who then runs such a task:
//  * a library thread that is not inside a task of any loop waits a few
//    microseconds (bounded) for the application's thread to leave and drains
//    the queue itself: the common case, a reactor or poller thread delivering
//    a completion while the application is still inside its call;
//  * every other thread returns from defer() at once, as the reference's
//    executor always does (tensorpipe/common/deferred_executor.h:101-124): a
//    thread inside a task of another loop may be exactly what the draining
//    thread's task is waiting for (two threads, each in a task of one loop and
//    deferring to the other's, would wait for each other for good), and an
//    application thread may hold a lock the draining task wants. The draining
//    thread, when it leaves with other threads' tasks still queued and nobody
//    waiting to take over, hands the loop to a helper thread of the library.
#pragma once

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>

#include <pthread.h>
#include <sched.h>
#include <unistd.h>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

using TTask = std::function<void()>;

// Set once by every thread the library starts.
inline bool& thisIsLibraryThread() {
  static thread_local bool flag = false;
  return flag;
}

// How many tasks of this library's loops (any of them) are on the calling
// thread's stack.
inline int& loopTaskDepth() {
  static thread_local int depth = 0;
  return depth;
}

struct LoopTaskScope {
  LoopTaskScope() {
    ++loopTaskDepth();
  }
  ~LoopTaskScope() {
    --loopTaskDepth();
  }
};

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

// Library threads that drain on-demand loops whose application-thread drainer
// left other threads' tasks behind. Started on first need; one more is started
// whenever work comes in and none is idle (a user's callback may block the one
// that runs it), up to a small limit; an idle one leaves after a second. Never
// destroyed: threads of it may still run when static destructors do.
class LoopHelpers {
 public:
  static LoopHelpers& get() {
    static LoopHelpers* const instance = [] {
      auto* h = new LoopHelpers();
      // A forked child has none of the parent's threads.
      ::pthread_atfork(nullptr, nullptr, [] { new (&LoopHelpers::get()) LoopHelpers(); });
      return h;
    }();
    return *instance;
  }

  void post(TTask work) {
    bool spawn = false;
    {
      std::unique_lock<std::mutex> lock(mutex_);
      queue_.push_back(std::move(work));
      if (idle_ == 0 && threads_ < kMaxThreads) {
        ++threads_;
        spawn = true;
      }
    }
    if (spawn) {
      std::thread([this] { run(); }).detach();
    } else {
      cv_.notify_one();
    }
  }

 private:
  static constexpr unsigned kMaxThreads = 8;

  void run() {
    thisIsLibraryThread() = true;
    ::pthread_setname_np(::pthread_self(), "tp_loop_helper");
    std::unique_lock<std::mutex> lock(mutex_);
    for (;;) {
      while (!queue_.empty()) {
        TTask work = std::move(queue_.front());
        queue_.pop_front();
        lock.unlock();
        work();
        work = nullptr;
        lock.lock();
      }
      ++idle_;
      // (wall-clock deadline: the sanitizers of this toolchain follow
      // pthread_cond_timedwait, not the monotonic variant wait_for() uses)
      const bool more = cv_.wait_until(
          lock, std::chrono::system_clock::now() + std::chrono::seconds(1), [this] { return !queue_.empty(); });
      --idle_;
      if (!more) {
        --threads_;
        return;
      }
    }
  }

  std::mutex mutex_;
  std::condition_variable cv_;
  std::deque<TTask> queue_;
  unsigned threads_{0};
  unsigned idle_{0};
};

class OnDemandLoop {
 public:
  OnDemandLoop() : state_(std::make_shared<State>()) {}
  OnDemandLoop(const OnDemandLoop&) = delete;
  OnDemandLoop& operator=(const OnDemandLoop&) = delete;

  // Nothing to wait for: the queue and its bookkeeping live in an object of
  // their own that a draining thread (the caller of defer(), a helper) keeps
  // alive for as long as it drains. The last reference to a loop's owner is
  // often dropped by a task of that very loop (a callback that held the last
  // pointer to a listener that held the last pointer to its context), so the
  // loop may be destroyed from inside one of its own tasks; what is still
  // queued then runs all the same.
  ~OnDemandLoop() = default;

  void defer(TTask fn) {
    State& s = *state_;
    const std::thread::id me = std::this_thread::get_id();
    std::shared_ptr<State> keep;
    {
      std::unique_lock<std::mutex> lock(s.mutex_);
      s.queue_.push_back(Item{std::move(fn), me});
      if (s.draining_) {
        if (s.drainer_ == me || !s.guestDrainer_) {
          return; // the draining thread will get to it
        }
        // An application thread is draining: it leaves our task alone.
        if (!thisIsLibraryThread() || loopTaskDepth() > 0) {
          return; // may not wait (see the top of this file); a helper will run it
        }
        ++s.waiters_;
        keep = state_;
      } else {
        s.takeOver(me);
        keep = state_;
        lock.unlock();
        s.drain(keep, me);
        return;
      }
    }
    // A library thread with no task of any loop on its stack: wait, briefly,
    // for the application's thread to leave.
    const auto giveUpAt = std::chrono::steady_clock::now() + std::chrono::microseconds(kMaxWaitUs);
    for (unsigned spins = 0;; ++spins) {
      {
        std::unique_lock<std::mutex> lock(s.mutex_);
        if (!s.draining_) {
          --s.waiters_;
          s.takeOver(me);
          break;
        }
        if (!s.guestDrainer_) {
          --s.waiters_;
          return; // a library thread took over and will run it
        }
        if ((spins & 63) == 63 && std::chrono::steady_clock::now() > giveUpAt) {
          --s.waiters_;
          return; // the drainer finds nobody waiting when it leaves and calls a helper
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
    s.drain(keep, me);
  }

  bool inLoop() const {
    return state_->owner_.load(std::memory_order_relaxed) == std::this_thread::get_id();
  }

 private:
  static constexpr int kMaxWaitUs = 100;

  struct Item {
    TTask fn;
    std::thread::id from;
  };

  struct State {
    // mutex_ held.
    void takeOver(std::thread::id me) {
      draining_ = true;
      drainer_ = me;
      guestDrainer_ = !thisIsLibraryThread();
    }

    // `self` is what keeps this object alive while a task destroys the loop.
    void drain(const std::shared_ptr<State>& self, std::thread::id me) {
      owner_.store(me, std::memory_order_relaxed);
      for (;;) {
        TTask task;
        {
          std::unique_lock<std::mutex> lock(mutex_);
          if (queue_.empty()) {
            owner_.store(std::thread::id(), std::memory_order_relaxed);
            draining_ = false;
            return;
          }
          if (guestDrainer_ && queue_.front().from != me) {
            // Not this application thread's task. Whoever waits takes over; with
            // nobody waiting a helper is called.
            owner_.store(std::thread::id(), std::memory_order_relaxed);
            draining_ = false;
            if (waiters_ == 0 && !helperCalled_) {
              helperCalled_ = true;
              lock.unlock();
              LoopHelpers::get().post([self] { self->drainAsHelper(self); });
            }
            return;
          }
          task = std::move(queue_.front().fn);
          queue_.pop_front();
        }
        LoopTaskScope scope;
        task();
      }
    }

    void drainAsHelper(const std::shared_ptr<State>& self) {
      const std::thread::id me = std::this_thread::get_id();
      {
        std::unique_lock<std::mutex> lock(mutex_);
        helperCalled_ = false;
        // Somebody drains already: a library thread runs everything, an
        // application thread calls again when it leaves.
        if (draining_ || queue_.empty()) {
          return;
        }
        takeOver(me);
      }
      drain(self, me);
    }

    std::mutex mutex_;
    std::deque<Item> queue_;
    bool draining_{false};
    bool guestDrainer_{false}; // the draining thread belongs to the application
    bool helperCalled_{false}; // a helper is on its way and has not looked yet
    std::thread::id drainer_;
    unsigned waiters_{0}; // library threads waiting for a guest drainer to leave
    std::atomic<std::thread::id> owner_{std::thread::id()};
  };

  const std::shared_ptr<State> state_;
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
        {
          LoopTaskScope scope;
          task();
        }
        task = nullptr;
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
