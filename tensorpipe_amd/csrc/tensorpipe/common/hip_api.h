// C++ convenience over the HIP C ABI (include/tphip.h): error checking that
// throws, RAII for events, streams, device and pinned slabs. The only way host
// code in this library touches the GPU.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include <tphip.h>

#include <tensorpipe/common/defs.h>
#include <tensorpipe/common/error.h>

#define TP_HIP_CHECK(call)                                                          \
  do {                                                                              \
    int tp_rc_ = (call);                                                            \
    if (tp_rc_ != 0) {                                                              \
      TP_THROW_MSG(#call << " failed: [" << tp_rc_ << "] " << tphip_strerror(tp_rc_)); \
    }                                                                               \
  } while (0)

TP_AMD_NAMESPACE_BEGIN

// Number of usable GPUs; 0 when the runtime reports none or fails to load.
int hipDeviceCountNoThrow();

// Device index owning ptr (tensorpipe/common/cuda.h:141-166): device memory and
// pinned host memory yield their device, memory the runtime does not know
// (plain host memory, null) yields -1, which callers turn into an exception as
// the reference's driver check does. Answers are remembered per allocation, so
// the runtime is asked once per allocation and not once per tensor -- and once
// more per allocation after every hipPointerCheckpoint() of the calling thread,
// whether the allocation is still the one remembered.
int hipDeviceForPointer(const void* ptr);

// Marks the start of a unit of work on this thread (a message, a send, a
// recv): remembered answers of hipDeviceForPointer are checked against the
// runtime once before they are used again, so that an address which has been
// freed and handed out anew since is not taken for what it used to be.
void hipPointerCheckpoint();

class HipEvent {
 public:
  HipEvent(int device, bool interprocess = false) : device_(device) {
    TP_HIP_CHECK(tphip_event_create(device, interprocess ? 1 : 0, &ev_));
  }
  HipEvent(const HipEvent&) = delete;
  HipEvent& operator=(const HipEvent&) = delete;
  ~HipEvent() {
    if (ev_ != nullptr) {
      tphip_event_destroy(device_, ev_);
    }
  }
  void record(void* stream) {
    TP_HIP_CHECK(tphip_event_record(device_, ev_, stream));
  }
  // Make `stream` (on `streamDevice`) wait for the work captured by the last record.
  void wait(void* stream, int streamDevice) {
    TP_HIP_CHECK(tphip_stream_wait_event(streamDevice, stream, ev_));
  }
  bool query() {
    int done = 0;
    TP_HIP_CHECK(tphip_event_query(device_, ev_, &done));
    return done != 0;
  }
  void* raw() const {
    return ev_;
  }
  int device() const {
    return device_;
  }
  // The one stream this event is used on (see HipEventPool).
  void* home() const {
    return home_;
  }
  void setHome(void* stream) {
    home_ = stream;
  }

 private:
  int device_;
  void* ev_{nullptr};
  void* home_{nullptr};
};

// Recycles events so that the per-message path creates none. An event is only
// ever reused on the stream it was first used on. A caller may destroy its
// stream as soon as the callbacks of its operations have fired, and an event
// that had been recorded on such a stream and was later handed out for another
// one has been seen to fail its query there ("operation not permitted on an
// event last recorded in a capturing stream", with no capture anywhere): what
// the runtime remembers inside an event about the stream of its last record
// is not ours to rely on once that stream is gone. Events that touched a
// stream stay with it; they go away with the pool.
class HipEventPool {
 public:
  std::unique_ptr<HipEvent> get(int device, void* stream) {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      auto it = free_.find(Key{device, stream});
      if (it != free_.end() && !it->second.empty()) {
        auto ev = std::move(it->second.back());
        it->second.pop_back();
        return ev;
      }
    }
    auto ev = std::make_unique<HipEvent>(device);
    ev->setHome(stream);
    return ev;
  }
  void put(std::unique_ptr<HipEvent> ev) {
    std::lock_guard<std::mutex> lock(mutex_);
    auto& list = free_[Key{ev->device(), ev->home()}];
    if (list.size() < kMaxPerStream) {
      list.push_back(std::move(ev));
    }
  }

 private:
  static constexpr size_t kMaxPerStream = 64;
  using Key = std::pair<int, void*>;
  std::mutex mutex_;
  std::map<Key, std::vector<std::unique_ptr<HipEvent>>> free_;
};

// Pinned, device-mapped host slab (tensorpipe/common/cuda.h:183-188).
class HipPinnedSlab {
 public:
  HipPinnedSlab(int device, size_t bytes) : bytes_(bytes) {
    TP_HIP_CHECK(tphip_host_alloc(device, bytes, &host_, &dev_));
  }
  HipPinnedSlab(const HipPinnedSlab&) = delete;
  ~HipPinnedSlab() {
    if (host_ != nullptr) {
      tphip_host_free(host_);
    }
  }
  uint8_t* host() const {
    return static_cast<uint8_t*>(host_);
  }
  // Address of the same bytes as seen by kernels.
  uint8_t* dev() const {
    return static_cast<uint8_t*>(dev_);
  }
  size_t size() const {
    return bytes_;
  }

 private:
  size_t bytes_;
  void* host_{nullptr};
  void* dev_{nullptr};
};

// Device slab (tensorpipe/common/cuda.h:213-218).
class HipDeviceSlab {
 public:
  HipDeviceSlab(int device, size_t bytes) : device_(device), bytes_(bytes) {
    TP_HIP_CHECK(tphip_malloc(device, bytes, &ptr_));
  }
  HipDeviceSlab(const HipDeviceSlab&) = delete;
  ~HipDeviceSlab() {
    if (ptr_ != nullptr) {
      tphip_free(device_, ptr_);
    }
  }
  uint8_t* ptr() const {
    return static_cast<uint8_t*>(ptr_);
  }
  size_t size() const {
    return bytes_;
  }
  int device() const {
    return device_;
  }

 private:
  int device_;
  size_t bytes_;
  void* ptr_{nullptr};
};

TP_AMD_NAMESPACE_END
