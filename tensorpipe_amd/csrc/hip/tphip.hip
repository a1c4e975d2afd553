// libtphip.so: the C ABI declared in include/tphip.h. Thin, exception-free
// wrappers over the HIP runtime plus the launch logic of the batched copy
// kernel. Nothing here knows about channels or pipes.

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>
#include <tuple>
#include <vector>

#include "copy_kernels.hip.h"
#include "tphip.h"

namespace {

using namespace tphip;

#define TPHIP_TRY(expr)                     \
  do {                                      \
    hipError_t e_ = (expr);                 \
    if (e_ != hipSuccess) {                 \
      (void)hipGetLastError();              \
      return static_cast<int>(e_);          \
    }                                       \
  } while (0)

constexpr int kMaxDevices = 16;
constexpr uint32_t kPlanSlots = 32;
// One plan = prefix[n+1] (padded to 16 B), n body pointer pairs, n descriptors.
constexpr size_t kPlanSlotBytes =
    ((TPHIP_MAX_BATCH + 1) * sizeof(uint32_t) + 15) / 16 * 16 +
    TPHIP_MAX_BATCH * (sizeof(CopyBody) + sizeof(tphip_copy_desc));
// Plans for small tables are packed into sub-slots so that a burst of
// messages does not wait for a slot.
constexpr uint64_t kMaxTableVectors = 0xFFFFFFFFull - 64ull * 8ull;
std::atomic<uint64_t> gTableLimit{kMaxTableVectors}; // lowered by tests only

struct DeviceState {
  std::atomic<bool> ready{false};
  std::mutex initMutex;
  int numCus{0};
  // Ring of plan slots: host side (pinned, device-mapped) and device side.
  char* hostPlans{nullptr};
  char* hostPlansDev{nullptr};
  char* devPlans{nullptr};
  hipEvent_t slotDone[kPlanSlots]{};
  bool slotUsed[kPlanSlots]{};
  uint32_t nextSlot{0};
  std::mutex mutex; // nextSlot
  std::mutex slotMutex[kPlanSlots]; // a slot from the wait for its last user to the record behind its next
  // Launch profiling (tphip_profile_start/stop).
  std::mutex profMutex;
  bool profiling{false};
  uint32_t profUsed{0};
  uint64_t profBytes{0};
  std::vector<std::pair<hipEvent_t, hipEvent_t>> profEvents;
};

// While profiling is on, hands a pair of timing events to the next kernel
// launch of this thread; the runtime stamps them with the kernel's own start
// and end, so their distance is the kernel's execution time.
thread_local hipEvent_t tlsProfStart = nullptr;
thread_local hipEvent_t tlsProfStop = nullptr;
// Event to attach to the next copy-kernel launch of this thread as its
// completion signal (instead of a marker of its own behind the kernel).
thread_local hipEvent_t tlsSignal = nullptr;
// Gate for the copy launches of this thread's current call (tphip_batched_copy_gated).
thread_local Gate tlsGate = {nullptr};

class ProfileScope {
 public:
  ProfileScope(DeviceState& st, hipStream_t /*stream*/, uint64_t bytes) {
    std::lock_guard<std::mutex> lock(st.profMutex);
    if (!st.profiling) {
      return;
    }
    if (st.profUsed >= st.profEvents.size()) {
      return;
    }
    auto& pair = st.profEvents[st.profUsed++];
    st.profBytes += bytes;
    tlsProfStart = pair.first;
    tlsProfStop = pair.second;
  }
  ~ProfileScope() {
    tlsProfStart = nullptr;
    tlsProfStop = nullptr;
  }
};

DeviceState gDevices[kMaxDevices];

// Launch shape defaults, from sweeps on MI355X (256 CUs, 256 MiB Infinity
// Cache). Each can be overridden through the environment for experiments.
int envInt(const char* name, int fallback) {
  const char* e = getenv(name);
  return e != nullptr ? atoi(e) : fallback;
}

// 16-byte vectors in flight per lane.
int defaultUnroll(bool table) {
  static const int single = [] {
    int u = envInt("TPHIP_COPY_UNROLL", 4);
    return (u == 1 || u == 2 || u == 4 || u == 8) ? u : 4;
  }();
  static const int multi = [] {
    int u = envInt("TPHIP_TABLE_UNROLL", 2);
    return (u == 1 || u == 2 || u == 4 || u == 8) ? u : 2;
  }();
  return table ? multi : single;
}

// Workgroups per CU: one for the single-entry kernel (the grid then sweeps one
// compact window of memory at a time), four for the table kernel (its lookups
// need more wavefronts to hide behind).
int defaultBlocksPerCu(bool table) {
  static const int single = [] {
    int b = envInt("TPHIP_COPY_BLOCKS_PER_CU", 1);
    return b > 0 && b <= 64 ? b : 1;
  }();
  static const int multi = [] {
    int b = envInt("TPHIP_TABLE_BLOCKS_PER_CU", 4);
    return b > 0 && b <= 64 ? b : 4;
  }();
  return table ? multi : single;
}

// Copies of two pieces and more leave as launches of this many bytes each
// (TPHIP_COPY_SPLIT_BYTES, 0 = never split).
uint64_t splitPieceBytes() {
  static const uint64_t v = [] {
    const char* e = getenv("TPHIP_COPY_SPLIT_BYTES");
    uint64_t b = e != nullptr ? strtoull(e, nullptr, 10) : (256ull << 20);
    return b / 4096 * 4096; // pieces keep the alignment of the whole
  }();
  return v;
}

// Cache policy mask (bit 0 = nontemporal loads, bit 1 = nontemporal stores),
// by the bytes of the launch. Up to 64 MiB everything may stay in the caches
// (256 MiB Infinity Cache): the bytes were usually just produced and will be
// consumed next, and a copy that reads what another copy has just written runs
// 15 % faster when that one's stores were cached (64 MiB ping-pong between two
// processes: 86 % of the HBM roofline against 75 % with streaming loads and
// stores). Up to 128 MiB -- source and destination together still fit that
// cache -- the stores stream and the loads do not: a source that is sent again
// or was just produced is found there (the 112 MiB many-tensor message: 39 us
// against 44 with streaming loads). Beyond that nothing of the kind survives
// until it is needed and both stream past the caches: 256 MiB 79-80 % against
// 76 % with cached loads and 74 % with everything cached, in the same
// ping-pong and over rotating buffers alike; 1 GiB 74-78 % against 72 %.
// A table of several entries keeps its stores cached in the middle band too:
// the bytes before and after an entry's vectors share their lines with
// streamed vectors, and a line that leaves the L2 half written is merged in
// memory (256 ragged tensors, 112 MiB: 37.7 us against 38.6 with streaming
// stores; every tensor ending 6 bytes past a vector: 36.0 against 37.1).
int defaultNontemporal(uint64_t totalBytes, bool table) {
  static const int forced = envInt("TPHIP_COPY_NT", -1);
  if (forced >= 0) {
    return forced & 3;
  }
  if (totalBytes <= (64ull << 20)) {
    return 0;
  }
  if (totalBytes <= (128ull << 20)) {
    return table ? 0 : 2;
  }
  return 3;
}

int planViaKernel() {
  static int v = [] {
    const char* e = getenv("TPHIP_PLAN_STAGE_KERNEL");
    return e ? (atoi(e) != 0) : 1;
  }();
  return v;
}

// Makes `dev` the calling thread's current device for the lifetime of the
// object and puts the previous one back afterwards, so that no entry point
// leaves the caller on another device (the role of CudaDeviceGuard,
// tensorpipe/common/cuda.h:168-179).
class DeviceScope {
 public:
  explicit DeviceScope(int dev) {
    err_ = hipGetDevice(&prev_);
    if (err_ == hipSuccess && prev_ != dev) {
      err_ = hipSetDevice(dev);
      changed_ = err_ == hipSuccess;
    }
    if (err_ != hipSuccess) {
      (void)hipGetLastError();
    }
  }
  ~DeviceScope() {
    if (changed_) {
      (void)hipSetDevice(prev_);
    }
  }
  DeviceScope(const DeviceScope&) = delete;
  DeviceScope& operator=(const DeviceScope&) = delete;
  int error() const {
    return static_cast<int>(err_);
  }

 private:
  int prev_{0};
  bool changed_{false};
  hipError_t err_{hipSuccess};
};

#define TPHIP_ON_DEVICE(dev)          \
  DeviceScope deviceScope_(dev);      \
  if (deviceScope_.error() != 0) {    \
    return deviceScope_.error();      \
  }

// TPHIP_INLINE_PLANS=0 sends small tables through the plan ring as well (A/B switch).
bool inlinePlansEnabled() {
  static const bool v = envInt("TPHIP_INLINE_PLANS", 1) != 0;
  return v;
}

int getDevice(int dev, DeviceState** out) {
  if (dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  DeviceState& st = gDevices[dev];
  TPHIP_ON_DEVICE(dev);
  // A failure is reported and forgotten: the next call tries again from the
  // start (an allocation refused once, say while another thread's stream is
  // being captured, must not disable the device for the rest of the process).
  if (!st.ready.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(st.initMutex);
    if (!st.ready.load(std::memory_order_relaxed)) {
      int cus = 0;
      char* hostPlans = nullptr;
      char* hostPlansDev = nullptr;
      char* devPlans = nullptr;
      hipEvent_t slotDone[kPlanSlots]{};
      hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e == hipSuccess) {
        e = hipHostMalloc(
            reinterpret_cast<void**>(&hostPlans),
            kPlanSlots * kPlanSlotBytes,
            hipHostMallocMapped | hipHostMallocPortable);
      }
      if (e == hipSuccess) {
        e = hipHostGetDevicePointer(reinterpret_cast<void**>(&hostPlansDev), hostPlans, 0);
      }
      if (e == hipSuccess) {
        e = hipMalloc(reinterpret_cast<void**>(&devPlans), kPlanSlots * kPlanSlotBytes);
      }
      for (uint32_t i = 0; e == hipSuccess && i < kPlanSlots; ++i) {
        e = hipEventCreateWithFlags(&slotDone[i], hipEventDisableTiming);
      }
      if (e != hipSuccess) {
        (void)hipGetLastError();
        for (uint32_t i = 0; i < kPlanSlots; ++i) {
          if (slotDone[i] != nullptr) {
            (void)hipEventDestroy(slotDone[i]);
          }
        }
        if (devPlans != nullptr) {
          (void)hipFree(devPlans);
        }
        if (hostPlans != nullptr) {
          (void)hipHostFree(hostPlans);
        }
        (void)hipGetLastError();
        return static_cast<int>(e);
      }
      st.numCus = cus;
      st.hostPlans = hostPlans;
      st.hostPlansDev = hostPlansDev;
      st.devPlans = devPlans;
      for (uint32_t i = 0; i < kPlanSlots; ++i) {
        st.slotDone[i] = slotDone[i];
      }
      st.ready.store(true, std::memory_order_release);
    }
  }
  *out = &st;
  return 0;
}

// Launch through hipLaunchKernel so that the error code is this launch's own
// (hipGetLastError would also report stale errors of unrelated earlier calls).
template <typename... Params, typename... Args>
int launchKernel(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                 Args... args) {
  std::tuple<Params...> values{static_cast<Params>(args)...};
  void* argv[sizeof...(Params)];
  size_t i = 0;
  std::apply([&](auto&... v) { ((argv[i++] = static_cast<void*>(&v)), ...); }, values);
  hipError_t e;
  if (tlsProfStart != nullptr || tlsProfStop != nullptr) {
    e = hipExtLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, argv, lds, stream,
                           tlsProfStart, tlsProfStop, 0);
    tlsProfStart = nullptr;
    tlsProfStop = nullptr;
  } else if (tlsSignal != nullptr) {
    e = hipExtLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, argv, lds, stream,
                           nullptr, tlsSignal, 0);
    if (e == hipSuccess) {
      tlsSignal = nullptr; // attached
    }
  } else {
    e = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, argv, lds, stream);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
  }
  return static_cast<int>(e);
}

template <int NT>
int launchSingle(int unroll, uint32_t blocks, hipStream_t stream, const char* src, char* dst,
                 uint64_t bytes) {
  switch (unroll) {
    case 1:
      return launchKernel(single_copy_kernel<1, NT>, dim3(blocks), dim3(kBlockThreads), 0, stream, src,
                          dst, bytes, tlsGate);
    case 2:
      return launchKernel(single_copy_kernel<2, NT>, dim3(blocks), dim3(kBlockThreads), 0, stream, src,
                          dst, bytes, tlsGate);
    case 8:
      return launchKernel(single_copy_kernel<8, NT>, dim3(blocks), dim3(kBlockThreads), 0, stream, src,
                          dst, bytes, tlsGate);
    default:
      return launchKernel(single_copy_kernel<4, NT>, dim3(blocks), dim3(kBlockThreads), 0, stream, src,
                          dst, bytes, tlsGate);
  }
}

template <int NT>
int launchTable(int unroll, uint32_t blocks, size_t lds, hipStream_t stream,
                const uint32_t* prefix, const CopyBody* bodies, const tphip_copy_desc* descs,
                uint32_t n, uint32_t nchunks) {
  switch (unroll) {
    case 1:
      return launchKernel(batched_copy_kernel<1, NT>, dim3(blocks), dim3(kBlockThreads), lds, stream,
                          prefix, bodies, descs, n, nchunks, tlsGate);
    case 2:
      return launchKernel(batched_copy_kernel<2, NT>, dim3(blocks), dim3(kBlockThreads), lds, stream,
                          prefix, bodies, descs, n, nchunks, tlsGate);
    case 8:
      return launchKernel(batched_copy_kernel<8, NT>, dim3(blocks), dim3(kBlockThreads), lds, stream,
                          prefix, bodies, descs, n, nchunks, tlsGate);
    default:
      return launchKernel(batched_copy_kernel<4, NT>, dim3(blocks), dim3(kBlockThreads), lds, stream,
                          prefix, bodies, descs, n, nchunks, tlsGate);
  }
}

template <int NT, uint32_t N>
int launchInline(int unroll, uint32_t blocks, hipStream_t stream, const InlinePlanT<N>& plan) {
  switch (unroll) {
    case 1:
      return launchKernel(inline_copy_kernel<1, NT, N>, dim3(blocks), dim3(kBlockThreads), 0, stream, plan,
                          tlsGate);
    case 2:
      return launchKernel(inline_copy_kernel<2, NT, N>, dim3(blocks), dim3(kBlockThreads), 0, stream, plan,
                          tlsGate);
    case 8:
      return launchKernel(inline_copy_kernel<8, NT, N>, dim3(blocks), dim3(kBlockThreads), 0, stream, plan,
                          tlsGate);
    default:
      return launchKernel(inline_copy_kernel<4, NT, N>, dim3(blocks), dim3(kBlockThreads), 0, stream, plan,
                          tlsGate);
  }
}

// Workgroups for `units` work units of one workgroup-iteration each: enough to
// give every unit a workgroup, capped at blocksPerCu * CUs (or `blocks`).
uint32_t pickBlocks(int numCus, uint64_t units, uint32_t minBlocks, uint32_t blocks, bool table) {
  uint64_t want = units > minBlocks ? units : minBlocks;
  if (want == 0) {
    want = 1;
  }
  const uint64_t cap = blocks != 0
      ? blocks
      : static_cast<uint64_t>(numCus > 0 ? numCus : 256) * defaultBlocksPerCu(table);
  return static_cast<uint32_t>(want < cap ? want : cap);
}

int copySingle(DeviceState& st, const tphip_copy_desc& d, hipStream_t stream, int unroll,
               uint32_t blocks, int nt) {
  if (d.bytes == 0) {
    return 0;
  }
  if (d.src == nullptr || d.dst == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  if (unroll == 0) {
    unroll = defaultUnroll(false);
  }
  if (nt < 0) {
    nt = defaultNontemporal(d.bytes, false);
  }
  const char* src = static_cast<const char*>(d.src);
  char* dst = static_cast<char*>(d.dst);
  ProfileScope prof(st, stream, d.bytes);
  auto launchOne = [&](const char* s, char* t, uint64_t bytes) {
    const uint64_t nvec = bytes >> 4;
    const uint64_t perBlock = uint64_t(kBlockThreads) * unroll;
    const uint32_t grid = pickBlocks(st.numCus, (nvec + perBlock - 1) / perBlock, 1, blocks, false);
    switch (nt & 3) {
      case 0:
        return launchSingle<0>(unroll, grid, stream, s, t, bytes);
      case 1:
        return launchSingle<1>(unroll, grid, stream, s, t, bytes);
      case 2:
        return launchSingle<2>(unroll, grid, stream, s, t, bytes);
      default:
        return launchSingle<3>(unroll, grid, stream, s, t, bytes);
    }
  };
  // A very large copy goes out as several launches in a row. The workgroups of
  // one launch sweep memory as one compact window only while they keep pace;
  // over hundreds of iterations they drift apart and the window widens (1 GiB
  // in one launch: 357 us; as four of 256 MiB: 337 us, the three gaps between
  // kernels included; as eight: 342 us; 256 MiB itself loses when split).
  const uint64_t piece = splitPieceBytes();
  if (piece == 0 || d.bytes < 2 * piece) {
    return launchOne(src, dst, d.bytes);
  }
  const uint64_t pieces = d.bytes / piece; // the last one takes the remainder
  // What rides on "the" launch is spread over the row: a gate holds the first
  // piece back (the others follow in stream order), the completion signal and
  // the profiling stop belong to the last one, the profiling start to the first.
  const hipEvent_t signal = tlsSignal;
  const hipEvent_t profStart = tlsProfStart;
  const hipEvent_t profStop = tlsProfStop;
  const Gate gate = tlsGate;
  struct Restore {
    Gate gate;
    ~Restore() {
      tlsGate = gate;
    }
  } restore{gate};
  tlsSignal = nullptr;
  tlsProfStart = nullptr;
  tlsProfStop = nullptr;
  for (uint64_t k = 0; k < pieces; ++k) {
    const bool first = k == 0;
    const bool last = k + 1 == pieces;
    const uint64_t offset = k * piece;
    const uint64_t bytes = last ? d.bytes - offset : piece;
    tlsGate = first ? gate : Gate{nullptr};
    tlsProfStart = first ? profStart : nullptr;
    tlsProfStop = last ? profStop : nullptr;
    if (last && profStart == nullptr && profStop == nullptr) {
      tlsSignal = signal;
    }
    const int rc = launchOne(src + offset, dst + offset, bytes);
    if (rc != 0) {
      tlsSignal = signal; // not attached: for the caller to see
      return rc;
    }
  }
  if (profStart != nullptr || profStop != nullptr) {
    tlsSignal = signal; // the profiling events took the last launch's slots: the caller records it
  }
  return 0;
}

// A table of at most N entries, plan in the kernel arguments.
template <uint32_t N>
int copyInline(DeviceState& st, const tphip_copy_desc* table, uint32_t n, hipStream_t stream,
               int unroll, uint32_t blocks, int nt, uint64_t payloadBytes) {
  InlinePlanT<N> plan;
  plan.n = n;
  uint64_t total = 0;
  for (uint32_t i = 0; i < n; ++i) {
    plan.prefix[i] = static_cast<uint32_t>(total);
    const uint64_t bytes = table[i].bytes;
    uint64_t head = (0 - reinterpret_cast<uintptr_t>(table[i].dst)) & 15u;
    if (head > bytes) {
      head = bytes;
    }
    plan.bodies[i].src = static_cast<const char*>(table[i].src) + head;
    plan.bodies[i].dst = static_cast<char*>(table[i].dst) + head;
    plan.edges[i] = static_cast<uint8_t>((head << 4) | ((bytes - head) & 15u));
    total += (bytes - head) >> 4;
  }
  for (uint32_t i = n; i < N + 2; ++i) {
    plan.prefix[i] = static_cast<uint32_t>(total); // prefix[n] = total; the rest is never read
  }
  for (uint32_t i = n; i < N; ++i) {
    plan.edges[i] = 0;
  }
  const uint64_t chunk = uint64_t(kBlockThreads) * unroll;
  plan.nchunks = static_cast<uint32_t>((total + chunk - 1) / chunk);
  const uint32_t edgeBlocks = (n + kEdgeGroup * kWavesPerBlock - 1) / (kEdgeGroup * kWavesPerBlock);
  const uint32_t grid = pickBlocks(st.numCus, plan.nchunks, edgeBlocks, blocks, true);
  ProfileScope prof(st, stream, payloadBytes);
  switch (nt & 3) {
    case 0:
      return launchInline<0>(unroll, grid, stream, plan);
    case 1:
      return launchInline<1>(unroll, grid, stream, plan);
    case 2:
      return launchInline<2>(unroll, grid, stream, plan);
    default:
      return launchInline<3>(unroll, grid, stream, plan);
  }
}

// Launch one table kernel over table[0..n) whose body vector total fits 32 bits.
int copyTable(DeviceState& st, const tphip_copy_desc* table, uint32_t n, hipStream_t stream,
              int unroll, uint32_t blocks, int nt) {
  if (unroll == 0) {
    unroll = defaultUnroll(true);
  }
  uint64_t payloadBytes = 0;
  for (uint32_t i = 0; i < n; ++i) {
    payloadBytes += table[i].bytes;
  }
  if (nt < 0) {
    nt = defaultNontemporal(payloadBytes, true);
  }

  if (n <= kInlineEntries && inlinePlansEnabled()) {
    // The whole plan fits the kernel arguments.
    return n <= kInlineEntriesSmall
        ? copyInline<kInlineEntriesSmall>(st, table, n, stream, unroll, blocks, nt, payloadBytes)
        : copyInline<kInlineEntries>(st, table, n, stream, unroll, blocks, nt, payloadBytes);
  }

  // The plan ring is rewritten by later calls: a graph that captured this
  // launch would replay it over someone else's plan.
  if (stream != nullptr) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    TPHIP_TRY(hipStreamIsCapturing(stream, &capture));
    if (capture != hipStreamCaptureStatusNone) {
      return TPHIP_ERR_CAPTURING;
    }
  }

  const size_t prefixBytes = ((size_t(n) + 1) * sizeof(uint32_t) + 15) / 16 * 16;
  const size_t bodyBytes = size_t(n) * sizeof(CopyBody);
  const size_t planBytes = prefixBytes + bodyBytes + size_t(n) * sizeof(tphip_copy_desc);
  const size_t planBytesPadded = (planBytes + 15) / 16 * 16;

  uint32_t slot;
  {
    std::lock_guard<std::mutex> lock(st.mutex);
    slot = st.nextSlot;
    st.nextSlot = (st.nextSlot + 1) % kPlanSlots;
  }
  {
    // Only this slot is held while its last user is waited for: a slow stream
    // there does not hold up table launches that take other slots.
    std::lock_guard<std::mutex> lock(st.slotMutex[slot]);
    if (st.slotUsed[slot]) {
      // The launch that last used this slot must have consumed its plan.
      TPHIP_TRY(hipEventSynchronize(st.slotDone[slot]));
    }
    st.slotUsed[slot] = true;

    char* host = st.hostPlans + size_t(slot) * kPlanSlotBytes;
    char* hostDev = st.hostPlansDev + size_t(slot) * kPlanSlotBytes;
    char* devp = st.devPlans + size_t(slot) * kPlanSlotBytes;
    uint32_t* prefix = reinterpret_cast<uint32_t*>(host);
    CopyBody* hostBodies = reinterpret_cast<CopyBody*>(host + prefixBytes);
    uint64_t total = 0;
    for (uint32_t i = 0; i < n; ++i) {
      prefix[i] = static_cast<uint32_t>(total);
      const uint64_t bytes = table[i].bytes;
      uint64_t head = (0 - reinterpret_cast<uintptr_t>(table[i].dst)) & 15u;
      if (head > bytes) {
        head = bytes;
      }
      hostBodies[i].src = static_cast<const char*>(table[i].src) + head;
      hostBodies[i].dst = static_cast<char*>(table[i].dst) + head;
      total += (bytes - head) >> 4;
    }
    prefix[n] = static_cast<uint32_t>(total);
    memcpy(host + prefixBytes + bodyBytes, table, size_t(n) * sizeof(tphip_copy_desc));

    if (planViaKernel()) {
      const uint32_t nv = static_cast<uint32_t>(planBytesPadded / 16);
      const uint32_t sb = (nv + kBlockThreads - 1) / kBlockThreads;
      hipEvent_t heldSignal = tlsSignal; // belongs to the copy kernel, not to this one
      tlsSignal = nullptr;
      int src = launchKernel(stage_plan_kernel, dim3(sb < 8 ? sb : 8), dim3(kBlockThreads), 0,
                             stream, reinterpret_cast<const u32x4*>(hostDev),
                             reinterpret_cast<u32x4*>(devp), nv);
      if (src != 0) {
        return src;
      }
      tlsSignal = heldSignal;
    } else {
      TPHIP_TRY(hipMemcpyAsync(devp, host, planBytesPadded, hipMemcpyHostToDevice, stream));
    }

    const uint64_t chunk = uint64_t(kBlockThreads) * unroll;
    const uint32_t nchunks = static_cast<uint32_t>((total + chunk - 1) / chunk);
    // one wave per kEdgeGroup entries for the heads and tails
    const uint32_t edgeBlocks = (n + kEdgeGroup * kWavesPerBlock - 1) / (kEdgeGroup * kWavesPerBlock);
    const uint32_t grid = pickBlocks(st.numCus, nchunks, edgeBlocks, blocks, true);
    const size_t lds = prefixBytes + (n <= kLdsBodies ? bodyBytes : 0);
    const uint32_t* dPrefix = reinterpret_cast<const uint32_t*>(devp);
    const CopyBody* dBodies = reinterpret_cast<const CopyBody*>(devp + prefixBytes);
    const tphip_copy_desc* dDescs =
        reinterpret_cast<const tphip_copy_desc*>(devp + prefixBytes + bodyBytes);
    int rc;
    {
      ProfileScope prof(st, stream, payloadBytes);
      switch (nt & 3) {
        case 0:
          rc = launchTable<0>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, n, nchunks);
          break;
        case 1:
          rc = launchTable<1>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, n, nchunks);
          break;
        case 2:
          rc = launchTable<2>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, n, nchunks);
          break;
        default:
          rc = launchTable<3>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, n, nchunks);
          break;
      }
    }
    if (rc != 0) {
      return rc;
    }
    TPHIP_TRY(hipEventRecord(st.slotDone[slot], stream));
  }
  return 0;
}

int batchedCopyImpl(int dev, const tphip_copy_desc* table, uint32_t n, void* streamPtr,
                    int unroll, uint32_t blocks, int nt, hipEvent_t signal = nullptr) {
  if (table == nullptr && n != 0) {
    return TPHIP_ERR_INVALID_ARG;
  }
  if (signal != nullptr) {
    // Validate before anything is enqueued, then make sure the event ends up
    // behind whatever this call enqueues, on every path that succeeds.
    if (n > TPHIP_MAX_BATCH ||
        !(unroll == 0 || unroll == 1 || unroll == 2 || unroll == 4 || unroll == 8) || dev < 0 ||
        dev >= kMaxDevices) {
      return batchedCopyImpl(dev, table, n, streamPtr, unroll, blocks, nt);
    }
    struct Disarm {
      ~Disarm() {
        tlsSignal = nullptr;
      }
    } disarm;
    tlsSignal = signal;
    int rc = batchedCopyImpl(dev, table, n, streamPtr, unroll, blocks, nt);
    if (rc == 0 && tlsSignal != nullptr) {
      // Nothing was launched, or the launch carried profiling events: a marker of its own.
      TPHIP_ON_DEVICE(dev);
      TPHIP_TRY(hipEventRecord(signal, static_cast<hipStream_t>(streamPtr)));
    }
    return rc;
  }
  if (n == 0) {
    return 0;
  }
  if (n > TPHIP_MAX_BATCH) {
    return TPHIP_ERR_TOO_LARGE;
  }
  // unroll 0 and nt < 0 select the defaults, resolved per launch.
  if (!(unroll == 0 || unroll == 1 || unroll == 2 || unroll == 4 || unroll == 8)) {
    return TPHIP_ERR_INVALID_ARG;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  DeviceState* st = nullptr;
  int rc = getDevice(dev, &st);
  if (rc != 0) {
    return rc;
  }
  hipStream_t stream = static_cast<hipStream_t>(streamPtr);

  // Drop empty entries up front; reject null pointers on non-empty ones.
  std::vector<tphip_copy_desc> live;
  const tphip_copy_desc* cur = table;
  uint32_t m = n;
  bool anyEmpty = false;
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].bytes == 0) {
      anyEmpty = true;
    } else if (table[i].src == nullptr || table[i].dst == nullptr) {
      return TPHIP_ERR_INVALID_ARG;
    }
  }
  if (anyEmpty) {
    live.reserve(n);
    for (uint32_t i = 0; i < n; ++i) {
      if (table[i].bytes != 0) {
        live.push_back(table[i]);
      }
    }
    cur = live.data();
    m = static_cast<uint32_t>(live.size());
    if (m == 0) {
      return 0;
    }
  }

  // Cut into launches whose body vector total fits the 32-bit prefix; entries
  // too large for that go through the single-entry kernel (64-bit counts).
  const uint64_t limit = gTableLimit.load(std::memory_order_relaxed);
  // A completion event rides on the last launch of the call only.
  hipEvent_t heldSignal = tlsSignal;
  tlsSignal = nullptr;
  bool armed = false;
  uint32_t begin = 0;
  uint64_t acc = 0;
  for (uint32_t i = 0; i <= m; ++i) {
    const uint64_t vecs = i < m ? (cur[i].bytes >> 4) : 0;
    const bool huge = i < m && vecs > limit;
    if (i == m || huge || acc + vecs > limit) {
      const uint32_t cnt = i - begin;
      if (cnt >= 1 && i == m) {
        tlsSignal = heldSignal;
        armed = true;
      }
      if (cnt == 1) {
        rc = copySingle(*st, cur[begin], stream, unroll, blocks, nt);
      } else if (cnt > 1) {
        rc = copyTable(*st, cur + begin, cnt, stream, unroll, blocks, nt);
      }
      if (rc != 0) {
        return rc;
      }
      begin = i;
      acc = 0;
      if (huge) {
        if (i + 1 == m) {
          tlsSignal = heldSignal;
          armed = true;
        }
        rc = copySingle(*st, cur[i], stream, unroll, blocks, nt);
        if (rc != 0) {
          return rc;
        }
        begin = i + 1;
        continue;
      }
    }
    acc += vecs;
  }
  if (!armed) {
    tlsSignal = heldSignal; // not attached: the caller records it behind the copies
  }
  return 0;
}

// ---- the entry point that allocates nothing ---------------------------------
//
// Its plan lives in a device array of the library image instead of the plan
// ring (which is allocated on first use). Each GPU holds its own copy of the
// array at its own address; the name below is only the host-side handle that
// hipGetSymbolAddress turns into that address, once per device.
constexpr size_t kNoAllocPrefixBytes =
    ((TPHIP_NOALLOC_MAX_BATCH + 1) * sizeof(uint32_t) + 15) / 16 * 16;
constexpr size_t kNoAllocPlanBytes =
    kNoAllocPrefixBytes + TPHIP_NOALLOC_MAX_BATCH * (sizeof(CopyBody) + sizeof(tphip_copy_desc));
constexpr size_t kNoAllocScratchBytes = (kNoAllocPlanBytes + 255) / 256 * 256;

static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

struct NoAllocDevice {
  std::mutex mutex;
  std::atomic<bool> ready{false};
  int numCus{0};
  char* scratchPtr{nullptr}; // this device's copy of `scratch`
};
NoAllocDevice gNoAlloc[kMaxDevices];

// Call with `dev` current. A failed set-up is not remembered: the next call
// tries again (a query refused once, say on a stream that is being captured,
// must not disable the entry point for the rest of the process).
int getNoAllocDevice(int dev, NoAllocDevice** out) {
  NoAllocDevice& st = gNoAlloc[dev];
  if (!st.ready.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(st.mutex);
    if (!st.ready.load(std::memory_order_relaxed)) {
      int cus = 0;
      void* p = nullptr;
      hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e == hipSuccess) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      }
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
      }
      if (p == nullptr || cus <= 0) {
        return TPHIP_ERR_INVALID_ARG;
      }
      st.numCus = cus;
      st.scratchPtr = static_cast<char*>(p);
      st.ready.store(true, std::memory_order_release);
    }
  }
  *out = &st;
  return 0;
}

int noAllocCopy(int dev, const tphip_copy_desc* table, uint32_t n, hipStream_t stream) {
  if (table == nullptr && n != 0) {
    return TPHIP_ERR_INVALID_ARG;
  }
  if (n > TPHIP_NOALLOC_MAX_BATCH) {
    return TPHIP_ERR_TOO_LARGE;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].bytes != 0 && (table[i].src == nullptr || table[i].dst == nullptr)) {
      return TPHIP_ERR_INVALID_ARG;
    }
  }
  TPHIP_ON_DEVICE(dev);
  NoAllocDevice* st = nullptr;
  int rc = getNoAllocDevice(dev, &st);
  if (rc != 0) {
    return rc;
  }

  // The plan, built on the stack: prefix | bodies | descriptors of the
  // non-empty entries (the layout batched_copy_kernel reads).
  alignas(16) unsigned char plan[kNoAllocPlanBytes];
  uint32_t m = 0;
  for (uint32_t i = 0; i < n; ++i) {
    m += table[i].bytes != 0 ? 1 : 0;
  }
  if (m == 0) {
    return 0;
  }
  const size_t prefixBytes = ((size_t(m) + 1) * sizeof(uint32_t) + 15) / 16 * 16;
  const size_t bodyBytes = size_t(m) * sizeof(CopyBody);
  const size_t planBytes = prefixBytes + bodyBytes + size_t(m) * sizeof(tphip_copy_desc);
  memset(plan, 0, prefixBytes);
  uint32_t* prefix = reinterpret_cast<uint32_t*>(plan);
  CopyBody* bodies = reinterpret_cast<CopyBody*>(plan + prefixBytes);
  tphip_copy_desc* descs = reinterpret_cast<tphip_copy_desc*>(plan + prefixBytes + bodyBytes);
  uint64_t total = 0;
  uint64_t payloadBytes = 0;
  uint32_t k = 0;
  for (uint32_t i = 0; i < n; ++i) {
    const uint64_t bytes = table[i].bytes;
    if (bytes == 0) {
      continue;
    }
    uint64_t head = (0 - reinterpret_cast<uintptr_t>(table[i].dst)) & 15u;
    if (head > bytes) {
      head = bytes;
    }
    prefix[k] = static_cast<uint32_t>(total);
    bodies[k].src = static_cast<const char*>(table[i].src) + head;
    bodies[k].dst = static_cast<char*>(table[i].dst) + head;
    descs[k] = table[i];
    total += (bytes - head) >> 4;
    payloadBytes += bytes;
    ++k;
    if (total > kMaxTableVectors) {
      return TPHIP_ERR_TOO_LARGE; // beyond what one launch can index
    }
  }
  prefix[m] = static_cast<uint32_t>(total);

  // Plan -> this device's scratch array, a kernel-argument load at a time.
  for (size_t off = 0; off < planBytes; off += kPlanPieceWords * 4) {
    PlanPiece piece;
    const size_t bytes = planBytes - off < kPlanPieceWords * 4 ? planBytes - off : kPlanPieceWords * 4;
    piece.words = static_cast<uint32_t>((bytes + 3) / 4);
    piece.byteOffset = static_cast<uint32_t>(off);
    memcpy(piece.data, plan + off, bytes);
    rc = launchKernel(write_plan_piece_kernel, dim3(1), dim3(kBlockThreads), 0, stream, piece,
                      st->scratchPtr);
    if (rc != 0) {
      return rc;
    }
  }

  const int unroll = defaultUnroll(true);
  const int nt = defaultNontemporal(payloadBytes, true);
  const uint64_t chunk = uint64_t(kBlockThreads) * unroll;
  const uint32_t nchunks = static_cast<uint32_t>((total + chunk - 1) / chunk);
  const uint32_t edgeBlocks = (m + kEdgeGroup * kWavesPerBlock - 1) / (kEdgeGroup * kWavesPerBlock);
  const uint32_t grid = pickBlocks(st->numCus, nchunks, edgeBlocks, 0, true);
  const size_t lds = prefixBytes + bodyBytes; // m <= kLdsBodies
  const char* devp = st->scratchPtr;
  const uint32_t* dPrefix = reinterpret_cast<const uint32_t*>(devp);
  const CopyBody* dBodies = reinterpret_cast<const CopyBody*>(devp + prefixBytes);
  const tphip_copy_desc* dDescs =
      reinterpret_cast<const tphip_copy_desc*>(devp + prefixBytes + bodyBytes);
  switch (nt & 3) {
    case 0:
      return launchTable<0>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, m, nchunks);
    case 1:
      return launchTable<1>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, m, nchunks);
    case 2:
      return launchTable<2>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, m, nchunks);
    default:
      return launchTable<3>(unroll, grid, lds, stream, dPrefix, dBodies, dDescs, m, nchunks);
  }
}

// ---- gates ------------------------------------------------------------------
//
// Verdicts of gate kernels, one word per gated call in flight, in a device
// array of the library image (each GPU has its own copy; the host-side name is
// turned into that GPU's address once).
constexpr uint32_t kGateStates = 256;
static __device__ __align__(256) uint64_t gateStates[kGateStates];

struct GateDevice {
  std::mutex mutex;
  std::atomic<bool> ready{false};
  int wallClockKhz{0};
  uint64_t* states{nullptr};
  std::atomic<uint64_t> next{0};
};
GateDevice gGateDevices[kMaxDevices];

// ---- resident copy agent ------------------------------------------------------

constexpr uint32_t kAgentRing = 64; // commands the host may have posted ahead

struct Agent {
  int dev{0};
  hipStream_t stream{nullptr};
  AgentCommand* ring{nullptr}; // pinned host memory, as the host sees it
  AgentCommand* ringDev{nullptr}; // and as kernels see it
  AgentControl* ctl{nullptr};
  AgentControl* ctlDev{nullptr};
  uint64_t idleTicks{0};
  uint64_t lifeTicks{0};
  std::mutex mutex;
  uint64_t nextTicket{1}; // under mutex
  std::atomic<uint64_t> epoch{0}; // of the last launch
  bool stopped{false}; // under mutex
};

uint64_t loadWord(const uint64_t* p) {
  return __atomic_load_n(p, __ATOMIC_ACQUIRE);
}

// With the mutex held: starts an agent unless one is (still) running.
int agentEnsureRunning(Agent& a) {
  const uint64_t epoch = a.epoch.load(std::memory_order_relaxed);
  if (epoch != 0 && loadWord(&a.ctl->exited) != epoch) {
    return 0;
  }
  // The previous agent has left: what it served is final.
  const uint64_t first = loadWord(&a.ctl->done) + 1;
  a.epoch.store(epoch + 1, std::memory_order_release);
  return launchKernel(agent_kernel, dim3(1), dim3(kWave), 0, a.stream, a.ringDev,
                      kAgentRing - 1, a.ctlDev, first, epoch + 1, a.idleTicks, a.lifeTicks);
}

struct HostFnThunk {
  tphip_host_fn fn;
  void* arg;
};

void hostFnTrampoline(hipStream_t, hipError_t status, void* userData) {
  HostFnThunk* t = static_cast<HostFnThunk*>(userData);
  t->fn(t->arg, static_cast<int>(status));
  delete t;
}

// Ticks of the wall clock per microsecond times 1000; 100 MHz where the runtime does not say.
int wallClockKhz(int dev) {
  static std::atomic<int> cached[kMaxDevices];
  int khz = cached[dev].load(std::memory_order_relaxed);
  if (khz == 0) {
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0) {
      (void)hipGetLastError();
      return 100000;
    }
    cached[dev].store(khz, std::memory_order_relaxed);
  }
  return khz;
}

template <bool PUSH>
int ringLaunch(int dev, const tphip_ring_end* ring, const void* user, uint64_t bytes, uint64_t firstSeq,
               uint32_t yieldUs, uint32_t blocks, void* stream, void* event) {
  if (ring == nullptr || ring->slots == nullptr || ring->slot_bytes == 0 || ring->slot_bytes % 16 != 0 ||
      ring->num_slots == 0 || ring->produced == nullptr || ring->consumed == nullptr ||
      ring->scratch == nullptr || ring->status == nullptr || ring->abort == nullptr || user == nullptr ||
      bytes == 0 || dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  RingArgs a;
  a.user = static_cast<char*>(const_cast<void*>(user));
  a.bytes = bytes;
  a.slots = static_cast<char*>(ring->slots);
  a.slotBytes = ring->slot_bytes;
  a.numSlots = ring->num_slots;
  a.firstSeq = firstSeq;
  a.produced = static_cast<uint64_t*>(ring->produced);
  a.consumed = static_cast<uint64_t*>(ring->consumed);
  a.scratch = static_cast<RingScratch*>(ring->scratch);
  a.status = static_cast<uint64_t*>(ring->status);
  a.abort = static_cast<const uint64_t*>(ring->abort);
  a.yieldTicks = static_cast<uint64_t>(yieldUs) * wallClockKhz(dev) / 1000;
  struct Disarm {
    ~Disarm() {
      tlsSignal = nullptr;
    }
  } disarm;
  tlsSignal = static_cast<hipEvent_t>(event);
  // Teams of workgroups that take chunks in turn: sixteen workgroups, each a
  // team of its own, moved the most through the host link with both
  // directions busy (256 MiB through a 16 MiB ring in 512 KiB chunks: 45 GB/s
  // against 39 with four teams of four, 37 with two of eight, 32 with one team;
  // 32 workgroups never beat 16). TPHIP_RING_GROUPS, TPHIP_RING_BLOCKS: tuning.
  static const uint32_t envGroups = static_cast<uint32_t>(envInt("TPHIP_RING_GROUPS", 16));
  static const uint32_t envBlocks = static_cast<uint32_t>(envInt("TPHIP_RING_BLOCKS", 16));
  uint32_t groups = envGroups > 0 ? envGroups : 1;
  groups = groups > ring->num_slots ? ring->num_slots : groups;
  uint32_t nblocks = blocks != 0 ? blocks : envBlocks;
  nblocks = (nblocks + groups - 1) / groups * groups;
  a.groups = groups;
  const dim3 grid(nblocks);
  int rc = launchKernel(ring_kernel<PUSH, 4>, grid, dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream), a);
  if (rc == 0 && tlsSignal != nullptr) {
    // launch profiling took the launch's event slots: record plainly
    rc = static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  }
  return rc;
}
} // namespace

extern "C" {

const char* tphip_strerror(int err) {
  switch (err) {
    case 0:
      return "success";
    case TPHIP_ERR_INVALID_ARG:
      return "tphip: invalid argument";
    case TPHIP_ERR_TOO_LARGE:
      return "tphip: table larger than this entry point takes in one call";
    case TPHIP_ERR_NO_DEVICE:
      return "tphip: no usable GPU";
    case TPHIP_ERR_BUSY:
      return "tphip: the copy agent's command ring is full";
    case TPHIP_ERR_CAPTURING:
      return "tphip: a table of more than 256 entries cannot be captured into a graph";
    default:
      return hipGetErrorString(static_cast<hipError_t>(err));
  }
}

int tphip_device_count(int* count) {
  if (count == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  *count = 0;
  hipError_t e = hipGetDeviceCount(count);
  if (e == hipErrorNoDevice) {
    *count = 0;
    (void)hipGetLastError();
    return 0;
  }
  return static_cast<int>(e);
}

int tphip_device_uuid(int dev, char out[TPHIP_UUID_STRLEN + 1]) {
  if (out == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  hipUUID uuid;
  TPHIP_TRY(hipDeviceGetUuid(&uuid, dev));
  static const char* hex = "0123456789abcdef";
  int o = 0;
  for (int i = 0; i < 16; ++i) {
    if (i == 4 || i == 6 || i == 8 || i == 10) {
      out[o++] = '-';
    }
    unsigned char b = static_cast<unsigned char>(uuid.bytes[i]);
    out[o++] = hex[b >> 4];
    out[o++] = hex[b & 15];
  }
  out[o] = '\0';
  return 0;
}

int tphip_device_for_ptr(const void* ptr, int* dev, int* is_host) {
  if (dev == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  hipPointerAttribute_t attr;
  memset(&attr, 0, sizeof(attr));
  hipError_t e = hipPointerGetAttributes(&attr, ptr);
  if (e == hipErrorInvalidValue) {
    // Plain host memory the runtime has never seen.
    (void)hipGetLastError();
    *dev = -1;
    if (is_host) {
      *is_host = 1;
    }
    return 0;
  }
  TPHIP_TRY(e);
  const bool host = attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeUnregistered;
  if (is_host) {
    *is_host = host ? 1 : 0;
  }
  *dev = attr.type == hipMemoryTypeUnregistered ? -1 : attr.device;
  return 0;
}

int tphip_mem_base(const void* ptr, void** base, size_t* size) {
  hipDeviceptr_t b = nullptr;
  size_t s = 0;
  TPHIP_TRY(hipMemGetAddressRange(&b, &s, const_cast<void*>(ptr)));
  if (base) {
    *base = b;
  }
  if (size) {
    *size = s;
  }
  return 0;
}

int tphip_mem_buffer_id(const void* ptr, uint64_t* id) {
  if (id == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  unsigned long long v = 0;
  hipError_t e = hipPointerGetAttribute(
      &v, HIP_POINTER_ATTRIBUTE_BUFFER_ID, reinterpret_cast<hipDeviceptr_t>(const_cast<void*>(ptr)));
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *id = 0;
    return 0;
  }
  *id = v;
  return 0;
}

int tphip_malloc(int dev, size_t bytes, void** ptr) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipMalloc(ptr, bytes));
  return 0;
}

int tphip_free(int dev, void* ptr) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipFree(ptr));
  return 0;
}

int tphip_host_alloc(int dev, size_t bytes, void** host_ptr, void** dev_ptr) {
  if (host_ptr == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipHostMalloc(host_ptr, bytes, hipHostMallocMapped | hipHostMallocPortable));
  if (dev_ptr != nullptr) {
    TPHIP_TRY(hipHostGetDevicePointer(dev_ptr, *host_ptr, 0));
  }
  return 0;
}

int tphip_host_free(void* host_ptr) {
  TPHIP_TRY(hipHostFree(host_ptr));
  return 0;
}

int tphip_stream_create(int dev, void** stream) {
  TPHIP_ON_DEVICE(dev);
  hipStream_t s;
  TPHIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return 0;
}

int tphip_stream_destroy(int dev, void* stream) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return 0;
}

int tphip_stream_sync(int dev, void* stream) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return 0;
}

int tphip_stream_query(int dev, void* stream, int* done) {
  TPHIP_ON_DEVICE(dev);
  hipError_t e = hipStreamQuery(static_cast<hipStream_t>(stream));
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    *done = 0;
    return 0;
  }
  TPHIP_TRY(e);
  *done = 1;
  return 0;
}

int tphip_event_create(int dev, int interprocess, void** event) {
  TPHIP_ON_DEVICE(dev);
  hipEvent_t e;
  unsigned flags = hipEventDisableTiming;
  if (interprocess) {
    flags |= hipEventInterprocess;
  }
  TPHIP_TRY(hipEventCreateWithFlags(&e, flags));
  *event = e;
  return 0;
}

int tphip_event_create_timed(int dev, void** event) {
  TPHIP_ON_DEVICE(dev);
  hipEvent_t e;
  TPHIP_TRY(hipEventCreate(&e));
  *event = e;
  return 0;
}

int tphip_event_destroy(int dev, void* event) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return 0;
}

int tphip_event_record(int dev, void* event, void* stream) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return 0;
}

int tphip_stream_wait_event(int dev, void* stream, void* event) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(
      hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
  return 0;
}

int tphip_event_query(int dev, void* event, int* done) {
  TPHIP_ON_DEVICE(dev);
  hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    *done = 0;
    return 0;
  }
  TPHIP_TRY(e);
  *done = 1;
  return 0;
}

int tphip_event_sync(int dev, void* event) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return 0;
}

int tphip_event_elapsed_ms(void* start, void* stop, float* ms) {
  TPHIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return 0;
}

int tphip_stream_on_complete(int dev, void* stream, tphip_host_fn fn, void* arg) {
  if (fn == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  HostFnThunk* t = new HostFnThunk{fn, arg};
  hipError_t e = hipStreamAddCallback(static_cast<hipStream_t>(stream), hostFnTrampoline, t, 0);
  if (e != hipSuccess) {
    delete t;
    return static_cast<int>(e);
  }
  return 0;
}

int tphip_ipc_mem_export(int dev, void* base, uint8_t out[TPHIP_IPC_HANDLE_BYTES]) {
  static_assert(sizeof(hipIpcMemHandle_t) == TPHIP_IPC_HANDLE_BYTES, "handle size");
  TPHIP_ON_DEVICE(dev);
  hipIpcMemHandle_t h;
  TPHIP_TRY(hipIpcGetMemHandle(&h, base));
  memcpy(out, &h, sizeof(h));
  return 0;
}

int tphip_ipc_mem_open(int dev, const uint8_t handle[TPHIP_IPC_HANDLE_BYTES], void** ptr) {
  TPHIP_ON_DEVICE(dev);
  hipIpcMemHandle_t h;
  memcpy(&h, handle, sizeof(h));
  TPHIP_TRY(hipIpcOpenMemHandle(ptr, h, hipIpcMemLazyEnablePeerAccess));
  return 0;
}

int tphip_ipc_mem_close(int dev, void* ptr) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipIpcCloseMemHandle(ptr));
  return 0;
}

int tphip_ipc_event_export(int dev, void* event, uint8_t out[TPHIP_IPC_HANDLE_BYTES]) {
  static_assert(sizeof(hipIpcEventHandle_t) == TPHIP_IPC_HANDLE_BYTES, "handle size");
  TPHIP_ON_DEVICE(dev);
  hipIpcEventHandle_t h;
  TPHIP_TRY(hipIpcGetEventHandle(&h, static_cast<hipEvent_t>(event)));
  memcpy(out, &h, sizeof(h));
  return 0;
}

int tphip_ipc_event_open(int dev, const uint8_t handle[TPHIP_IPC_HANDLE_BYTES], void** event) {
  TPHIP_ON_DEVICE(dev);
  hipIpcEventHandle_t h;
  memcpy(&h, handle, sizeof(h));
  hipEvent_t e;
  TPHIP_TRY(hipIpcOpenEventHandle(&e, h));
  *event = e;
  return 0;
}

int tphip_batched_copy(int dev, const tphip_copy_desc* table, uint32_t n, void* stream) {
  return batchedCopyImpl(dev, table, n, stream, 0, 0, -1);
}

int tphip_batched_copy_signal(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                              void* event, int unroll, uint32_t blocks, int nontemporal) {
  if (event == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  return batchedCopyImpl(dev, table, n, stream, unroll, blocks,
                         nontemporal < 0 ? -1 : (nontemporal & 3), static_cast<hipEvent_t>(event));
}

int tphip_batched_copy_noalloc(int dev, const tphip_copy_desc* table, uint32_t n, void* stream) {
  return noAllocCopy(dev, table, n, static_cast<hipStream_t>(stream));
}

int tphip_stream_signal(int dev, void* stream, void* word, uint64_t value) {
  if (word == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  return launchKernel(raise_signal_kernel, dim3(1), dim3(kWave), 0, static_cast<hipStream_t>(stream),
                      static_cast<uint64_t*>(word), value);
}

int tphip_agent_create(int dev, void** agent) {
  if (agent == nullptr || dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  auto a = std::make_unique<Agent>();
  a->dev = dev;
  int khz = 0;
  TPHIP_TRY(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
  if (khz <= 0) {
    khz = 100000;
  }
  const int idleUs = envInt("TPHIP_AGENT_IDLE_US", 50);
  const int lifeUs = envInt("TPHIP_AGENT_LIFE_US", 1000);
  a->idleTicks = static_cast<uint64_t>(idleUs > 0 ? idleUs : 1) * khz / 1000;
  a->lifeTicks = static_cast<uint64_t>(lifeUs > 0 ? lifeUs : 1) * khz / 1000;
  void* host = nullptr;
  const size_t bytes = sizeof(AgentCommand) * kAgentRing + sizeof(AgentControl);
  TPHIP_TRY(hipHostMalloc(&host, bytes, hipHostMallocMapped | hipHostMallocPortable));
  memset(host, 0, bytes);
  void* devp = nullptr;
  hipError_t e = hipHostGetDevicePointer(&devp, host, 0);
  if (e == hipSuccess) {
    e = hipStreamCreateWithFlags(&a->stream, hipStreamNonBlocking);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    (void)hipHostFree(host);
    return static_cast<int>(e);
  }
  a->ring = static_cast<AgentCommand*>(host);
  a->ringDev = static_cast<AgentCommand*>(devp);
  a->ctl = reinterpret_cast<AgentControl*>(a->ring + kAgentRing);
  a->ctlDev = reinterpret_cast<AgentControl*>(a->ringDev + kAgentRing);
  *agent = a.release();
  return 0;
}

int tphip_agent_submit(void* agent, const tphip_copy_desc* table, uint32_t n, void* notify,
                       uint64_t notify_value, uint64_t* ticket) {
  Agent* a = static_cast<Agent*>(agent);
  if (a == nullptr || table == nullptr || n == 0 || n > kAgentRing / 2 || ticket == nullptr ||
      notify_value > kAgentPayloadMask || reinterpret_cast<uintptr_t>(notify) > kAgentPayloadMask) {
    return TPHIP_ERR_INVALID_ARG;
  }
  uint32_t live = 0;
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].bytes == 0) {
      continue;
    }
    if (table[i].src == nullptr || table[i].dst == nullptr || table[i].bytes >= kAgentStopBytes ||
        reinterpret_cast<uintptr_t>(table[i].src) > kAgentPayloadMask ||
        reinterpret_cast<uintptr_t>(table[i].dst) > kAgentPayloadMask) {
      return TPHIP_ERR_INVALID_ARG;
    }
    ++live;
  }
  if (live == 0) {
    return TPHIP_ERR_INVALID_ARG;
  }
  std::lock_guard<std::mutex> lock(a->mutex);
  if (a->stopped) {
    return TPHIP_ERR_INVALID_ARG;
  }
  if (a->nextTicket + live - 1 - loadWord(&a->ctl->done) > kAgentRing) {
    return TPHIP_ERR_BUSY;
  }
  uint32_t k = 0;
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].bytes == 0) {
      continue;
    }
    ++k;
    const uint64_t t = a->nextTicket++;
    const uint64_t tag = (t & 0xffffu) << 48;
    AgentCommand& c = a->ring[t & (kAgentRing - 1)];
    const bool last = k == live;
    c.w[1] = reinterpret_cast<uintptr_t>(table[i].src) | tag;
    c.w[2] = reinterpret_cast<uintptr_t>(table[i].dst) | tag;
    c.w[3] = table[i].bytes | tag;
    c.w[4] = (last ? reinterpret_cast<uintptr_t>(notify) : 0) | tag;
    c.w[5] = (last ? notify_value : 0) | tag;
    __atomic_store_n(&c.w[0], t, __ATOMIC_RELEASE);
    *ticket = t;
  }
  TPHIP_ON_DEVICE(a->dev);
  return agentEnsureRunning(*a);
}

int tphip_agent_done(void* agent, uint64_t ticket, int* done) {
  Agent* a = static_cast<Agent*>(agent);
  if (a == nullptr || done == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  if (loadWord(&a->ctl->done) >= ticket) {
    *done = 1;
    return 0;
  }
  *done = 0;
  // An agent that left (idle, or its time was up) just before the command
  // was posted has not seen it: start the next one.
  const uint64_t epoch = a->epoch.load(std::memory_order_acquire);
  if (epoch != 0 && loadWord(&a->ctl->exited) == epoch) {
    std::lock_guard<std::mutex> lock(a->mutex);
    if (!a->stopped && loadWord(&a->ctl->done) < a->nextTicket - 1) {
      TPHIP_ON_DEVICE(a->dev);
      return agentEnsureRunning(*a);
    }
  }
  return 0;
}

int tphip_agent_destroy(void* agent) {
  Agent* a = static_cast<Agent*>(agent);
  if (a == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  int unserved = 0;
  {
    std::unique_lock<std::mutex> lock(a->mutex);
    a->stopped = true; // nothing is posted from here on
    // Everything posted so far is served first: the stop command needs a free
    // line of the ring (with the ring full it would land on the oldest
    // unserved command), and an agent that left just before the last command
    // was posted has to be started once more for it.
    DeviceScope scope(a->dev);
    const auto giveUpAt = std::chrono::steady_clock::now() + std::chrono::seconds(5);
    while (loadWord(&a->ctl->done) < a->nextTicket - 1) {
      if (agentEnsureRunning(*a) != 0 || std::chrono::steady_clock::now() > giveUpAt) {
        unserved = 1; // the GPU does not run the agent any more; say so below
        break;
      }
      lock.unlock();
      std::this_thread::yield();
      lock.lock();
    }
    const uint64_t epoch = a->epoch.load(std::memory_order_relaxed);
    if (unserved == 0 && epoch != 0 && loadWord(&a->ctl->exited) != epoch) {
      // A running agent leaves at this command.
      const uint64_t t = a->nextTicket++;
      const uint64_t tag = (t & 0xffffu) << 48;
      AgentCommand& c = a->ring[t & (kAgentRing - 1)];
      c.w[1] = tag;
      c.w[2] = tag;
      c.w[3] = kAgentStopBytes | tag;
      c.w[4] = tag;
      c.w[5] = tag;
      __atomic_store_n(&c.w[0], t, __ATOMIC_RELEASE);
    }
  }
  int rc = 0;
  {
    DeviceScope scope(a->dev);
    hipError_t e = hipStreamSynchronize(a->stream);
    if (e == hipSuccess) {
      e = hipStreamDestroy(a->stream);
    }
    if (e == hipSuccess) {
      e = hipHostFree(a->ring);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      rc = static_cast<int>(e);
    }
  }
  delete a;
  return rc != 0 ? rc : (unserved != 0 ? TPHIP_ERR_BUSY : 0);
}

int tphip_batched_copy_gated(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                             void* event, const void* gate_word, uint64_t gate_value,
                             uint32_t max_wait_us, void* expired_word) {
  if (event == nullptr || gate_word == nullptr || expired_word == nullptr || dev < 0 ||
      dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  GateDevice& gd = gGateDevices[dev];
  if (!gd.ready.load(std::memory_order_acquire)) {
    // A failed set-up is not remembered: the next call tries again.
    std::lock_guard<std::mutex> lock(gd.mutex);
    if (!gd.ready.load(std::memory_order_relaxed)) {
      int khz = 0;
      void* p = nullptr;
      hipError_t e = hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev);
      if (e == hipSuccess) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(gateStates));
      }
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
      }
      if (p == nullptr) {
        return TPHIP_ERR_INVALID_ARG;
      }
      gd.wallClockKhz = khz;
      gd.states = static_cast<uint64_t*>(p);
      gd.ready.store(true, std::memory_order_release);
    }
  }
  const int khz = gd.wallClockKhz > 0 ? gd.wallClockKhz : 100000;
  uint64_t* state = gd.states + gd.next.fetch_add(1, std::memory_order_relaxed) % kGateStates;
  int rc = launchKernel(gate_kernel, dim3(1), dim3(kWave), 0, static_cast<hipStream_t>(stream),
                        static_cast<const uint64_t*>(gate_word), gate_value,
                        static_cast<uint64_t>(max_wait_us) * khz / 1000,
                        static_cast<uint64_t*>(expired_word), state);
  if (rc != 0) {
    return rc;
  }
  struct Disarm {
    ~Disarm() {
      tlsGate = Gate{nullptr};
    }
  } disarm;
  tlsGate = Gate{state};
  return batchedCopyImpl(dev, table, n, stream, 0, 0, -1, static_cast<hipEvent_t>(event));
}

size_t tphip_ring_scratch_bytes(uint32_t num_slots) {
  return (offsetof(RingScratch, arrivals) + sizeof(uint32_t) * (num_slots > 0 ? num_slots : 1) + 255) / 256 * 256;
}

int tphip_ring_push(int dev, const tphip_ring_end* ring, const void* src, uint64_t bytes,
                    uint64_t first_seq, uint32_t yield_us, uint32_t blocks, void* stream, void* event) {
  return ringLaunch<true>(dev, ring, src, bytes, first_seq, yield_us, blocks, stream, event);
}

int tphip_ring_pull(int dev, const tphip_ring_end* ring, void* dst, uint64_t bytes,
                    uint64_t first_seq, uint32_t yield_us, uint32_t blocks, void* stream, void* event) {
  return ringLaunch<false>(dev, ring, dst, bytes, first_seq, yield_us, blocks, stream, event);
}

int tphip_copy(int dev, void* dst, const void* src, uint64_t bytes, void* stream) {
  tphip_copy_desc d{src, dst, bytes};
  return batchedCopyImpl(dev, &d, 1, stream, 0, 0, -1);
}

int tphip_batched_copy_tuned(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                             int unroll, uint32_t blocks, int nontemporal) {
  return batchedCopyImpl(dev, table, n, stream, unroll, blocks, nontemporal & 3);
}

int tphip_profile_start(int dev, uint32_t max_launches) {
  if (dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  DeviceState* st = nullptr;
  int rc = getDevice(dev, &st);
  if (rc != 0) {
    return rc;
  }
  std::lock_guard<std::mutex> lock(st->profMutex);
  for (auto& p : st->profEvents) {
    (void)hipEventDestroy(p.first);
    (void)hipEventDestroy(p.second);
  }
  st->profEvents.clear();
  st->profEvents.reserve(max_launches);
  // Events are created up front so that the measured region creates none.
  for (uint32_t i = 0; i < max_launches; ++i) {
    hipEvent_t begin = nullptr, end = nullptr;
    if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) {
      (void)hipGetLastError();
      break;
    }
    st->profEvents.emplace_back(begin, end);
  }
  st->profUsed = 0;
  st->profBytes = 0;
  st->profiling = true;
  return 0;
}

int tphip_profile_stop(int dev, uint32_t* launches, double* total_ms, uint64_t* total_bytes) {
  if (dev < 0 || dev >= kMaxDevices) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  DeviceState* st = nullptr;
  int rc = getDevice(dev, &st);
  if (rc != 0) {
    return rc;
  }
  std::lock_guard<std::mutex> lock(st->profMutex);
  st->profiling = false;
  double sum = 0;
  uint32_t count = 0;
  int err = 0;
  for (uint32_t i = 0; i < st->profEvents.size(); ++i) {
    auto& p = st->profEvents[i];
    if (i < st->profUsed) {
      hipError_t e = hipEventSynchronize(p.second);
      float ms = 0;
      if (e == hipSuccess) {
        e = hipEventElapsedTime(&ms, p.first, p.second);
      }
      if (e == hipSuccess) {
        sum += ms;
        ++count;
      } else {
        (void)hipGetLastError();
        err = static_cast<int>(e);
      }
    }
    (void)hipEventDestroy(p.first);
    (void)hipEventDestroy(p.second);
  }
  st->profUsed = 0;
  st->profEvents.clear();
  if (launches) {
    *launches = count;
  }
  if (total_ms) {
    *total_ms = sum;
  }
  if (total_bytes) {
    *total_bytes = st->profBytes;
  }
  return count > 0 ? 0 : err;
}

int tphip_bench_stream(int dev, int write, void* ptr, uint64_t bytes, void* stream) {
  if (ptr == nullptr || (reinterpret_cast<uintptr_t>(ptr) & 15u) != 0 || bytes < 16) {
    return TPHIP_ERR_INVALID_ARG;
  }
  TPHIP_ON_DEVICE(dev);
  DeviceState* st = nullptr;
  int rc = getDevice(dev, &st);
  if (rc != 0) {
    return rc;
  }
  const dim3 grid(static_cast<uint32_t>(st->numCus > 0 ? st->numCus : 256));
  ProfileScope prof(*st, static_cast<hipStream_t>(stream), bytes);
  if (write != 0) {
    return launchKernel(write_stream_kernel<8>, grid, dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream),
                        static_cast<char*>(ptr), bytes, 0x5bd1e995u);
  }
  // the sink is never written (see the kernel): the buffer itself will do
  return launchKernel(read_stream_kernel<8>, grid, dim3(kBlockThreads), 0, static_cast<hipStream_t>(stream),
                      static_cast<const char*>(ptr), bytes, static_cast<u32x4*>(ptr));
}

int tphip_memcpy_async(int dev, void* dst, const void* src, uint64_t bytes, void* stream) {
  TPHIP_ON_DEVICE(dev);
  TPHIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, static_cast<hipStream_t>(stream)));
  return 0;
}

int tphip_fill(int dev, void* ptr, int value, uint64_t bytes, void* stream) {
  if (bytes == 0) {
    return 0;
  }
  TPHIP_ON_DEVICE(dev);
  uint64_t blocks = (bytes + kBlockThreads - 1) / kBlockThreads;
  if (blocks > 2048) {
    blocks = 2048;
  }
  return launchKernel(fill_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlockThreads), 0,
                      static_cast<hipStream_t>(stream), static_cast<unsigned char*>(ptr),
                      static_cast<unsigned char>(value), bytes);
}

int tphip_test_set_table_limit(uint64_t vectors) {
  if (vectors > kMaxTableVectors) {
    return TPHIP_ERR_INVALID_ARG;
  }
  gTableLimit.store(vectors == 0 ? kMaxTableVectors : vectors, std::memory_order_relaxed);
  return 0;
}

int tphip_test_slow_kernel(int dev, void* ptr, uint64_t n, void* stream) {
  TPHIP_ON_DEVICE(dev);
  return launchKernel(slow_kernel, dim3(128), dim3(128), 0, static_cast<hipStream_t>(stream),
                      static_cast<volatile unsigned char*>(ptr), n);
}

} // extern "C"
