// Batched multi-tensor copy kernels for gfx950 (wave64).
//
// Work decomposition
// ------------------
// Every table entry {src, dst, bytes} is cut into
//   head : the 0..15 bytes before the first 16-byte aligned destination address
//   body : whole 16-byte vectors, destination aligned, source possibly not
//   tail : the 0..15 bytes left after the last whole vector
// The bodies of all entries are concatenated into one virtual sequence of
// vectors (an exclusive prefix sum over per-entry vector counts, computed on
// the host and shipped with the table). That sequence is cut into chunks of
// 256*U vectors; workgroup b of B takes chunks b, b+B, b+2B, ... and inside a
// chunk wavefront w takes the 64-vector pieces w, w+4, w+8, ... A piece that
// lies inside one entry is a plain coalesced 1 KiB load/store per wavefront,
// with the U loads of a lane issued before its U stores; a piece that
// straddles entries makes each lane look up the entry of its vector, so small
// tensors are packed lane-tight into wavefronts instead of costing a launch
// (or a wavefront) each. With one workgroup per CU the whole grid sweeps a
// compact window of memory at a time, which keeps HBM pages open; measured on
// MI355X this beats "many small slices per wavefront" by 10-15 %.
// Heads and tails are moved by the waves at the far end of the grid, sixteen
// lanes per entry (four entries per wavefront): lane k of an entry's sixteen
// owns byte k of its head and byte k of its tail, loads them ahead of the
// wave's chunks and stores them behind the first one. No lane needs to know
// about another entry, so nothing is scanned or searched across lanes.
//
// No LDS tiling is needed beyond the prefix array: the kernel is a pure HBM
// stream (2 bytes of traffic per payload byte), never touches MFMA.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "tphip.h"

namespace tphip {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
// Same vector, but the compiler may not assume any alignment: gfx950 global
// loads accept unaligned addresses, so this still becomes one dwordx4 load.
typedef u32x4 u32x4_unaligned __attribute__((aligned(1)));

constexpr int kWave = 64;
constexpr int kBlockThreads = 256;
constexpr int kWavesPerBlock = kBlockThreads / kWave;

// NT is a mask: bit 0 = nontemporal loads, bit 1 = nontemporal stores.
template <int NT>
__device__ __forceinline__ u32x4 load16(const char* p) {
  if (NT & 1) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_unaligned*>(p));
  }
  return *reinterpret_cast<const u32x4_unaligned*>(p);
}

template <int NT>
__device__ __forceinline__ void store16(char* p, u32x4 v) {
  if (NT & 2) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
  } else {
    *reinterpret_cast<u32x4*>(p) = v;
  }
}

__device__ __forceinline__ uint32_t head_bytes(const void* dst, uint64_t bytes) {
  uint64_t h = (0 - reinterpret_cast<uintptr_t>(dst)) & 15u;
  return static_cast<uint32_t>(h < bytes ? h : bytes);
}

__device__ __forceinline__ uint64_t shfl64(uint64_t v, int srcLane) {
  uint32_t lo = __shfl(static_cast<uint32_t>(v), srcLane);
  uint32_t hi = __shfl(static_cast<uint32_t>(v >> 32), srcLane);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// ---- signal words -----------------------------------------------------------
//
// 64-bit words in pinned host memory that both ends of a channel have mapped
// (their own page and, through an IPC handle, the peer's). A word is raised to
// a value once -- by a kernel in stream order, by a copy when it has finished,
// or by a CPU -- and read by kernels and CPUs of either process. They stand in
// for the inter-process events of the reference
// (tensorpipe/channel/cuda_ipc/channel_impl.cc:238-252,453-463): the GPU orders
// producer, copy and consumer by itself and the hosts only watch memory.

__device__ __forceinline__ uint64_t read_signal(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Everything this thread wrote before is visible to whoever sees the value.
__device__ __forceinline__ void raise_signal(uint64_t* p, uint64_t value) {
  __hip_atomic_store(p, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// A copy may be told to wait for a signal word before it touches its sources:
// the sender raises the word in stream order behind the work that produces the
// tensor (tphip_stream_signal) and announces the tensor at once; the receiver
// enqueues a gate kernel and, behind it on the same stream, the copy. The gate
// kernel is one wavefront that watches the word; the copy kernel is not
// resident meanwhile (256 workgroups polling a word in host memory while the
// producer still runs cost the producer two thirds of its bandwidth), it
// starts when the gate kernel has ended and first looks at the verdict the
// gate left in device memory. The wait is bounded: after `maxTicks` of the
// 100 MHz wall clock the gate gives up, says so in *expired (for the host) and
// in *state (for the copy, which then does nothing), and the host enqueues the
// pair again.
constexpr uint64_t kGateOpen = 1;
constexpr uint64_t kGateExpired = 2;

__global__ void gate_kernel(
    const uint64_t* word, uint64_t value, uint64_t maxTicks, uint64_t* expired, uint64_t* state) {
  if (threadIdx.x != 0) {
    return;
  }
  uint64_t verdict = kGateOpen;
  const uint64_t t0 = wall_clock64();
  while (read_signal(word) < value) {
    if (wall_clock64() - t0 > maxTicks) {
      verdict = kGateExpired;
      break;
    }
    __builtin_amdgcn_s_sleep(4);
  }
  if (verdict == kGateExpired) {
    raise_signal(expired, 1);
  }
  __hip_atomic_store(state, verdict, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

struct Gate {
  const uint64_t* state; // nullptr: no gate; else the verdict of the gate kernel ahead on the stream
};

__device__ __forceinline__ bool pass_gate(const Gate& g) {
  if (g.state == nullptr) {
    return true;
  }
  return __hip_atomic_load(g.state, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) == kGateOpen;
}

// Entries whose heads and tails one wavefront moves: sixteen lanes per entry,
// lane k of them owning byte k of the head and byte k of the tail (each at
// most 15 bytes long). No lane needs to know about another entry, so the
// wave spends a few LDS reads and two byte loads on it, nothing that depends
// on a neighbour. (Gathering the bytes of more entries densely over the lanes
// took a prefix scan and a search through cross-lane moves, about 1.5 us of
// dependent latencies on the waves that did it, and those waves finished last.)
constexpr uint32_t kEdgeGroup = kWave / 16;

// In two halves, so that the latency of the byte loads hides behind the
// wave's share of the bodies: edge_loads() before the chunk loop issues the
// loads and keeps value and destination per lane, edge_stores() after it
// writes them out. `entry(t, &src, &dst, &bytes)` yields entry t as the caller
// gave it.
struct EdgeBytes {
  char* dst[2]; // head byte, tail byte; nullptr: none held
  uint8_t val[2];
};

template <typename Entry>
__device__ __forceinline__ void edge_loads(
    Entry entry, uint32_t n, uint32_t group, uint32_t lane, EdgeBytes& held) {
  held.dst[0] = held.dst[1] = nullptr;
  held.val[0] = held.val[1] = 0;
  const uint32_t t = group * kEdgeGroup + (lane >> 4);
  const uint32_t k = lane & 15u;
  if (t >= n) {
    return;
  }
  uint64_t src = 0, dst = 0, bytes = 0;
  entry(t, &src, &dst, &bytes);
  const uint32_t head = head_bytes(reinterpret_cast<const void*>(dst), bytes);
  const uint32_t tail = static_cast<uint32_t>((bytes - head) & 15u);
  if (k < head) {
    held.val[0] = reinterpret_cast<const uint8_t*>(src)[k];
    held.dst[0] = reinterpret_cast<char*>(dst) + k;
  }
  if (k < tail) {
    const uint64_t off = bytes - tail + k;
    held.val[1] = reinterpret_cast<const uint8_t*>(src)[off];
    held.dst[1] = reinterpret_cast<char*>(dst) + off;
  }
}

__device__ __forceinline__ void edge_stores(const EdgeBytes& held) {
  if (held.dst[0] != nullptr) {
    __builtin_nontemporal_store(static_cast<char>(held.val[0]), held.dst[0]);
  }
  if (held.dst[1] != nullptr) {
    __builtin_nontemporal_store(static_cast<char>(held.val[1]), held.dst[1]);
  }
}

// One wavefront moves the heads and tails of entries
// [kEdgeGroup*group, kEdgeGroup*(group+1)).
template <typename Entry>
__device__ __forceinline__ void copy_edges(Entry entry, uint32_t n, uint32_t group, uint32_t lane) {
  EdgeBytes held;
  edge_loads(entry, n, group, lane, held);
  edge_stores(held);
}

// Where the 16-byte aligned body of an entry starts (src + head, dst + head),
// precomputed on the host.
struct CopyBody {
  const char* src;
  char* dst;
};

// Entries whose bodies are also kept in LDS (16 B each) next to the prefix;
// larger tables read them from global memory.
constexpr uint32_t kLdsBodies = 1024;

// Table variant. prefix[0..n] is the exclusive prefix sum of body vector
// counts (prefix[n] = total). Dynamic LDS: prefix padded to 16 B, then the
// bodies if n <= kLdsBodies. A chunk's lookup then costs LDS reads only; a
// dependent global load per chunk used to stall every workgroup for the best
// part of a microsecond.
// The work of a table copy once the plan is where the workgroup can read it
// cheaply: sPrefix (and normally body) in LDS, descs wherever they are.
template <int U, int NT, typename Entry>
__device__ __forceinline__ void table_copy(
    const uint32_t* sPrefix,
    const CopyBody* body,
    Entry entry,
    uint32_t n,
    uint32_t nchunks) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t waveInBlock = threadIdx.x >> 6;
  const uint32_t wave = blockIdx.x * kWavesPerBlock + waveInBlock;
  const uint32_t nwaves = gridDim.x * kWavesPerBlock;
  const uint32_t total = sPrefix[n];
  constexpr uint32_t kChunk = kBlockThreads * U;

  // Entry that holds vector `first` (largest index with prefix <= first),
  // searched from `from` onwards: a workgroup's chunks only move forward.
  auto locate = [&](uint32_t first, uint32_t from) -> uint32_t {
    uint32_t lo = from, hi = n;
    while (hi - lo > 1) {
      const uint32_t mid = (lo + hi) >> 1;
      if (sPrefix[mid] <= first) {
        lo = mid;
      } else {
        hi = mid;
      }
    }
    return __builtin_amdgcn_readfirstlane(lo);
  };

  // Where a chunk lives: entry, addresses of its first vector, vector count and
  // whether it lies inside one entry. Resolving costs a chain of dependent LDS
  // reads, so the NEXT chunk is resolved while the loads of the current one are
  // in flight (LDS and global memory have separate wait counters); only the
  // first resolve of a workgroup is exposed.
  struct Where {
    const char* s;
    char* d;
    uint32_t c0;
    uint32_t cnt;
    uint32_t t;
    bool inside;
  };
  auto resolve = [&](uint32_t c, uint32_t from) -> Where {
    Where w;
    w.c0 = c * kChunk;
    const uint32_t cEnd = total - w.c0 < kChunk ? total : w.c0 + kChunk;
    w.cnt = cEnd - w.c0;
    w.t = locate(w.c0, from);
    const uint32_t tBegin = sPrefix[w.t];
    w.inside = cEnd <= sPrefix[w.t + 1];
    const uint64_t off = static_cast<uint64_t>(w.c0 - tBegin) * 16;
    w.s = body[w.t].src + off;
    w.d = body[w.t].dst + off;
    return w;
  };

  // Heads and tails go to the waves at the far end of the grid, whose
  // workgroups run out of chunks first. The byte-wise gather is a chain of
  // dependent memory latencies: its loads are issued here, ahead of the wave's
  // chunks, and its stores follow them.
  const uint32_t edgeGroup = nwaves - 1 - wave;
  const bool hasEdges = edgeGroup * kEdgeGroup < n;
  EdgeBytes held;
  if (hasEdges) {
    edge_loads(entry, n, edgeGroup, lane, held);
  }
  bool edgesHeld = hasEdges;

  Where cur{};
  if (blockIdx.x < nchunks) {
    cur = resolve(blockIdx.x, 0);
  }
#pragma clang loop unroll(disable)
  for (uint32_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const uint32_t cNext = c + gridDim.x;
    Where nxt = cur;
    u32x4 v[U];
    if (cur.inside) {
      // Whole chunk inside one entry: uniform base, contiguous addresses.
      const char* s = cur.s;
      char* d = cur.d;
      const uint32_t cnt = cur.cnt;
      if (cnt == kChunk) {
#pragma unroll
        for (int j = 0; j < U; ++j) {
          v[j] = load16<NT>(s + (static_cast<size_t>(j) * kBlockThreads + threadIdx.x) * 16);
        }
        if (cNext < nchunks) {
          nxt = resolve(cNext, cur.t);
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
          store16<NT>(d + (static_cast<size_t>(j) * kBlockThreads + threadIdx.x) * 16, v[j]);
        }
      } else {
        // Partial chunk (cnt >= 1): out-of-range lanes re-read the last vector
        // so that all loads issue back to back; only stores are predicated.
#pragma unroll
        for (int j = 0; j < U; ++j) {
          const uint32_t idx = j * kBlockThreads + threadIdx.x;
          v[j] = load16<NT>(s + static_cast<size_t>(idx < cnt ? idx : cnt - 1) * 16);
        }
        if (cNext < nchunks) {
          nxt = resolve(cNext, cur.t);
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
          const uint32_t idx = j * kBlockThreads + threadIdx.x;
          if (idx < cnt) {
            store16<NT>(d + static_cast<size_t>(idx) * 16, v[j]);
          }
        }
      }
    } else {
      // Chunk straddles entries: per-lane lookup packs small tensors tightly.
      const uint32_t cnt = cur.cnt;
      char* dp[U];
#pragma unroll
      for (int j = 0; j < U; ++j) {
        const uint32_t idx = j * kBlockThreads + threadIdx.x;
        const uint32_t vv = cur.c0 + (idx < cnt ? idx : cnt - 1);
        uint32_t l = cur.t, h = n;
        while (h - l > 1) {
          const uint32_t m = (l + h) >> 1;
          if (sPrefix[m] <= vv) {
            l = m;
          } else {
            h = m;
          }
        }
        const uint64_t off = static_cast<uint64_t>(vv - sPrefix[l]) * 16;
        v[j] = load16<NT>(body[l].src + off);
        dp[j] = body[l].dst + off;
      }
      if (cNext < nchunks) {
        nxt = resolve(cNext, cur.t);
      }
#pragma unroll
      for (int j = 0; j < U; ++j) {
        if (j * kBlockThreads + threadIdx.x < cnt) {
          store16<NT>(dp[j], v[j]);
        }
      }
    }
    cur = nxt;
    if (edgesHeld) {
      // Right behind the wave's first chunk: the loads have long returned, and
      // the partly written lines leave the L2 while the copy is still running
      // rather than in the write-back at the end of the kernel.
      edge_stores(held);
      edgesHeld = false;
    }
  }

  if (hasEdges) {
    if (edgesHeld) {
      edge_stores(held);
    }
    // Tables with more groups than the grid has waves: the rest, one by one.
    for (uint32_t g = edgeGroup + nwaves; g * kEdgeGroup < n; g += nwaves) {
      copy_edges(entry, n, g, lane);
    }
  }
}

template <int U, int NT>
__global__ __launch_bounds__(kBlockThreads) void batched_copy_kernel(
    const uint32_t* __restrict__ prefix,
    const CopyBody* __restrict__ bodies,
    const tphip_copy_desc* __restrict__ descs,
    uint32_t n,
    uint32_t nchunks,
    const Gate gate) {
  extern __shared__ __align__(16) uint32_t sPrefix[];
  if (!pass_gate(gate)) {
    return;
  }
  const bool cached = n <= kLdsBodies;
  CopyBody* sBodies = reinterpret_cast<CopyBody*>(sPrefix + ((n + 1 + 3) & ~3u));
  // Four loads per thread in flight before the first LDS write: a pass that
  // waits for every load before issuing the next costs a memory latency per
  // 256 entries, and every workgroup pays it before its first chunk.
  constexpr int kBatch = 4;
  for (uint32_t base = 0; base <= n; base += kBatch * kBlockThreads) {
    uint32_t w[kBatch];
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      const uint32_t i = base + k * kBlockThreads + threadIdx.x;
      w[k] = i <= n ? prefix[i] : 0u;
    }
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      const uint32_t i = base + k * kBlockThreads + threadIdx.x;
      if (i <= n) {
        sPrefix[i] = w[k];
      }
    }
  }
  if (cached) {
    const u32x4* in = reinterpret_cast<const u32x4*>(bodies);
    u32x4* out = reinterpret_cast<u32x4*>(sBodies);
    for (uint32_t base = 0; base < n; base += kBatch * kBlockThreads) {
      u32x4 w[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const uint32_t i = base + k * kBlockThreads + threadIdx.x;
        w[k] = in[i < n ? i : n - 1];
      }
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const uint32_t i = base + k * kBlockThreads + threadIdx.x;
        if (i < n) {
          out[i] = w[k];
        }
      }
    }
  }
  __syncthreads();
  table_copy<U, NT>(
      sPrefix,
      cached ? sBodies : bodies,
      [descs](uint32_t t, uint64_t* src, uint64_t* dst, uint64_t* bytes) {
        *src = reinterpret_cast<uint64_t>(descs[t].src);
        *dst = reinterpret_cast<uint64_t>(descs[t].dst);
        *bytes = descs[t].bytes;
      },
      n,
      nchunks);
}

// Small tables travel in the kernel arguments: no plan upload, no staging
// kernel, nothing to recycle afterwards -- one launch is the whole cost (the
// runtime writes kernel arguments into device memory, 5.4 KiB of them for 256
// entries cost about a microsecond more per launch call than a few bytes).
// What travels is what the workgroups keep in LDS anyway: the prefix sums, the
// bodies, and one byte per entry holding how many bytes precede and follow the
// body (4 bits each), from which the wave that moves heads and tails rebuilds
// the entry as the caller gave it. Two sizes, so that a two-tensor message
// does not pay for 256 entries.
constexpr uint32_t kInlineEntries = 256;
constexpr uint32_t kInlineEntriesSmall = 64;

template <uint32_t N>
struct InlinePlanT {
  uint32_t n;
  uint32_t nchunks;
  uint32_t prefix[N + 2]; // n+1 used; padded to keep 8-byte alignment below
  CopyBody bodies[N];
  uint8_t edges[N]; // head << 4 | tail
};
static_assert(sizeof(InlinePlanT<kInlineEntries>) % 4 == 0, "copied word by word");
static_assert(sizeof(InlinePlanT<kInlineEntriesSmall>) % 4 == 0, "copied word by word");
static_assert(sizeof(InlinePlanT<kInlineEntries>) <= 6144, "kernel argument budget");

template <int U, int NT, uint32_t N>
__global__ __launch_bounds__(kBlockThreads) void inline_copy_kernel(
    const InlinePlanT<N> plan, const Gate gate) {
  __shared__ __align__(16) InlinePlanT<N> sPlan;
  if (!pass_gate(gate)) {
    return;
  }
  // Only what n entries use: header + prefix, bodies, edge bytes. All loads
  // of a thread are issued before its first LDS write, so the fill costs one
  // memory latency, not one per pass.
  const uint32_t n = plan.n;
  const uint32_t* in = reinterpret_cast<const uint32_t*>(&plan);
  uint32_t* out = reinterpret_cast<uint32_t*>(&sPlan);
  constexpr uint32_t kBodiesAt = offsetof(InlinePlanT<N>, bodies) / 4;
  constexpr uint32_t kEdgesAt = offsetof(InlinePlanT<N>, edges) / 4;
  constexpr uint32_t kWords = sizeof(InlinePlanT<N>) / 4;
  constexpr int kPerThread = (kWords + kBlockThreads - 1) / kBlockThreads;
  uint32_t word[kPerThread];
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const uint32_t i = k * kBlockThreads + threadIdx.x;
    const bool used = i < 2 + n + 1 || (i >= kBodiesAt && i < kBodiesAt + n * 4) ||
        (i >= kEdgesAt && i < kEdgesAt + (n + 3) / 4);
    word[k] = used ? in[i] : 0u;
  }
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const uint32_t i = k * kBlockThreads + threadIdx.x;
    if (i < kWords) {
      out[i] = word[k];
    }
  }
  __syncthreads();
  const InlinePlanT<N>* p = &sPlan;
  table_copy<U, NT>(
      sPlan.prefix,
      sPlan.bodies,
      [p](uint32_t t, uint64_t* src, uint64_t* dst, uint64_t* bytes) {
        const uint32_t head = p->edges[t] >> 4;
        const uint32_t tail = p->edges[t] & 15u;
        *src = reinterpret_cast<uint64_t>(p->bodies[t].src) - head;
        *dst = reinterpret_cast<uint64_t>(p->bodies[t].dst) - head;
        *bytes = head + (static_cast<uint64_t>(p->prefix[t + 1] - p->prefix[t]) << 4) + tail;
      },
      n,
      sPlan.nchunks);
}

// Single-entry variant: the descriptor travels in the kernel arguments, no
// table upload, no LDS, 64-bit vector counts (any size). Lane g of the G lanes
// of the grid copies vectors g, g+G, g+2G, ... U at a time: the grid sweeps
// one contiguous G*U*16-byte window per iteration.
template <int U, int NT>
__global__ __launch_bounds__(kBlockThreads) void single_copy_kernel(
    const char* __restrict__ src, char* __restrict__ dst, uint64_t bytes, const Gate gate) {
  if (!pass_gate(gate)) {
    return;
  }
  const uint64_t g = static_cast<uint64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
  const uint64_t G = static_cast<uint64_t>(gridDim.x) * kBlockThreads;
  const uint32_t head = head_bytes(dst, bytes);
  const uint64_t nvec = (bytes - head) >> 4;
  const uint32_t tail = static_cast<uint32_t>((bytes - head) & 15u);

  if (g < 64) {
    const uint32_t lane = static_cast<uint32_t>(g);
    if (lane < head) {
      dst[lane] = src[lane];
    } else if (lane >= 16 && lane - 16 < tail) {
      const uint64_t o = bytes - tail + (lane - 16);
      dst[o] = src[o];
    }
  }
  const char* s = src + head;
  char* d = dst + head;
  const uint64_t step = G * U;
  const uint64_t full = nvec / step * step;
#pragma clang loop unroll(disable)
  for (uint64_t base = 0; base < full; base += step) {
    u32x4 v[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      v[j] = load16<NT>(s + (base + j * G + g) * 16);
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      store16<NT>(d + (base + j * G + g) * 16, v[j]);
    }
  }
#pragma clang loop unroll(disable)
  for (uint64_t i = full + g; i < nvec; i += G) {
    store16<NT>(d + i * 16, load16<NT>(s + i * 16));
  }
}

// Stages the host-written (pinned, device-mapped) plan into device memory so
// that the copy kernel's table reads hit L2/HBM instead of the host link.
__global__ __launch_bounds__(kBlockThreads) void stage_plan_kernel(
    const u32x4* __restrict__ hostPlan, u32x4* __restrict__ devPlan, uint32_t nvec) {
  for (uint32_t i = blockIdx.x * kBlockThreads + threadIdx.x; i < nvec;
       i += gridDim.x * kBlockThreads) {
    devPlan[i] = hostPlan[i];
  }
}

// Raises a word in stream order: enqueued behind the work that produces a
// tensor, it tells the peer's copy that the bytes are there.
__global__ void raise_signal_kernel(uint64_t* word, uint64_t value) {
  if (threadIdx.x == 0) {
    raise_signal(word, value);
  }
}

// K vectors per lane in flight over as many whole K * THREADS blocks as are
// left from vector `done` on; returns the first vector not yet copied.
template <uint32_t THREADS, int K>
__device__ __forceinline__ uint64_t team_sweep(
    const char* s, char* d, uint64_t done, uint64_t nvec, uint32_t tid) {
  constexpr uint64_t kStep = static_cast<uint64_t>(K) * THREADS;
  const uint64_t end = done + (nvec - done) / kStep * kStep;
#pragma clang loop unroll(disable)
  for (uint64_t base = done; base < end; base += kStep) {
    u32x4 v[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
      v[j] = load16<0>(s + (base + j * THREADS + tid) * 16);
    }
#pragma unroll
    for (int j = 0; j < K; ++j) {
      store16<0>(d + (base + j * THREADS + tid) * 16, v[j]);
    }
  }
  return end;
}

// THREADS lanes (a workgroup, or one wavefront of it) copy `bytes` bytes, any
// alignment: the same head / body / tail split as the grid-wide kernels.
template <uint32_t THREADS>
__device__ __forceinline__ void team_copy(const char* src, char* dst, uint64_t bytes, uint32_t tid) {
  const uint32_t head = head_bytes(dst, bytes);
  const uint64_t nvec = (bytes - head) >> 4;
  const uint32_t tail = static_cast<uint32_t>((bytes - head) & 15u);
  if (tid < head) {
    dst[tid] = src[tid];
  } else if (tid >= 16 && tid - 16 < tail) {
    const uint64_t o = bytes - tail + (tid - 16);
    dst[o] = src[o];
  }
  const char* s = src + head;
  char* d = dst + head;
  // A team this small is bound by memory latency, not bandwidth: sixteen
  // vectors per lane in flight while whole blocks of that size are left (one
  // wavefront: 16 KiB per round trip to memory), then four, then one.
  uint64_t done = team_sweep<THREADS, 16>(s, d, 0, nvec, tid);
  done = team_sweep<THREADS, 4>(s, d, done, nvec, tid);
  done = team_sweep<THREADS, 1>(s, d, done, nvec, tid);
  if (done + tid < nvec) {
    store16<0>(d + (done + tid) * 16, load16<0>(s + (done + tid) * 16));
  }
}

// ---- resident copy agent ------------------------------------------------------
//
// A launch costs about 7 us from the call to the host seeing the end of a
// 4 KiB copy; a workgroup that is already running and watches a command ring
// in pinned host memory does the same copy 2.5-3.5 us after the host wrote the
// command. The agent is that workgroup: started when small transfers arrive,
// it serves them while they keep coming and leaves by itself when nothing has
// come for `idleTicks` of the 100 MHz wall clock, when `lifeTicks` have passed
// since it started (so that no queue it may share with other work is held for
// long), or on a stop command. The host starts it again when needed.
//
// A command is one 64-byte line written by the host: word 0 is its ticket
// (tickets count up from 1), words 1-5 carry 48 bits of payload each under the
// low 16 bits of the ticket as a tag in the top bits. The line may reach the
// GPU in pieces, so a command counts as arrived only when ticket and all tags
// agree -- no second round trip over the host link to re-read it.
struct AgentCommand {
  uint64_t w[8]; // ticket, src, dst, bytes, notify address, notify value, -, -
};
constexpr uint64_t kAgentPayloadMask = (1ull << 48) - 1;
constexpr uint64_t kAgentStopBytes = kAgentPayloadMask; // "bytes" of the stop command

struct AgentControl {
  uint64_t done; // last ticket served (raised by the agent)
  uint64_t exited; // epoch of the last agent that has left (raised by the agent)
  uint64_t pad[6];
};

__global__ __launch_bounds__(kWave) void agent_kernel(
    const AgentCommand* __restrict__ ring,
    uint32_t ringMask,
    AgentControl* __restrict__ ctl,
    uint64_t ticket,
    uint64_t epoch,
    uint64_t idleTicks,
    uint64_t lifeTicks) {
  // One wavefront: nothing to synchronise between finding a command, copying
  // and reporting, and 64 lanes move the few KiB a command carries in a
  // microsecond.
  const uint32_t lane = threadIdx.x;
  const uint64_t born = wall_clock64();
  uint64_t lastWork = born;
  for (;;) {
    const AgentCommand* slot = ring + (ticket & ringMask);
    const uint64_t tag = ticket & 0xffffu;
    uint64_t w = 0;
    bool leave = false;
    for (;;) {
      if (lane < 6) {
        w = read_signal(&slot->w[lane]);
      }
      const bool ok = lane == 0 ? w == ticket : (lane < 6 ? (w >> 48) == tag : true);
      if (__ballot(ok) == ~0ull) {
        break;
      }
      const uint64_t now = wall_clock64();
      if (now - lastWork > idleTicks || now - born > lifeTicks) {
        leave = true;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (leave) {
      break;
    }
    const uint64_t src = shfl64(w, 1) & kAgentPayloadMask;
    const uint64_t dst = shfl64(w, 2) & kAgentPayloadMask;
    const uint64_t bytes = shfl64(w, 3) & kAgentPayloadMask;
    const uint64_t notify = shfl64(w, 4) & kAgentPayloadMask;
    const uint64_t notifyValue = shfl64(w, 5) & kAgentPayloadMask;
    const bool stop = bytes == kAgentStopBytes;
    if (!stop) {
      // What other kernels (of this or the peer process) wrote since the last
      // command must not be served from this CU's caches.
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
      team_copy<kWave>(reinterpret_cast<const char*>(src), reinterpret_cast<char*>(dst), bytes, lane);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    }
    if (lane == 0) {
      if (notify != 0) {
        raise_signal(reinterpret_cast<uint64_t*>(notify), notifyValue);
      }
      raise_signal(&ctl->done, ticket);
    }
    if (stop) {
      break;
    }
    ++ticket;
    lastWork = wall_clock64();
  }
  if (lane == 0) {
    raise_signal(&ctl->exited, epoch);
  }
}


// ---- GPU-driven staging ring ---------------------------------------------------
//
// The host-staged channel moves a tensor through a ring of pinned host slots
// (tensorpipe/channel/cuda_basic/channel_impl.cc:117-229 send, :380-506 recv:
// one copy, one stream callback and two control messages per chunk). Here one
// kernel per tensor and side walks the ring by itself: the pushing kernel
// copies chunk after chunk from the source into slot (sequence % slots) and
// raises `produced`, the pulling kernel of the other process waits for
// `produced`, copies slot -> destination and raises `consumed`, which is what
// the pusher waits for before it overwrites a slot. Chunks are numbered over
// the life of the ring, so the two counters only ever grow. The slots and the
// two counters are pinned host memory that both processes' GPUs have mapped
// (plain loads and stores only: nothing relies on atomics across the host
// link, nor on two processes seeing each other's device memory mid-kernel).
//
// The workgroups form `groups` teams; team t copies chunks t, t + groups, ...
// so that while one team sits at a chunk boundary (its stores draining, the
// counter of the other side being read) the others keep the link busy. Every
// workgroup of a team copies its share of the team's chunk. A chunk is complete
// when the whole team has arrived at its slot's counter (device memory of this
// side); the last one to arrive resets that counter, waits until the chunk
// before has been published (the last arrivals of two consecutive chunks may
// be different workgroups, and the shared word must never step back) and
// raises the shared word.
//
// No wait is unbounded, and no kernel relies on another kernel of its own
// process running at the same time (two streams may share one hardware queue):
// a workgroup that sees no progress for `yieldTicks` of the 100 MHz wall
// clock, or finds `*abort` raised by the host, sets the launch's stop flag and
// everybody leaves at their next wait. The last workgroup to leave tells the
// host (`status`, pinned memory) how many chunks are complete and whether the
// kernel gave up (kRingYielded), and leaves the scratch words as the next
// launch needs them (a chunk may have been half arrived); the host launches
// again from there, behind whatever else it has queued meanwhile.
constexpr uint64_t kRingYielded = 1ull << 63;

// This side's own words in device memory, all zero before the first launch.
struct RingScratch {
  uint64_t published; // chunks complete on this side (ring sequence)
  uint32_t stop;      // raised by the workgroup that gave up
  uint32_t exits;     // workgroups that have left
  uint32_t arrivals[1]; // numSlots of them
};

struct RingArgs {
  char* user;          // source (push) or destination (pull) of this launch's first chunk
  uint64_t bytes;      // bytes this launch moves (whole chunks but the last)
  char* slots;         // slot 0 of the ring
  uint64_t slotBytes;
  uint32_t numSlots;
  uint64_t firstSeq;   // ring sequence number of this launch's first chunk
  uint64_t* produced;  // shared, host memory
  uint64_t* consumed;  // shared, host memory
  RingScratch* scratch;
  uint64_t* status;    // host-visible: chunks complete (ring sequence) | kRingYielded
  const uint64_t* abort; // host-written; non-zero: leave
  uint64_t yieldTicks;
  uint32_t groups;     // teams of workgroups; gridDim.x is a multiple of it
};

template <bool PUSH, int U>
__global__ __launch_bounds__(kBlockThreads) void ring_kernel(const RingArgs a) {
  __shared__ uint32_t sGo;
  const uint32_t team = blockIdx.x % a.groups;
  const uint32_t teamBlocks = gridDim.x / a.groups;
  const uint64_t g = static_cast<uint64_t>(blockIdx.x / a.groups) * kBlockThreads + threadIdx.x;
  const uint64_t G = static_cast<uint64_t>(teamBlocks) * kBlockThreads;
  const uint64_t nChunks = (a.bytes + a.slotBytes - 1) / a.slotBytes;
  RingScratch* sc = a.scratch;
  if (threadIdx.x == 0) {
    sGo = 1; // a team without a chunk leaves as "not stopped"
  }
  // What thread 0 last read of the other side's counter: the counter only
  // grows, so a value that is enough needs no second look (a look costs a
  // round trip that queues behind the copy's own traffic).
  uint64_t seen = 0;
  const uint64_t* awaited = PUSH ? a.consumed : a.produced;
  uint64_t* raised = PUSH ? a.produced : a.consumed;

  for (uint64_t k = team; k < nChunks; k += a.groups) {
    const uint64_t seq = a.firstSeq + k;
    const uint32_t slot = static_cast<uint32_t>(seq % a.numSlots);
    if (threadIdx.x == 0) {
      // push: the chunk that used this slot last has been read out;
      // pull: this chunk has been written.
      const uint64_t need = PUSH ? (seq >= a.numSlots ? seq - a.numSlots + 1 : 0) : seq + 1;
      uint32_t go = 1;
      if (seen < need) {
        const uint64_t t0 = wall_clock64();
        for (uint32_t spins = 0;; ++spins) {
          seen = read_signal(awaited);
          if (seen >= need) {
            break;
          }
          if (__hip_atomic_load(&sc->stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
            go = 0;
            break;
          }
          if (wall_clock64() - t0 > a.yieldTicks || ((spins & 63u) == 63u && read_signal(a.abort) != 0)) {
            __hip_atomic_store(&sc->stop, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            go = 0;
            break;
          }
          // about a microsecond: every look may be a read across the host link
          __builtin_amdgcn_s_sleep(32);
        }
      }
      sGo = go;
    }
    __syncthreads();
    if (sGo == 0) {
      break;
    }
    // Nothing the other side wrote may be served from this CU's caches.
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");

    const uint64_t off = k * a.slotBytes;
    const uint64_t len = a.bytes - off < a.slotBytes ? a.bytes - off : a.slotBytes;
    const char* src = PUSH ? a.user + off : a.slots + static_cast<uint64_t>(slot) * a.slotBytes;
    char* dst = PUSH ? a.slots + static_cast<uint64_t>(slot) * a.slotBytes : a.user + off;
    {
      // The grid-wide single-entry copy: destination-aligned 16-byte vectors,
      // lane g of G takes vectors g, g+G, ... U at a time; device memory is
      // streamed past the caches, the host side is uncached anyway.
      constexpr int NT = 3;
      const uint32_t head = head_bytes(dst, len);
      const uint64_t nvec = (len - head) >> 4;
      const uint32_t tail = static_cast<uint32_t>((len - head) & 15u);
      if (g < 64) {
        const uint32_t lane = static_cast<uint32_t>(g);
        if (lane < head) {
          dst[lane] = src[lane];
        } else if (lane >= 16 && lane - 16 < tail) {
          const uint64_t o = len - tail + (lane - 16);
          dst[o] = src[o];
        }
      }
      const char* s = src + head;
      char* d = dst + head;
      const uint64_t step = G * U;
      const uint64_t full = nvec / step * step;
#pragma clang loop unroll(disable)
      for (uint64_t base = 0; base < full; base += step) {
        u32x4 v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
          v[j] = load16<NT>(s + (base + j * G + g) * 16);
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
          store16<NT>(d + (base + j * G + g) * 16, v[j]);
        }
      }
#pragma clang loop unroll(disable)
      for (uint64_t i = full + g; i < nvec; i += G) {
        store16<NT>(d + i * 16, load16<NT>(s + i * 16));
      }
    }
    // Before the workgroup arrives: a pushing thread's stores have been taken
    // by the host's memory (the slots are uncached host memory: a store is
    // counted done when it is, there is nothing of it in a cache to write
    // back); a pulling thread's loads have returned, which its stores already
    // waited for -- what it wrote to the destination is nobody's business
    // before the kernel ends.
    if (PUSH) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      const uint32_t before =
          __hip_atomic_fetch_add(&sc->arrivals[slot], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      if (before == teamBlocks - 1) {
        // (The slot's next chunk cannot arrive before the word below has been
        // raised and answered by the other side.)
        __hip_atomic_store(&sc->arrivals[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // In order: the chunk before belongs to another team; its word is
        // on its way at the latest -- unless its team gave up, in which case
        // this chunk stays unpublished as well and is copied again later.
        bool inOrder = true;
        while (__hip_atomic_load(&sc->published, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < seq) {
          if (__hip_atomic_load(&sc->stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
            inOrder = false;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        if (inOrder) {
          raise_signal(raised, seq + 1);
          __hip_atomic_store(&sc->published, seq + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }
  if (threadIdx.x == 0) {
    const uint32_t before =
        __hip_atomic_fetch_add(&sc->exits, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    if (before == gridDim.x - 1) {
      // Last one out: everybody else has left, the scratch words are ours.
      const uint32_t yielded = __hip_atomic_load(&sc->stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint64_t done = __hip_atomic_load(&sc->published, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
      for (uint32_t i = 0; i < a.numSlots; ++i) {
        __hip_atomic_store(&sc->arrivals[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __hip_atomic_store(&sc->stop, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&sc->exits, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
      raise_signal(a.status, done | (yielded != 0 ? kRingYielded : 0));
    }
  }
}

// One-directional streams, for measurement only: what HBM gives a kernel that
// only reads, or only writes, with the access pattern of the copy kernels
// (lane g of G touches vectors g, g+G, ... U at a time, nontemporal). A copy
// moves one byte each way, so its rate is bounded by the mix of the two.
template <int U>
__global__ __launch_bounds__(kBlockThreads) void read_stream_kernel(
    const char* __restrict__ src, uint64_t bytes, u32x4* __restrict__ sink) {
  const uint64_t g = static_cast<uint64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
  const uint64_t G = static_cast<uint64_t>(gridDim.x) * kBlockThreads;
  const uint64_t nvec = bytes >> 4;
  const uint64_t step = G * U;
  const uint64_t full = nvec / step * step;
  u32x4 acc = {0, 0, 0, 0};
#pragma clang loop unroll(disable)
  for (uint64_t base = 0; base < full; base += step) {
    u32x4 v[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      v[j] = load16<1>(src + (base + j * G + g) * 16);
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      acc ^= v[j];
    }
  }
  for (uint64_t i = full + g; i < nvec; i += G) {
    acc ^= load16<1>(src + i * 16);
  }
  // Keeps the loads alive; random data never produces this value in every lane.
  if (acc.x == 0x9e3779b9u && acc.y == 0x7f4a7c15u && acc.z == 0xf39cc060u && acc.w == 0x5cedc834u) {
    sink[0] = acc;
  }
}

template <int U>
__global__ __launch_bounds__(kBlockThreads) void write_stream_kernel(char* __restrict__ dst, uint64_t bytes, uint32_t seed) {
  const uint64_t g = static_cast<uint64_t>(blockIdx.x) * kBlockThreads + threadIdx.x;
  const uint64_t G = static_cast<uint64_t>(gridDim.x) * kBlockThreads;
  const uint64_t nvec = bytes >> 4;
  const uint64_t step = G * U;
  const uint64_t full = nvec / step * step;
  const u32x4 v = {seed, static_cast<uint32_t>(g), seed ^ 0xa5a5a5a5u, static_cast<uint32_t>(g >> 32)};
#pragma clang loop unroll(disable)
  for (uint64_t base = 0; base < full; base += step) {
#pragma unroll
    for (int j = 0; j < U; ++j) {
      store16<2>(dst + (base + j * G + g) * 16, v);
    }
  }
  for (uint64_t i = full + g; i < nvec; i += G) {
    store16<2>(dst + i * 16, v);
  }
}

// A piece of a plan carried in the kernel arguments, written to device memory
// at `byteOffset` of `dst` by one workgroup. Lets a caller that may not touch
// pinned host memory or the copy engines put a plan of any size into device
// memory with nothing but kernel launches.
constexpr uint32_t kPlanPieceWords = 896;
struct PlanPiece {
  uint32_t words; // used entries of data[]
  uint32_t byteOffset; // multiple of 4
  uint32_t data[kPlanPieceWords];
};
static_assert(sizeof(PlanPiece) <= 3600, "kernel argument budget");

__global__ __launch_bounds__(kBlockThreads) void write_plan_piece_kernel(
    const PlanPiece piece, char* __restrict__ dst) {
  uint32_t* out = reinterpret_cast<uint32_t*>(dst + piece.byteOffset);
  for (uint32_t i = threadIdx.x; i < piece.words; i += kBlockThreads) {
    out[i] = piece.data[i];
  }
}

__global__ __launch_bounds__(kBlockThreads) void fill_kernel(
    unsigned char* __restrict__ p, unsigned char value, uint64_t n) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * kBlockThreads;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < n;
       i += stride) {
    p[i] = value;
  }
}

// Long dependent chain of byte updates per element; bounded, always exits.
__global__ __launch_bounds__(128) void slow_kernel(volatile unsigned char* p, uint64_t n) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    unsigned char x = p[i];
    for (int k = 0; k < 100000; ++k) {
      x = static_cast<unsigned char>(x * 5u + 1u);
      p[i] = x;
      __builtin_amdgcn_s_sleep(1);
    }
  }
}

} // namespace tphip
