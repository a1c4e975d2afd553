// ref_pipe_bench.cc -- TEST / BASELINE INFRASTRUCTURE ONLY.
//
// Ping-pong over the GENUINE reference: the TensorPipe that PyTorch's wheel
// carries prebuilt in libtorch_cpu.so (core + shm transport + basic channel),
// driven through its public headers in torch/include/tensorpipe. Nothing of
// the reference is copied or rebuilt; this file only calls its API the way
// tensorpipe/benchmark/benchmark_pipe.cc:422-636 does (two processes, the
// client times write -> echoed read, percentiles as measurements.h:51-53).
// Built by oracle/Makefile into oracle/_ref/ when the wheel's headers are
// present; the bench reports its figures as the reference CPU baseline and
// falls back to the port (cpu_shm_basic.c) when it is absent.
//
// Usage: ref_pipe_bench <tensor_bytes> <payload_bytes> <warmup> <iters>
#include <tensorpipe/tensorpipe.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <future>
#include <string>
#include <vector>

#include <sys/wait.h>
#include <unistd.h>

using namespace tensorpipe;

static std::shared_ptr<Context> makeContext(const char* name) {
  auto ctx = std::make_shared<Context>(ContextOptions().name(name));
  ctx->registerTransport(0, "shm", transport::shm::create());
  ctx->registerChannel(0, "basic", channel::basic::create());
  return ctx;
}

struct Buffers {
  std::vector<uint8_t> tensor, payload;
};

static Message makeMessage(Buffers& b) {
  Message m;
  if (!b.payload.empty()) {
    Message::Payload p;
    p.data = b.payload.data();
    p.length = b.payload.size();
    m.payloads.push_back(std::move(p));
  }
  Message::Tensor t;
  t.buffer = CpuBuffer{b.tensor.data()};
  t.length = b.tensor.size();
  m.tensors.push_back(std::move(t));
  return m;
}

// Everything below is callback-chained on the library's own threads, as in
// benchmark_pipe.cc: no thread hand-off is on the clock.

// Reads one message into `into`, then calls next(ok).
static void readOne(Pipe& pipe, Buffers& into, std::function<void(bool)> next) {
  pipe.readDescriptor([&pipe, &into, next](const Error& error, Descriptor d) {
    if (error) {
      fprintf(stderr, "readDescriptor: %s\n", error.what().c_str());
      next(false);
      return;
    }
    Allocation a;
    a.payloads.resize(d.payloads.size());
    for (size_t i = 0; i < d.payloads.size(); ++i) {
      a.payloads[i].data = into.payload.data();
    }
    a.tensors.resize(d.tensors.size());
    for (size_t i = 0; i < d.tensors.size(); ++i) {
      a.tensors[i].buffer = CpuBuffer{into.tensor.data()};
    }
    pipe.read(std::move(a), [next](const Error& e2) {
      if (e2) {
        fprintf(stderr, "read: %s\n", e2.what().c_str());
      }
      next(!e2);
    });
  });
}

struct Server {
  std::shared_ptr<Pipe> pipe;
  Buffers buffers;
  int remaining{0};
  std::promise<bool> finished;

  void step() {
    if (remaining == 0) {
      finished.set_value(true);
      return;
    }
    --remaining;
    readOne(*pipe, buffers, [this](bool ok) {
      if (!ok) {
        finished.set_value(false);
        return;
      }
      pipe->write(makeMessage(buffers), [this](const Error& error) {
        if (error) {
          fprintf(stderr, "write: %s\n", error.what().c_str());
          finished.set_value(false);
          return;
        }
        step();
      });
    });
  }
};

struct Client {
  std::shared_ptr<Pipe> pipe;
  Buffers out, back;
  int warmup{0}, iters{0}, done{0}, mismatches{0};
  std::vector<double> samples;
  std::chrono::steady_clock::time_point begin, t0;
  double totalUs{0};
  std::promise<bool> finished;

  void step() {
    if (done == warmup + iters) {
      totalUs = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - begin)
                    .count();
      finished.set_value(true);
      return;
    }
    if (done == warmup) {
      begin = std::chrono::steady_clock::now();
    }
    t0 = std::chrono::steady_clock::now();
    pipe->write(makeMessage(out), [this](const Error& error) {
      if (error) {
        fprintf(stderr, "write: %s\n", error.what().c_str());
      }
    });
    readOne(*pipe, back, [this](bool ok) {
      if (!ok) {
        finished.set_value(false);
        return;
      }
      auto t1 = std::chrono::steady_clock::now();
      if (done >= warmup) {
        samples.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count());
      }
      if (back.tensor != out.tensor || back.payload != out.payload) {
        ++mismatches;
      }
      ++done;
      step();
    });
  }
};

int main(int argc, char** argv) {
  if (argc < 5) {
    fprintf(stderr, "usage: %s tensor_bytes payload_bytes warmup iters\n", argv[0]);
    return 2;
  }
  const size_t tensorBytes = strtoull(argv[1], nullptr, 10);
  const size_t payloadBytes = strtoull(argv[2], nullptr, 10);
  const int warmup = atoi(argv[3]);
  const int iters = atoi(argv[4]);
  const std::string addr = "tp_ref_bench_" + std::to_string(getpid());

  pid_t pid = fork();
  if (pid == 0) {
    // server: accept one pipe, echo
    auto ctx = makeContext("server");
    auto listener = ctx->listen({"shm://" + addr});
    std::promise<std::shared_ptr<Pipe>> pp;
    listener->accept([&](const Error& error, std::shared_ptr<Pipe> pipe) {
      if (error) {
        fprintf(stderr, "accept: %s\n", error.what().c_str());
      }
      pp.set_value(std::move(pipe));
    });
    Server server;
    server.pipe = pp.get_future().get();
    server.buffers = Buffers{std::vector<uint8_t>(tensorBytes), std::vector<uint8_t>(payloadBytes)};
    server.remaining = warmup + iters;
    bool ok = server.pipe != nullptr;
    if (ok) {
      server.step();
      ok = server.finished.get_future().get();
    }
    server.pipe.reset();
    listener.reset();
    ctx->join();
    _exit(ok ? 0 : 1);
  }

  usleep(300 * 1000); // let the server bind
  auto ctx = makeContext("client");
  Client client;
  client.pipe = ctx->connect("shm://" + addr);
  client.out = Buffers{std::vector<uint8_t>(tensorBytes), std::vector<uint8_t>(payloadBytes)};
  client.back = Buffers{std::vector<uint8_t>(tensorBytes), std::vector<uint8_t>(payloadBytes)};
  for (size_t i = 0; i < tensorBytes; ++i) {
    client.out.tensor[i] = static_cast<uint8_t>((i >> 8) ^ (i & 0xff));
  }
  for (size_t i = 0; i < payloadBytes; ++i) {
    client.out.payload[i] = static_cast<uint8_t>((i >> 8) ^ (i & 0xff));
  }
  client.warmup = warmup;
  client.iters = iters;
  client.step();
  const bool ok = client.finished.get_future().get();
  client.pipe.reset();
  ctx->join();
  int st = 0;
  waitpid(pid, &st, 0);
  std::vector<double>& samples = client.samples;
  const double totalUs = client.totalUs;
  const int mismatches = client.mismatches;
  if (!ok || samples.empty()) {
    fprintf(stderr, "ping-pong failed\n");
    return 1;
  }
  std::sort(samples.begin(), samples.end());
  double p50 = samples[static_cast<size_t>(0.5 * samples.size())];
  double gbps = 2.0 * tensorBytes * samples.size() / (totalUs * 1e-6) / 1e9;
  printf(
      "{\"kind\": \"reference\", \"tensor_bytes\": %zu, \"payload_bytes\": %zu, \"iters\": %zu, "
      "\"rtt_p50_us\": %.3f, \"rtt_min_us\": %.3f, \"payload_GBps\": %.4f, \"mismatches\": %d, "
      "\"child_status\": %d}\n",
      tensorBytes, payloadBytes, samples.size(), p50, samples[0], gbps, mismatches, WEXITSTATUS(st));
  return mismatches == 0 ? 0 : 1;
}
