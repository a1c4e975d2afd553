// A small endpoint that speaks a stock TensorPipe pipe's protocol over TCP (its
// uv transport) well enough to exchange messages of payloads and CPU tensors
// with an unmodified peer: the handshake of tensorpipe/core/pipe_impl.cc:262-345,
// 987-1157 (spontaneous connection, brochure, brochure answer, one requested
// connection for descriptor replies and one for the `basic` channel), then
// descriptors, payloads, descriptor replies and tensors as
// pipe_impl.cc:918-985, 440-470 and channel/basic/channel_impl.cc:60-110 put
// them on the wire. Everything is encoded by nop_wire.
//
// Blocking and single-threaded on purpose: it exists to show, and to test
// against the real thing, that the encodings and the sequence are right; it is
// not the asynchronous pipe of this library and it does not carry GPU tensors
// (those need this library's channels on both ends; a host that wants them
// registers the channels in its own TensorPipe).
#pragma once

#include <memory>
#include <string>
#include <vector>

#include <nopwire/nop_wire.h>

namespace tpnop {

struct CompatMessage {
  struct Payload {
    std::string bytes;
    std::string metadata;
  };
  struct Tensor {
    std::string bytes; // CPU memory
    std::string metadata;
    // Whether the sender names the target device in the descriptor; when it
    // does not, the receiver answers with a descriptor reply.
    bool nameTarget{true};
  };
  std::string metadata;
  std::vector<Payload> payloads;
  std::vector<Tensor> tensors;
};

class CompatPipe {
 public:
  // Client: opens a pipe to the listener at "host:port" (what follows "uv://"
  // in a stock address).
  static std::unique_ptr<CompatPipe> connect(
      const std::string& address, const std::string& contextName, std::string* error);
  ~CompatPipe();
  CompatPipe(const CompatPipe&) = delete;
  CompatPipe& operator=(const CompatPipe&) = delete;

  bool write(const CompatMessage& message, std::string* error);
  bool read(CompatMessage* message, std::string* error);
  const std::string& remoteName() const {
    return remoteName_;
  }
  // Every frame this end wrote or read, in order, for a test that wants to
  // look at the bytes: 'w' or 'r', the connection ('d'escriptor, 'r'eply,
  // 'c'hannel), the bytes.
  struct Frame {
    char direction;
    char connection;
    Bytes bytes;
  };
  const std::vector<Frame>& frames() const {
    return frames_;
  }

 private:
  friend class CompatListener;
  CompatPipe() = default;
  bool writeFrame(int fd, char which, const void* data, size_t size, std::string* error);
  bool readFrame(int fd, char which, Bytes* out, std::string* error);

  int descriptorFd_{-1};
  int replyFd_{-1};
  int channelFd_{-1};
  std::string remoteName_;
  std::vector<Frame> frames_;
};

class CompatListener {
 public:
  // Listens on 127.0.0.1, port chosen by the system.
  static std::unique_ptr<CompatListener> create(std::string* error);
  ~CompatListener();
  std::string address() const; // "127.0.0.1:port"
  // Takes one incoming pipe through its handshake.
  std::unique_ptr<CompatPipe> accept(const std::string& contextName, std::string* error);

 private:
  CompatListener() = default;
  int fd_{-1};
  int port_{0};
  uint64_t nextToken_{0};
};

} // namespace tpnop
