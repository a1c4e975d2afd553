// See compat_pipe.h.
#include <nopwire/compat_pipe.h>

#include <arpa/inet.h>
#include <netinet/in.h>
#include <netinet/tcp.h>
#include <poll.h>
#include <sys/socket.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>

namespace tpnop {

namespace {

constexpr int kTimeoutMs = 20000;
const char* const kTransport = "uv";
const char* const kTransportDomain = "uv:*"; // what a stock uv context announces
const char* const kChannel = "basic";
const char* const kChannelDomain = "any"; // what a stock basic channel announces for cpu:0

bool fail(std::string* error, const std::string& what) {
  if (error != nullptr) {
    *error = what;
  }
  return false;
}

bool readAll(int fd, void* p, size_t n) {
  uint8_t* q = static_cast<uint8_t*>(p);
  while (n > 0) {
    pollfd pf{fd, POLLIN, 0};
    const int rc = ::poll(&pf, 1, kTimeoutMs);
    if (rc < 0 && errno == EINTR) {
      continue;
    }
    if (rc <= 0) {
      return false;
    }
    const ssize_t r = ::read(fd, q, n);
    if (r < 0 && (errno == EINTR || errno == EAGAIN)) {
      continue;
    }
    if (r <= 0) {
      return false;
    }
    q += r;
    n -= static_cast<size_t>(r);
  }
  return true;
}

bool writeAll(int fd, const void* p, size_t n) {
  const uint8_t* q = static_cast<const uint8_t*>(p);
  while (n > 0) {
    const ssize_t r = ::send(fd, q, n, MSG_NOSIGNAL);
    if (r < 0 && errno == EINTR) {
      continue;
    }
    if (r <= 0) {
      return false;
    }
    q += r;
    n -= static_cast<size_t>(r);
  }
  return true;
}

int dial(const std::string& address) {
  const size_t colon = address.rfind(':');
  if (colon == std::string::npos) {
    return -1;
  }
  sockaddr_in sa{};
  sa.sin_family = AF_INET;
  sa.sin_port = htons(static_cast<uint16_t>(std::atoi(address.c_str() + colon + 1)));
  if (::inet_pton(AF_INET, address.substr(0, colon).c_str(), &sa.sin_addr) != 1) {
    return -1;
  }
  const int fd = ::socket(AF_INET, SOCK_STREAM, 0);
  if (fd < 0) {
    return -1;
  }
  if (::connect(fd, reinterpret_cast<sockaddr*>(&sa), sizeof(sa)) != 0) {
    ::close(fd);
    return -1;
  }
  int one = 1;
  ::setsockopt(fd, IPPROTO_TCP, TCP_NODELAY, &one, sizeof(one));
  return fd;
}

const Device kCpu{"cpu", 0};

WireMap<std::string, WireMap<Device, std::string>> ownChannels() {
  return {{kChannel, {{kCpu, kChannelDomain}}}};
}

bool offersBasicOnCpu(const WireMap<std::string, WireMap<Device, std::string>>& channels) {
  for (auto& c : channels) {
    if (c.first != kChannel) {
      continue;
    }
    for (auto& d : c.second) {
      if (d.first == kCpu && d.second == kChannelDomain) {
        return true;
      }
    }
  }
  return false;
}

} // namespace

CompatPipe::~CompatPipe() {
  for (int fd : {descriptorFd_, replyFd_, channelFd_}) {
    if (fd >= 0) {
      ::close(fd);
    }
  }
}

bool CompatPipe::writeFrame(int fd, char which, const void* data, size_t size, std::string* error) {
  uint8_t header[kFrameHeaderBytes];
  putFrameHeader(size, header);
  if (!writeAll(fd, header, sizeof(header)) || (size > 0 && !writeAll(fd, data, size))) {
    return fail(error, std::string("writing a frame failed: ") + std::strerror(errno));
  }
  const uint8_t* p = static_cast<const uint8_t*>(data);
  frames_.push_back(Frame{'w', which, Bytes(p, p + size)});
  return true;
}

bool CompatPipe::readFrame(int fd, char which, Bytes* out, std::string* error) {
  uint8_t header[kFrameHeaderBytes];
  if (!readAll(fd, header, sizeof(header))) {
    return fail(error, "no frame arrived in time");
  }
  const uint64_t size = getFrameHeader(header);
  if (size > (uint64_t(1) << 32)) {
    return fail(error, "frame too large");
  }
  // The buffer grows with what arrives, not with what the header announces.
  out->clear();
  constexpr size_t kStep = 1 << 20;
  for (size_t have = 0; have < size;) {
    const size_t n = static_cast<size_t>(std::min<uint64_t>(size - have, kStep));
    out->resize(have + n);
    if (!readAll(fd, out->data() + have, n)) {
      return fail(error, "a frame stopped short");
    }
    have += n;
  }
  frames_.push_back(Frame{'r', which, *out});
  return true;
}

std::unique_ptr<CompatPipe> CompatPipe::connect(
    const std::string& address, const std::string& contextName, std::string* error) {
  std::unique_ptr<CompatPipe> pipe(new CompatPipe());
  pipe->descriptorFd_ = dial(address);
  if (pipe->descriptorFd_ < 0) {
    fail(error, "cannot connect to " + address);
    return nullptr;
  }
  Packet hello;
  hello.which = Packet::kSpontaneous;
  hello.spontaneous.contextName = contextName;
  Bytes bytes = encode(hello);
  if (!pipe->writeFrame(pipe->descriptorFd_, 'd', bytes.data(), bytes.size(), error)) {
    return nullptr;
  }
  Brochure brochure;
  brochure.transportDomainDescriptors = {{kTransport, kTransportDomain}};
  brochure.channelDeviceDescriptors = ownChannels();
  bytes = encode(brochure);
  if (!pipe->writeFrame(pipe->descriptorFd_, 'd', bytes.data(), bytes.size(), error)) {
    return nullptr;
  }
  if (!pipe->readFrame(pipe->descriptorFd_, 'd', &bytes, error)) {
    return nullptr;
  }
  BrochureAnswer answer;
  if (!decode(bytes.data(), bytes.size(), &answer)) {
    fail(error, "the brochure answer does not parse");
    return nullptr;
  }
  if (answer.transport != kTransport) {
    fail(error, "the peer chose transport " + answer.transport);
    return nullptr;
  }
  // The connection in use stays the descriptor connection (the transport did
  // not change); descriptor replies and the channel get one more each.
  const uint64_t* replyToken = nullptr;
  for (auto& kv : answer.transportRegistrationIds) {
    if (kv.first == 1) {
      replyToken = &kv.second;
    }
  }
  const std::vector<uint64_t>* channelTokens = nullptr;
  for (auto& kv : answer.channelRegistrationIds) {
    if (kv.first == kChannel) {
      channelTokens = &kv.second;
    }
  }
  if (replyToken == nullptr || channelTokens == nullptr || channelTokens->size() != 1) {
    fail(error, "the brochure answer lacks the descriptor reply connection or the basic channel");
    return nullptr;
  }
  auto requested = [&](uint64_t token, char which, int* fd) {
    *fd = dial(answer.address);
    if (*fd < 0) {
      return fail(error, "cannot connect to " + answer.address);
    }
    Packet p;
    p.which = Packet::kRequested;
    p.requested.registrationId = token;
    Bytes b = encode(p);
    return pipe->writeFrame(*fd, which, b.data(), b.size(), error);
  };
  if (!requested(*replyToken, 'r', &pipe->replyFd_) ||
      !requested((*channelTokens)[0], 'c', &pipe->channelFd_)) {
    return nullptr;
  }
  return pipe;
}

bool CompatPipe::write(const CompatMessage& message, std::string* error) {
  Descriptor d;
  d.metadata = message.metadata;
  bool missingTargets = false;
  for (auto& p : message.payloads) {
    d.payloads.push_back(PayloadDescriptor{p.bytes.size(), p.metadata});
  }
  for (auto& t : message.tensors) {
    TensorDescriptor td;
    td.length = t.bytes.size();
    td.sourceDevice = kCpu;
    td.hasTargetDevice = t.nameTarget;
    td.targetDevice = kCpu;
    td.metadata = t.metadata;
    missingTargets |= !t.nameTarget;
    d.tensors.push_back(std::move(td));
  }
  Bytes bytes = encode(d);
  if (!writeFrame(descriptorFd_, 'd', bytes.data(), bytes.size(), error)) {
    return false;
  }
  for (auto& p : message.payloads) {
    if (!writeFrame(descriptorFd_, 'd', p.bytes.data(), p.bytes.size(), error)) {
      return false;
    }
  }
  if (missingTargets) {
    // tensorpipe/core/pipe_impl.cc:961-985: the receiver says where the
    // tensors without a target go before any tensor is sent.
    if (!readFrame(replyFd_, 'r', &bytes, error)) {
      return false;
    }
    DescriptorReply reply;
    if (!decode(bytes.data(), bytes.size(), &reply)) {
      return fail(error, "the descriptor reply does not parse");
    }
    size_t missing = 0;
    for (auto& t : message.tensors) {
      missing += t.nameTarget ? 0 : 1;
    }
    if (reply.targetDevices.size() != missing) {
      return fail(error, "the descriptor reply names the wrong number of devices");
    }
    for (auto& dev : reply.targetDevices) {
      if (!(dev == kCpu)) {
        return fail(error, "the peer wants a tensor on " + dev.type + ", which this endpoint cannot serve");
      }
    }
  }
  for (auto& t : message.tensors) {
    // channel/basic/channel_impl.cc:60-76: nothing travels for an empty tensor
    if (!t.bytes.empty() && !writeFrame(channelFd_, 'c', t.bytes.data(), t.bytes.size(), error)) {
      return false;
    }
  }
  return true;
}

bool CompatPipe::read(CompatMessage* message, std::string* error) {
  Bytes bytes;
  if (!readFrame(descriptorFd_, 'd', &bytes, error)) {
    return false;
  }
  Descriptor d;
  if (!decode(bytes.data(), bytes.size(), &d)) {
    return fail(error, "the descriptor does not parse");
  }
  *message = CompatMessage();
  message->metadata = d.metadata;
  for (auto& p : d.payloads) {
    if (!readFrame(descriptorFd_, 'd', &bytes, error)) {
      return false;
    }
    if (bytes.size() != p.length) {
      return fail(error, "a payload has another length than its descriptor says");
    }
    message->payloads.push_back(
        CompatMessage::Payload{std::string(bytes.begin(), bytes.end()), p.metadata});
  }
  DescriptorReply reply;
  for (auto& t : d.tensors) {
    if (t.sourceDevice.type != "cpu" || (t.hasTargetDevice && t.targetDevice.type != "cpu")) {
      return fail(error, "a tensor on " + t.sourceDevice.type + ": this endpoint takes CPU tensors only");
    }
    if (!t.hasTargetDevice) {
      reply.targetDevices.push_back(kCpu);
    }
  }
  if (!reply.targetDevices.empty()) {
    bytes = encode(reply);
    if (!writeFrame(replyFd_, 'r', bytes.data(), bytes.size(), error)) {
      return false;
    }
  }
  for (auto& t : d.tensors) {
    CompatMessage::Tensor out;
    out.metadata = t.metadata;
    out.nameTarget = t.hasTargetDevice;
    if (t.length > 0) {
      if (!readFrame(channelFd_, 'c', &bytes, error)) {
        return false;
      }
      if (bytes.size() != t.length) {
        return fail(error, "a tensor has another length than its descriptor says");
      }
      out.bytes.assign(bytes.begin(), bytes.end());
    }
    message->tensors.push_back(std::move(out));
  }
  return true;
}

std::unique_ptr<CompatListener> CompatListener::create(std::string* error) {
  std::unique_ptr<CompatListener> l(new CompatListener());
  l->fd_ = ::socket(AF_INET, SOCK_STREAM, 0);
  sockaddr_in sa{};
  sa.sin_family = AF_INET;
  sa.sin_addr.s_addr = htonl(INADDR_LOOPBACK);
  sa.sin_port = 0;
  int one = 1;
  if (l->fd_ < 0 || ::setsockopt(l->fd_, SOL_SOCKET, SO_REUSEADDR, &one, sizeof(one)) != 0 ||
      ::bind(l->fd_, reinterpret_cast<sockaddr*>(&sa), sizeof(sa)) != 0 || ::listen(l->fd_, 16) != 0) {
    fail(error, std::string("cannot listen: ") + std::strerror(errno));
    return nullptr;
  }
  socklen_t len = sizeof(sa);
  ::getsockname(l->fd_, reinterpret_cast<sockaddr*>(&sa), &len);
  l->port_ = ntohs(sa.sin_port);
  return l;
}

CompatListener::~CompatListener() {
  if (fd_ >= 0) {
    ::close(fd_);
  }
}

std::string CompatListener::address() const {
  return "127.0.0.1:" + std::to_string(port_);
}

std::unique_ptr<CompatPipe> CompatListener::accept(const std::string& contextName, std::string* error) {
  auto acceptOne = [&]() -> int {
    pollfd pf{fd_, POLLIN, 0};
    if (::poll(&pf, 1, kTimeoutMs) <= 0) {
      return -1;
    }
    const int fd = ::accept(fd_, nullptr, nullptr);
    if (fd >= 0) {
      int one = 1;
      ::setsockopt(fd, IPPROTO_TCP, TCP_NODELAY, &one, sizeof(one));
    }
    return fd;
  };
  std::unique_ptr<CompatPipe> pipe(new CompatPipe());
  pipe->descriptorFd_ = acceptOne();
  if (pipe->descriptorFd_ < 0) {
    fail(error, "nobody connected");
    return nullptr;
  }
  Bytes bytes;
  Packet hello;
  if (!pipe->readFrame(pipe->descriptorFd_, 'd', &bytes, error)) {
    return nullptr;
  }
  if (!decode(bytes.data(), bytes.size(), &hello) || hello.which != Packet::kSpontaneous) {
    fail(error, "the first packet is not a spontaneous connection");
    return nullptr;
  }
  pipe->remoteName_ = hello.spontaneous.contextName;
  Brochure brochure;
  if (!pipe->readFrame(pipe->descriptorFd_, 'd', &bytes, error)) {
    return nullptr;
  }
  if (!decode(bytes.data(), bytes.size(), &brochure)) {
    fail(error, "the brochure does not parse");
    return nullptr;
  }
  bool sameTransport = false;
  for (auto& t : brochure.transportDomainDescriptors) {
    sameTransport |= t.first == kTransport && t.second == kTransportDomain;
  }
  if (!sameTransport || !offersBasicOnCpu(brochure.channelDeviceDescriptors)) {
    fail(error, "the peer does not offer the uv transport and the basic channel");
    return nullptr;
  }
  (void)contextName; // a listening end never says its name on the wire
  BrochureAnswer answer;
  answer.transport = kTransport;
  answer.address = address();
  const uint64_t replyToken = nextToken_++;
  const uint64_t channelToken = nextToken_++;
  answer.transportRegistrationIds = {{1, replyToken}}; // same transport: only the reply connection is new
  answer.transportDomainDescriptor = kTransportDomain;
  answer.channelRegistrationIds = {{kChannel, {channelToken}}};
  answer.channelDeviceDescriptors = ownChannels();
  answer.channelForDevicePair = {{{kCpu, kCpu}, kChannel}};
  bytes = encode(answer);
  if (!pipe->writeFrame(pipe->descriptorFd_, 'd', bytes.data(), bytes.size(), error)) {
    return nullptr;
  }
  // The two requested connections, in whichever order they come.
  for (int k = 0; k < 2; ++k) {
    const int fd = acceptOne();
    if (fd < 0) {
      fail(error, "a requested connection never came");
      return nullptr;
    }
    // Which of the two it is shows in its first packet; until then the frame
    // is read on behalf of neither.
    uint8_t header[kFrameHeaderBytes];
    Packet p;
    if (!readAll(fd, header, sizeof(header))) {
      ::close(fd);
      fail(error, "a requested connection said nothing");
      return nullptr;
    }
    bytes.resize(static_cast<size_t>(getFrameHeader(header) & 0xffff));
    if ((!bytes.empty() && !readAll(fd, bytes.data(), bytes.size())) ||
        !decode(bytes.data(), bytes.size(), &p) || p.which != Packet::kRequested) {
      ::close(fd);
      fail(error, "a requested connection did not introduce itself");
      return nullptr;
    }
    if (p.requested.registrationId == replyToken && pipe->replyFd_ < 0) {
      pipe->replyFd_ = fd;
      pipe->frames_.push_back(CompatPipe::Frame{'r', 'r', bytes});
    } else if (p.requested.registrationId == channelToken && pipe->channelFd_ < 0) {
      pipe->channelFd_ = fd;
      pipe->frames_.push_back(CompatPipe::Frame{'r', 'c', bytes});
    } else {
      ::close(fd);
      fail(error, "a requested connection carries an unknown token");
      return nullptr;
    }
  }
  return pipe;
}

} // namespace tpnop
