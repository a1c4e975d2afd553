// See nop_wire.h.
#include <nopwire/nop_wire.h>

#include <cstring>
#include <limits>

namespace tpnop {

namespace {

enum Prefix : uint8_t {
  kU8 = 0x80,
  kU16 = 0x81,
  kU32 = 0x82,
  kU64 = 0x83,
  kI8 = 0x84,
  kI16 = 0x85,
  kI32 = 0x86,
  kI64 = 0x87,
  kVariant = 0xb8,
  kStructure = 0xb9,
  kArray = 0xba,
  kMap = 0xbb,
  kBinary = 0xbc,
  kString = 0xbd,
  kNil = 0xbe,
};

class Writer {
 public:
  void byte(uint8_t b) {
    out_.push_back(b);
  }
  void raw(const void* p, size_t n) {
    const uint8_t* q = static_cast<const uint8_t*>(p);
    out_.insert(out_.end(), q, q + n);
  }
  template <typename T>
  void le(T v) {
    for (size_t i = 0; i < sizeof(T); ++i) {
      out_.push_back(static_cast<uint8_t>(static_cast<uint64_t>(v) >> (8 * i)));
    }
  }
  void uinteger(uint64_t v) {
    if (v < 0x80) {
      byte(static_cast<uint8_t>(v));
    } else if (v <= 0xff) {
      byte(kU8);
      le<uint8_t>(static_cast<uint8_t>(v));
    } else if (v <= 0xffff) {
      byte(kU16);
      le<uint16_t>(static_cast<uint16_t>(v));
    } else if (v <= 0xffffffffull) {
      byte(kU32);
      le<uint32_t>(static_cast<uint32_t>(v));
    } else {
      byte(kU64);
      le<uint64_t>(v);
    }
  }
  void integer(int64_t v) {
    if (v >= -64 && v <= 127) {
      byte(static_cast<uint8_t>(v));
    } else if (v >= std::numeric_limits<int8_t>::min() && v <= std::numeric_limits<int8_t>::max()) {
      byte(kI8);
      le<uint8_t>(static_cast<uint8_t>(v));
    } else if (v >= std::numeric_limits<int16_t>::min() && v <= std::numeric_limits<int16_t>::max()) {
      byte(kI16);
      le<uint16_t>(static_cast<uint16_t>(v));
    } else if (v >= std::numeric_limits<int32_t>::min() && v <= std::numeric_limits<int32_t>::max()) {
      byte(kI32);
      le<uint32_t>(static_cast<uint32_t>(v));
    } else {
      byte(kI64);
      le<uint64_t>(static_cast<uint64_t>(v));
    }
  }
  void string(const std::string& s) {
    byte(kString);
    uinteger(s.size());
    raw(s.data(), s.size());
  }
  void structure(size_t members) {
    byte(kStructure);
    uinteger(members);
  }
  void array(size_t elements) {
    byte(kArray);
    uinteger(elements);
  }
  void map(size_t entries) {
    byte(kMap);
    uinteger(entries);
  }
  void integers(const std::vector<uint64_t>& v) {
    byte(kBinary);
    uinteger(v.size() * sizeof(uint64_t));
    for (uint64_t x : v) {
      le<uint64_t>(x);
    }
  }
  void device(const Device& d) {
    structure(2);
    string(d.type);
    integer(d.index);
  }
  void deviceDescriptors(const WireMap<std::string, WireMap<Device, std::string>>& m) {
    map(m.size());
    for (auto& channel : m) {
      string(channel.first);
      map(channel.second.size());
      for (auto& kv : channel.second) {
        device(kv.first);
        string(kv.second);
      }
    }
  }
  Bytes take() {
    return std::move(out_);
  }

 private:
  Bytes out_;
};

class Reader {
 public:
  Reader(const uint8_t* p, size_t n) : p_(p), end_(p + n) {}
  bool ok() const {
    return ok_;
  }
  bool atEnd() const {
    return ok_ && p_ == end_;
  }
  uint8_t byte() {
    if (!ok_ || p_ == end_) {
      ok_ = false;
      return 0;
    }
    return *p_++;
  }
  template <typename T>
  T le() {
    if (!ok_ || static_cast<size_t>(end_ - p_) < sizeof(T)) {
      ok_ = false;
      return T(0);
    }
    uint64_t v = 0;
    for (size_t i = 0; i < sizeof(T); ++i) {
      v |= static_cast<uint64_t>(p_[i]) << (8 * i);
    }
    p_ += sizeof(T);
    return static_cast<T>(v);
  }
  // Any integer encoding whose value is not negative.
  uint64_t uinteger() {
    const uint8_t b = byte();
    if (b < 0x80) {
      return b;
    }
    switch (b) {
      case kU8:
        return le<uint8_t>();
      case kU16:
        return le<uint16_t>();
      case kU32:
        return le<uint32_t>();
      case kU64:
        return le<uint64_t>();
      default:
        break;
    }
    const int64_t s = signedTail(b);
    if (s < 0) {
      ok_ = false;
    }
    return static_cast<uint64_t>(s);
  }
  int64_t integer() {
    const uint8_t b = byte();
    if (b < 0x80) {
      return b;
    }
    switch (b) {
      case kU8:
        return le<uint8_t>();
      case kU16:
        return le<uint16_t>();
      case kU32:
        return le<uint32_t>();
      case kU64: {
        const uint64_t v = le<uint64_t>();
        if (v > static_cast<uint64_t>(std::numeric_limits<int64_t>::max())) {
          ok_ = false;
        }
        return static_cast<int64_t>(v);
      }
      default:
        return signedTail(b);
    }
  }
  bool expect(uint8_t prefix) {
    if (byte() != prefix) {
      ok_ = false;
    }
    return ok_;
  }
  // A count of things that take at least `unit` bytes each.
  size_t count(size_t unit) {
    const uint64_t n = uinteger();
    if (ok_ && n > static_cast<uint64_t>(end_ - p_) / (unit == 0 ? 1 : unit)) {
      ok_ = false;
    }
    return ok_ ? static_cast<size_t>(n) : 0;
  }
  std::string string() {
    expect(kString);
    const size_t n = count(1);
    std::string s;
    if (ok_) {
      s.assign(reinterpret_cast<const char*>(p_), n);
      p_ += n;
    }
    return s;
  }
  bool structure(size_t members) {
    expect(kStructure);
    if (uinteger() != members) {
      ok_ = false;
    }
    return ok_;
  }
  size_t array() {
    expect(kArray);
    return count(1);
  }
  size_t map() {
    expect(kMap);
    return count(2);
  }
  std::vector<uint64_t> integers() {
    expect(kBinary);
    const size_t bytes = count(1);
    std::vector<uint64_t> v;
    if (ok_ && bytes % sizeof(uint64_t) != 0) {
      ok_ = false;
    }
    for (size_t i = 0; ok_ && i < bytes / sizeof(uint64_t); ++i) {
      v.push_back(le<uint64_t>());
    }
    return v;
  }
  Device device() {
    Device d;
    structure(2);
    d.type = string();
    d.index = integer();
    return d;
  }
  bool peekNil() {
    if (ok_ && p_ != end_ && *p_ == kNil) {
      ++p_;
      return true;
    }
    return false;
  }
  WireMap<std::string, WireMap<Device, std::string>> deviceDescriptors() {
    WireMap<std::string, WireMap<Device, std::string>> m;
    const size_t channels = map();
    for (size_t i = 0; ok_ && i < channels; ++i) {
      std::string name = string();
      WireMap<Device, std::string> inner;
      const size_t devices = map();
      for (size_t k = 0; ok_ && k < devices; ++k) {
        Device d = device();
        std::string descriptor = string();
        inner.emplace_back(std::move(d), std::move(descriptor));
      }
      m.emplace_back(std::move(name), std::move(inner));
    }
    return m;
  }

 private:
  int64_t signedTail(uint8_t b) {
    if (b >= 0xc0) {
      return static_cast<int64_t>(b) - 256;
    }
    switch (b) {
      case kI8:
        return static_cast<int8_t>(le<uint8_t>());
      case kI16:
        return static_cast<int16_t>(le<uint16_t>());
      case kI32:
        return static_cast<int32_t>(le<uint32_t>());
      case kI64:
        return static_cast<int64_t>(le<uint64_t>());
      default:
        ok_ = false;
        return 0;
    }
  }

  const uint8_t* p_;
  const uint8_t* end_;
  bool ok_{true};
};

} // namespace

Bytes encode(const Packet& v) {
  Writer w;
  w.byte(kVariant);
  w.integer(v.which);
  w.structure(1);
  if (v.which == Packet::kSpontaneous) {
    w.string(v.spontaneous.contextName);
  } else {
    w.uinteger(v.requested.registrationId);
  }
  return w.take();
}

bool decode(const uint8_t* data, size_t size, Packet* out) {
  Reader r(data, size);
  r.expect(kVariant);
  const int64_t which = r.integer();
  if (!r.ok() || (which != Packet::kSpontaneous && which != Packet::kRequested)) {
    return false;
  }
  out->which = static_cast<int>(which);
  r.structure(1);
  if (which == Packet::kSpontaneous) {
    out->spontaneous.contextName = r.string();
  } else {
    out->requested.registrationId = r.uinteger();
  }
  return r.atEnd();
}

Bytes encode(const Brochure& v) {
  Writer w;
  w.structure(2);
  w.map(v.transportDomainDescriptors.size());
  for (auto& kv : v.transportDomainDescriptors) {
    w.string(kv.first);
    w.string(kv.second);
  }
  w.deviceDescriptors(v.channelDeviceDescriptors);
  return w.take();
}

bool decode(const uint8_t* data, size_t size, Brochure* out) {
  Reader r(data, size);
  r.structure(2);
  const size_t transports = r.map();
  out->transportDomainDescriptors.clear();
  for (size_t i = 0; r.ok() && i < transports; ++i) {
    std::string name = r.string();
    std::string descriptor = r.string();
    out->transportDomainDescriptors.emplace_back(std::move(name), std::move(descriptor));
  }
  out->channelDeviceDescriptors = r.deviceDescriptors();
  return r.atEnd();
}

Bytes encode(const BrochureAnswer& v) {
  Writer w;
  w.structure(7);
  w.string(v.transport);
  w.string(v.address);
  w.map(v.transportRegistrationIds.size());
  for (auto& kv : v.transportRegistrationIds) {
    w.uinteger(kv.first);
    w.uinteger(kv.second);
  }
  w.string(v.transportDomainDescriptor);
  w.map(v.channelRegistrationIds.size());
  for (auto& kv : v.channelRegistrationIds) {
    w.string(kv.first);
    w.integers(kv.second);
  }
  w.deviceDescriptors(v.channelDeviceDescriptors);
  w.map(v.channelForDevicePair.size());
  for (auto& kv : v.channelForDevicePair) {
    w.array(2);
    w.device(kv.first.first);
    w.device(kv.first.second);
    w.string(kv.second);
  }
  return w.take();
}

bool decode(const uint8_t* data, size_t size, BrochureAnswer* out) {
  Reader r(data, size);
  *out = BrochureAnswer();
  r.structure(7);
  out->transport = r.string();
  out->address = r.string();
  const size_t ids = r.map();
  for (size_t i = 0; r.ok() && i < ids; ++i) {
    const uint64_t k = r.uinteger();
    const uint64_t v = r.uinteger();
    out->transportRegistrationIds.emplace_back(k, v);
  }
  out->transportDomainDescriptor = r.string();
  const size_t channels = r.map();
  for (size_t i = 0; r.ok() && i < channels; ++i) {
    std::string name = r.string();
    std::vector<uint64_t> tokens = r.integers();
    out->channelRegistrationIds.emplace_back(std::move(name), std::move(tokens));
  }
  out->channelDeviceDescriptors = r.deviceDescriptors();
  const size_t pairs = r.map();
  for (size_t i = 0; r.ok() && i < pairs; ++i) {
    if (r.array() != 2) {
      return false;
    }
    Device a = r.device();
    Device b = r.device();
    std::string channel = r.string();
    out->channelForDevicePair.emplace_back(std::make_pair(std::move(a), std::move(b)), std::move(channel));
  }
  return r.atEnd();
}

Bytes encode(const Descriptor& v) {
  Writer w;
  w.structure(3);
  w.string(v.metadata);
  w.array(v.payloads.size());
  for (auto& p : v.payloads) {
    w.structure(2);
    w.uinteger(p.length);
    w.string(p.metadata);
  }
  w.array(v.tensors.size());
  for (auto& t : v.tensors) {
    w.structure(4);
    w.uinteger(t.length);
    w.device(t.sourceDevice);
    if (t.hasTargetDevice) {
      w.device(t.targetDevice);
    } else {
      w.byte(kNil);
    }
    w.string(t.metadata);
  }
  return w.take();
}

bool decode(const uint8_t* data, size_t size, Descriptor* out) {
  Reader r(data, size);
  *out = Descriptor();
  r.structure(3);
  out->metadata = r.string();
  const size_t payloads = r.array();
  for (size_t i = 0; r.ok() && i < payloads; ++i) {
    PayloadDescriptor p;
    r.structure(2);
    p.length = r.uinteger();
    p.metadata = r.string();
    out->payloads.push_back(std::move(p));
  }
  const size_t tensors = r.array();
  for (size_t i = 0; r.ok() && i < tensors; ++i) {
    TensorDescriptor t;
    r.structure(4);
    t.length = r.uinteger();
    t.sourceDevice = r.device();
    if (!r.peekNil()) {
      t.hasTargetDevice = true;
      t.targetDevice = r.device();
    }
    t.metadata = r.string();
    out->tensors.push_back(std::move(t));
  }
  return r.atEnd();
}

Bytes encode(const DescriptorReply& v) {
  Writer w;
  w.structure(1);
  w.array(v.targetDevices.size());
  for (auto& d : v.targetDevices) {
    w.device(d);
  }
  return w.take();
}

bool decode(const uint8_t* data, size_t size, DescriptorReply* out) {
  Reader r(data, size);
  out->targetDevices.clear();
  r.structure(1);
  const size_t n = r.array();
  for (size_t i = 0; r.ok() && i < n; ++i) {
    out->targetDevices.push_back(r.device());
  }
  return r.atEnd();
}

void putFrameHeader(uint64_t length, uint8_t out[kFrameHeaderBytes]) {
  for (size_t i = 0; i < kFrameHeaderBytes; ++i) {
    out[i] = static_cast<uint8_t>(length >> (8 * i));
  }
}

uint64_t getFrameHeader(const uint8_t in[kFrameHeaderBytes]) {
  uint64_t v = 0;
  for (size_t i = 0; i < kFrameHeaderBytes; ++i) {
    v |= static_cast<uint64_t>(in[i]) << (8 * i);
  }
  return v;
}

} // namespace tpnop
