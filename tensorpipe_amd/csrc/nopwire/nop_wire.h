// The control messages of a stock TensorPipe pipe, in the encoding stock
// endpoints put on the wire: the structures of tensorpipe/core/nop_types.h:26-80
// serialised the way libnop (google/libnop, the serializer behind
// tensorpipe/common/nop.h) does, and the length-prefixed framing of the stream
// transports (tensorpipe/common/stream_read_write_ops.h:30-65,146-188).
//
// libnop's format, as far as these messages use it (one prefix byte per value):
//   0x00..0x7f  the integer itself                 0xc0..0xff  the integer - 256 (-64..-1)
//   0x80 u8   0x81 u16   0x82 u32   0x83 u64       0x84 i8   0x85 i16   0x86 i32   0x87 i64
//             (little endian; a writer takes the shortest form that holds the value)
//   0xb8 variant:   index (integer, -1 = empty), then the alternative
//   0xb9 structure: member count, then the members in declaration order
//   0xba array:     element count, then the elements        (std::vector of structures, std::pair)
//   0xbb map:       entry count, then key, value, key, value ...
//   0xbc binary:    byte count, then raw little-endian data (std::vector of integers)
//   0xbd string:    byte count, then the bytes
//   0xbe nil        (an empty optional; a full one is just its value)
// Pinned by byte strings captured from the TensorPipe that PyTorch ships
// (tests/golden/stock_wire_vectors.txt).
//
// This header names no TensorPipe type on purpose: it can be included next to
// this library's headers or next to a stock TensorPipe's.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace tpnop {

struct Device {
  std::string type;
  int64_t index{0};
  bool operator==(const Device& o) const {
    return type == o.type && index == o.index;
  }
};

// Maps keep the order they had on the wire (stock endpoints write theirs in
// hash order), so that decoding and encoding again gives the same bytes.
template <typename K, typename V>
using WireMap = std::vector<std::pair<K, V>>;

// tensorpipe/core/nop_types.h:26-34
struct SpontaneousConnection {
  std::string contextName;
};
struct RequestedConnection {
  uint64_t registrationId{0};
};
// nop_types.h:80: Variant<SpontaneousConnection, RequestedConnection>
struct Packet {
  enum Which : int { kSpontaneous = 0, kRequested = 1 };
  int which{kSpontaneous};
  SpontaneousConnection spontaneous;
  RequestedConnection requested;
};

// nop_types.h:38-43
struct Brochure {
  WireMap<std::string, std::string> transportDomainDescriptors;
  WireMap<std::string, WireMap<Device, std::string>> channelDeviceDescriptors;
};

// nop_types.h:45-64
struct BrochureAnswer {
  std::string transport;
  std::string address;
  WireMap<uint64_t, uint64_t> transportRegistrationIds;
  std::string transportDomainDescriptor;
  WireMap<std::string, std::vector<uint64_t>> channelRegistrationIds;
  WireMap<std::string, WireMap<Device, std::string>> channelDeviceDescriptors;
  WireMap<std::pair<Device, Device>, std::string> channelForDevicePair;
};

// nop_types.h:66-73 over tensorpipe/core/message.h:63-98
struct PayloadDescriptor {
  uint64_t length{0};
  std::string metadata;
};
struct TensorDescriptor {
  uint64_t length{0};
  Device sourceDevice;
  bool hasTargetDevice{false};
  Device targetDevice;
  std::string metadata;
};
struct Descriptor {
  std::string metadata;
  std::vector<PayloadDescriptor> payloads;
  std::vector<TensorDescriptor> tensors;
};

// nop_types.h:75-78
struct DescriptorReply {
  std::vector<Device> targetDevices;
};

using Bytes = std::vector<uint8_t>;

Bytes encode(const Packet& v);
Bytes encode(const Brochure& v);
Bytes encode(const BrochureAnswer& v);
Bytes encode(const Descriptor& v);
Bytes encode(const DescriptorReply& v);

// False when the bytes are not a complete, well-formed encoding of the type
// (trailing bytes count as malformed).
bool decode(const uint8_t* data, size_t size, Packet* out);
bool decode(const uint8_t* data, size_t size, Brochure* out);
bool decode(const uint8_t* data, size_t size, BrochureAnswer* out);
bool decode(const uint8_t* data, size_t size, Descriptor* out);
bool decode(const uint8_t* data, size_t size, DescriptorReply* out);

// A message on a stream transport: its length as a 64-bit little-endian word,
// then the bytes.
constexpr size_t kFrameHeaderBytes = 8;
void putFrameHeader(uint64_t length, uint8_t out[kFrameHeaderBytes]);
uint64_t getFrameHeader(const uint8_t in[kFrameHeaderBytes]);

} // namespace tpnop
