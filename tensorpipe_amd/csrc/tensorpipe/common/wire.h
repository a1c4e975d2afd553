// Little-endian byte packing for control messages (handshake, descriptors).
// Own framing; no third-party serializer.
#pragma once

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

class WireWriter {
 public:
  void u8(uint8_t v) {
    buf_.push_back(v);
  }
  void u32(uint32_t v) {
    raw(&v, sizeof(v));
  }
  void u64(uint64_t v) {
    raw(&v, sizeof(v));
  }
  void str(const std::string& s) {
    u32(static_cast<uint32_t>(s.size()));
    raw(s.data(), s.size());
  }
  void raw(const void* p, size_t n) {
    const uint8_t* b = static_cast<const uint8_t*>(p);
    buf_.insert(buf_.end(), b, b + n);
  }
  std::vector<uint8_t>& bytes() {
    return buf_;
  }

 private:
  std::vector<uint8_t> buf_;
};

class WireReader {
 public:
  WireReader(const void* p, size_t n) : p_(static_cast<const uint8_t*>(p)), n_(n) {}

  bool ok() const {
    return ok_;
  }
  bool atEnd() const {
    return off_ == n_;
  }
  uint8_t u8() {
    uint8_t v = 0;
    raw(&v, 1);
    return v;
  }
  uint32_t u32() {
    uint32_t v = 0;
    raw(&v, sizeof(v));
    return v;
  }
  uint64_t u64() {
    uint64_t v = 0;
    raw(&v, sizeof(v));
    return v;
  }
  std::string str() {
    uint32_t len = u32();
    if (!ok_ || len > n_ - off_) {
      ok_ = false;
      return std::string();
    }
    std::string s(reinterpret_cast<const char*>(p_ + off_), len);
    off_ += len;
    return s;
  }
  void raw(void* out, size_t n) {
    if (!ok_ || n > n_ - off_) {
      ok_ = false;
      std::memset(out, 0, n);
      return;
    }
    std::memcpy(out, p_ + off_, n);
    off_ += n;
  }

 private:
  const uint8_t* p_;
  size_t n_;
  size_t off_{0};
  bool ok_{true};
};

TP_AMD_NAMESPACE_END
