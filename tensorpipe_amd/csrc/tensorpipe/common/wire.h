// Little-endian byte packing for control messages (handshake, descriptors).
// Own framing; no third-party serializer.
#pragma once

#include <cstdint>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

class WireWriter {
 public:
  WireWriter() {
    buf_.reserve(256);
  }
  // Room for n more bytes without further allocation.
  void reserve(size_t n) {
    buf_.reserve(buf_.size() + n);
  }
  void u8(uint8_t v) {
    buf_.push_back(v);
  }
  void u32(uint32_t v) {
    fixed(&v, std::integral_constant<size_t, sizeof(v)>());
  }
  void u64(uint64_t v) {
    fixed(&v, std::integral_constant<size_t, sizeof(v)>());
  }
  void str(const std::string& s) {
    u32(static_cast<uint32_t>(s.size()));
    if (!s.empty()) {
      raw(s.data(), s.size());
    }
  }
  void raw(const void* p, size_t n) {
    const size_t at = buf_.size();
    buf_.resize(at + n);
    std::memcpy(buf_.data() + at, p, n);
  }
  std::vector<uint8_t>& bytes() {
    return buf_;
  }

 private:
  // Compile-time length: the copy becomes one or two plain stores.
  template <size_t N>
  void fixed(const void* p, std::integral_constant<size_t, N>) {
    const size_t at = buf_.size();
    buf_.resize(at + N);
    std::memcpy(buf_.data() + at, p, N);
  }

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
  // Same as str() into an existing string (no temporary).
  void str(std::string* out) {
    uint32_t len = u32();
    if (!ok_ || len > n_ - off_) {
      ok_ = false;
      out->clear();
      return;
    }
    out->assign(reinterpret_cast<const char*>(p_ + off_), len);
    off_ += len;
  }
  size_t remaining() const {
    return n_ - off_;
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
