// Type-erased, non-owning tensor handle: a small-buffer wrapper around any
// trivially copyable buffer struct that has getDevice(). Same contract as
// tensorpipe/common/buffer.h:21-133 (32 bytes, 8-aligned, unwrap<T>() throws
// std::runtime_error on a type mismatch).
#pragma once

#include <cstddef>
#include <cstdint>
#include <new>
#include <stdexcept>
#include <type_traits>
#include <utility>

#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/device.h>

TP_AMD_NAMESPACE_BEGIN

namespace buffer_detail {
// T::getDeviceKey() where a buffer type has one, 0 ("ask getDevice()") otherwise.
template <typename T>
auto deviceKeyOf(const T& v, int) -> decltype(v.getDeviceKey()) {
  return v.getDeviceKey();
}
template <typename T>
uint32_t deviceKeyOf(const T&, long) {
  return 0;
}
} // namespace buffer_detail

class Buffer {
  struct Concept {
    virtual Device device() const = 0;
    virtual void cloneInto(void* where) const = 0;
    virtual uint32_t deviceKey() const = 0;
    virtual ~Concept() = default;
  };

  template <typename T>
  struct Model final : Concept {
    static_assert(std::is_trivially_copyable<T>::value, "wrapping non-trivially copyable class");
    T value;
    explicit Model(T v) : value(std::move(v)) {}
    Device device() const override {
      return value.getDevice();
    }
    void cloneInto(void* where) const override {
      new (where) Model(*this);
    }
    uint32_t deviceKey() const override {
      return buffer_detail::deviceKeyOf(value, 0);
    }
  };

 public:
  template <
      typename T,
      typename = typename std::enable_if<!std::is_same<typename std::decay<T>::type, Buffer>::value>::type>
  /* implicit */ Buffer(T b) {
    static_assert(sizeof(Model<T>) <= kStructSize, "kStructSize too small");
    static_assert(alignof(Model<T>) <= kStructAlign, "kStructAlign too small");
    new (&raw_) Model<T>(std::move(b));
  }

  Buffer() : Buffer(CpuBuffer{}) {}

  Buffer(const Buffer& other) {
    other.self()->cloneInto(&raw_);
  }

  Buffer& operator=(const Buffer& other) {
    if (this != &other) {
      self()->~Concept();
      other.self()->cloneInto(&raw_);
    }
    return *this;
  }

  ~Buffer() {
    self()->~Concept();
  }

  template <typename T>
  T& unwrap() {
    auto* m = dynamic_cast<Model<T>*>(self());
    if (m == nullptr) {
      throw std::runtime_error("Invalid unwrapping of tensorpipe::Buffer");
    }
    return m->value;
  }

  template <typename T>
  const T& unwrap() const {
    auto* m = dynamic_cast<const Model<T>*>(self());
    if (m == nullptr) {
      throw std::runtime_error("Invalid unwrapping of tensorpipe::Buffer");
    }
    return m->value;
  }

  Device device() const {
    return self()->device();
  }

  // Not in the reference: a small number that is equal for two buffers exactly
  // when their devices are equal, or 0 where the buffer's type cannot say
  // without building the Device. Lets a loop over the tensors of a message
  // build and compare a Device (a string and an index) once per run of equal
  // devices instead of once per tensor.
  uint32_t deviceKey() const {
    return self()->deviceKey();
  }

 private:
  static constexpr int kStructSize = 32;
  static constexpr int kStructAlign = 8;
  alignas(kStructAlign) unsigned char raw_[kStructSize];

  const Concept* self() const {
    return std::launder(reinterpret_cast<const Concept*>(&raw_));
  }
  Concept* self() {
    return std::launder(reinterpret_cast<Concept*>(&raw_));
  }
};

TP_AMD_NAMESPACE_END
