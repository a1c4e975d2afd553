#include <cstring>
#include <sstream>

#include <tensorpipe/common/error.h>
#include <tensorpipe/common/hip_api.h>
#include <tensorpipe/common/hip_buffer.h>

TP_AMD_NAMESPACE_BEGIN

const Error Error::kSuccess{};

std::string Error::what() const {
  if (!error_) {
    return "success";
  }
  std::ostringstream ss;
  ss << error_->what() << " (this error originated at " << file_ << ":" << line_ << ")";
  return ss.str();
}

std::string SystemError::what() const {
  std::ostringstream ss;
  ss << syscall_ << ": " << std::strerror(error_);
  return ss.str();
}

std::string ShortReadError::what() const {
  std::ostringstream ss;
  ss << "short read: got " << actual_ << " bytes while expecting to read " << expected_
     << " bytes";
  return ss.str();
}

std::string ShortWriteError::what() const {
  std::ostringstream ss;
  ss << "short write: wrote " << actual_ << " bytes while expecting to write " << expected_
     << " bytes";
  return ss.str();
}

std::string EOFError::what() const {
  return "eof";
}

std::string HipError::what() const {
  std::ostringstream ss;
  ss << call_ << ": [" << code_ << "] " << tphip_strerror(code_);
  return ss.str();
}

int hipDeviceCountNoThrow() {
  int count = 0;
  if (tphip_device_count(&count) != 0) {
    return 0;
  }
  return count;
}

int hipDeviceForPointer(const void* ptr) {
  // With a single visible GPU every device pointer belongs to device 0: skip
  // the driver query, which would otherwise run several times per tensor.
  static const int count = hipDeviceCountNoThrow();
  if (count == 1 && ptr != nullptr) {
    return 0;
  }
  int dev = -1;
  int isHost = 0;
  TP_HIP_CHECK(tphip_device_for_ptr(ptr, &dev, &isHost));
  return isHost ? -1 : dev;
}

Device HipBuffer::getDevice() const {
  int dev = hipDeviceForPointer(ptr);
  TP_THROW_ASSERT_IF(dev < 0);
  return Device{kHipDeviceType, dev};
}

TP_AMD_NAMESPACE_END
