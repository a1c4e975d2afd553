#pragma once

#include <optional>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN
// The reference vendors an optional for C++14 (tensorpipe/common/optional.h);
// this build is C++17.
template <typename T>
using optional = std::optional<T>;
using std::nullopt;
TP_AMD_NAMESPACE_END
