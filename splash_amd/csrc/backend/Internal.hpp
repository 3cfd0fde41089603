// Shared by the translation units of libsplash_hip.so; not part of the C ABI.
#pragma once
#include <string>

namespace splash::hipbackend {
// Sets the calling thread's sp_last_error() message.
void setLastError(const std::string &message);
} // namespace splash::hipbackend
