// Turns the operators' exceptions into the C ABI's status codes.
#pragma once
#include "backend/Internal.hpp"
#include "hip/Backend.hpp"

#include <new>
#include <stdexcept>

namespace splash::capi {

inline void require(bool present, const char *what) {
  if (!present) throw std::invalid_argument(std::string("null ") + what);
}

template <class Body> sp_status guard(Body body) noexcept {
  try {
    body();
    return SP_OK;
  } catch (const std::invalid_argument &e) {
    hipbackend::setLastError(e.what());
    return SP_INVALID_ARGUMENT;
  } catch (const hip::BackendError &e) {
    hipbackend::setLastError(e.what());
    return SP_BACKEND_ERROR;
  } catch (const std::bad_alloc &) {
    hipbackend::setLastError("out of host memory");
    return SP_OUT_OF_MEMORY;
  } catch (const std::exception &e) {
    hipbackend::setLastError(e.what());
    return SP_BACKEND_ERROR;
  }
}

} // namespace splash::capi
