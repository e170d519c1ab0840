// Errors the host core raises towards its caller.
#pragma once

#include <stdexcept>

namespace mercury {

// Something about the device side went wrong: a kernel library that is missing or refuses
// its arguments, a program whose operations do not fit together, a workspace too small.
class KernelError : public std::runtime_error {
 public:
  using std::runtime_error::runtime_error;
};

}  // namespace mercury
