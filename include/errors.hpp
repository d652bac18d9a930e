// Exception type for unimplemented template branches.
// Same role as the reference's include/errors.hpp:8-19.
#pragma once

#include <stdexcept>
#include <string>

namespace tiledcuda::errors {

class NotImplementedException : public std::logic_error {
  public:
    explicit NotImplementedException(const std::string& what = "")
        : std::logic_error("Not implemented yet: " + what) {}
};

}  // namespace tiledcuda::errors
