// Errors of the host core. Each carries the kind of Python exception that the binding raises.
#pragma once
#include <stdexcept>
#include <string>

namespace dinfer {

enum ErrorKind : int {
    ERR_KEY = 1,      // unknown or duplicate request
    ERR_RUNTIME = 2,  // the state does not allow the call (no slot free, page not held, ...)
    ERR_VALUE = 3,    // an argument is out of range
    ERR_ASSERT = 4,   // an invariant is broken (reported by check())
};

struct Error : std::runtime_error {
    ErrorKind kind;
    Error(ErrorKind k, const std::string& what) : std::runtime_error(what), kind(k) {}
};

}  // namespace dinfer
