// Error convention of the host layer (rocAL/include/pipeline/exception.h:28-39): internals throw a
// RocalException carrying "function: message"; the API layer catches, stores the text in the context,
// prints it to stderr and returns nullptr / ROCAL_RUNTIME_ERROR.
#pragma once
#include <exception>
#include <sstream>
#include <string>

class RocalException : public std::exception {
   public:
    explicit RocalException(const std::string &message) : _message(message) {}
    const char *what() const noexcept override { return _message.c_str(); }

   private:
    std::string _message;
};

template <typename T>
inline std::string TOSTR(const T &v) {
    std::ostringstream s;
    s << v;
    return s.str();
}

#define THROW(X) throw RocalException(std::string(__func__) + ": " + (X));
