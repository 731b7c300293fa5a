// Error values of the MI355X host layer. Codes and their meaning follow
// glow::ErrorValue::ErrorCode (reference include/glow/Support/Error.h:292-337);
// inside a Glow build these map one-to-one onto MAKE_ERR(code, msg).
#ifndef GLOW_MI355X_HOST_ERROR_H
#define GLOW_MI355X_HOST_ERROR_H

#include <memory>
#include <string>
#include <utility>

namespace glow_mi355x {

enum class ErrorCode {
  SUCCESS = 0,
  UNKNOWN,
  RUNTIME_ERROR,
  RUNTIME_OUT_OF_DEVICE_MEMORY,
  RUNTIME_NET_NOT_FOUND,
  RUNTIME_REQUEST_REFUSED,
  RUNTIME_DEVICE_NOT_FOUND,
  RUNTIME_DEVICE_NONRECOVERABLE,
  RUNTIME_NET_BUSY,
  DEVICE_FEATURE_NOT_SUPPORTED,
  COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE,
  COMPILE_CONTEXT_MALFORMED,
};

const char *errorCodeName(ErrorCode c);

// Success or (code, message). Unlike glow::Error it may be dropped unchecked.
class Error {
public:
  Error() = default;
  Error(ErrorCode code, std::string msg) : code_(code), msg_(std::move(msg)) {}
  static Error success() { return Error(); }
  explicit operator bool() const { return code_ != ErrorCode::SUCCESS; } // true = failed
  ErrorCode code() const { return code_; }
  const std::string &message() const { return msg_; }
  std::string str() const;

private:
  ErrorCode code_ = ErrorCode::SUCCESS;
  std::string msg_;
};

template <typename T> class Expected {
public:
  Expected(T v) : val_(std::move(v)) {}
  Expected(Error e) : err_(std::move(e)) {}
  explicit operator bool() const { return !err_; } // true = has a value
  T &get() { return val_; }
  T &operator*() { return val_; }
  T *operator->() { return &val_; }
  Error takeError() { return std::move(err_); }
  const Error &error() const { return err_; }

private:
  T val_{};
  Error err_;
};

std::string strFormat(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define MI355X_MAKE_ERR(code, ...)                                             \
  ::glow_mi355x::Error((code), ::glow_mi355x::strFormat(__VA_ARGS__))

#define MI355X_RETURN_IF_ERR(expr)                                             \
  do {                                                                         \
    ::glow_mi355x::Error e__ = (expr);                                         \
    if (e__) return e__;                                                       \
  } while (0)

} // namespace glow_mi355x
#endif
