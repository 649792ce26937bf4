// Error-as-value plumbing and the environment-driven logger of the graph API.
//
// Mirrors the conventions of the reference (support/logging.h:58-292,
// 383-471): every fallible call returns ErrorObject or ErrorOr<T>, both
// [[nodiscard]]; no exceptions.  Logging is off unless FUSILLI_LOG_INFO is set;
// FUSILLI_LOG_FILE chooses stdout, stderr or a file path.
#ifndef FUSILLI_ERRORS_H
#define FUSILLI_ERRORS_H

#include <cassert>
#include <cstdint>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <memory>
#include <ostream>
#include <string>
#include <type_traits>
#include <utility>
#include <variant>

namespace fusilli {

enum class [[nodiscard]] ErrorCode : uint8_t {
  OK,
  NotImplemented,
  NotValidated,
  NotCompiled,
  AttributeNotSet,
  InternalError,
  InvalidAttribute,
  InvalidArgument,
  VariantPackError,
  CompileFailure,
  RuntimeFailure,
  FileSystemFailure,
};

inline const char *errorCodeName(ErrorCode c) {
  switch (c) {
  case ErrorCode::OK:
    return "OK";
  case ErrorCode::NotImplemented:
    return "NOT_IMPLEMENTED";
  case ErrorCode::NotValidated:
    return "NOT_VALIDATED";
  case ErrorCode::NotCompiled:
    return "NOT_COMPILED";
  case ErrorCode::AttributeNotSet:
    return "ATTRIBUTE_NOT_SET";
  case ErrorCode::InternalError:
    return "INTERNAL_ERROR";
  case ErrorCode::InvalidAttribute:
    return "INVALID_ATTRIBUTE";
  case ErrorCode::InvalidArgument:
    return "INVALID_ARGUMENT";
  case ErrorCode::VariantPackError:
    return "VARIANT_PACK_ERROR";
  case ErrorCode::CompileFailure:
    return "COMPILE_FAILURE";
  case ErrorCode::RuntimeFailure:
    return "RUNTIME_FAILURE";
  case ErrorCode::FileSystemFailure:
    return "FILE_SYSTEM_FAILURE";
  }
  return "UNKNOWN_ERROR_CODE";
}

struct [[nodiscard]] ErrorObject {
  ErrorCode code = ErrorCode::OK;
  std::string errMsg;

  ErrorObject() = default;
  ErrorObject(ErrorCode c, std::string msg) : code(c), errMsg(std::move(msg)) {}

  ErrorCode getCode() const { return code; }
  const std::string &getMessage() const { return errMsg; }
  bool isOk() const { return code == ErrorCode::OK; }
  bool isError() const { return !isOk(); }
  bool operator==(ErrorCode other) const { return code == other; }
  bool operator!=(ErrorCode other) const { return code != other; }
};

inline bool isOk(const ErrorObject &e) { return e.isOk(); }
inline bool isError(const ErrorObject &e) { return e.isError(); }
inline ErrorObject ok() { return {}; }
inline ErrorObject error(ErrorCode code, std::string msg) {
  return ErrorObject(code, std::move(msg));
}

// Either a T or the error that prevented producing it.  Move-only.
template <typename T> class [[nodiscard]] ErrorOr {
public:
  template <typename U>
    requires(std::is_constructible_v<T, U &&> &&
             !std::is_same_v<std::decay_t<U>, ErrorObject> &&
             !std::is_same_v<std::decay_t<U>, ErrorOr<T>>)
  ErrorOr(U &&value) : state_(std::in_place_index<0>, std::forward<U>(value)) {}

  ErrorOr(ErrorObject err) : state_(std::in_place_index<1>, std::move(err)) {
    assert(std::get<1>(state_).isError() &&
           "an ErrorOr built from an ErrorObject must hold an error");
  }

  template <typename U>
    requires std::is_constructible_v<T, U>
  ErrorOr(ErrorOr<U> &&other)
      : state_(other.hasValue()
                   ? State(std::in_place_index<0>, std::move(*other))
                   : State(std::in_place_index<1>, ErrorObject(other))) {}

  ErrorOr(ErrorOr &&) noexcept = default;
  ErrorOr(const ErrorOr &) = delete;
  ErrorOr &operator=(const ErrorOr &) = delete;
  ErrorOr &operator=(ErrorOr &&) = delete;

  operator ErrorObject() const {
    return hasValue() ? ok() : std::get<1>(state_);
  }

  T &operator*() { return value(); }
  const T &operator*() const { return value(); }
  T *operator->() { return &value(); }
  const T *operator->() const { return &value(); }

  bool hasValue() const noexcept { return state_.index() == 0; }

private:
  using State = std::variant<T, ErrorObject>;
  State state_;

  T &value() {
    dieIfError();
    return std::get<0>(state_);
  }
  const T &value() const {
    dieIfError();
    return std::get<0>(state_);
  }
  void dieIfError() const {
    if (!hasValue()) [[unlikely]] {
      std::cerr << "ErrorOr<T> dereferenced while holding an error ("
                << errorCodeName(std::get<1>(state_).code) << ": "
                << std::get<1>(state_).errMsg
                << "); check isOk()/isError() first" << std::endl;
      std::abort();
    }
  }
  template <typename U> friend class ErrorOr;
};

template <typename T> bool isOk(const ErrorOr<T> &e) { return e.hasValue(); }
template <typename T> bool isError(const ErrorOr<T> &e) {
  return !e.hasValue();
}
template <typename T> auto ok(T &&value) {
  return ErrorOr<std::decay_t<T>>(std::forward<T>(value));
}

inline std::ostream &operator<<(std::ostream &os, const ErrorCode &c) {
  return os << errorCodeName(c);
}
inline std::ostream &operator<<(std::ostream &os, const ErrorObject &e) {
  return os << e.getCode() << ": " << e.getMessage();
}

// ---- logger ---------------------------------------------------------------
inline bool &isLoggingEnabled() {
  static bool enabled = [] {
    const char *v = std::getenv("FUSILLI_LOG_INFO");
    return v && std::string(v) != "0" && std::string(v) != "";
  }();
  return enabled;
}

class NullStream : public std::ostream {
  class NullBuf : public std::streambuf {
    int overflow(int c) override { return c; }
  } buf_;

public:
  NullStream() : std::ostream(&buf_) {}
};

inline std::ostream &getStream() {
  static std::ofstream file;
  static std::ostream *chosen = [] () -> std::ostream * {
    const char *v = std::getenv("FUSILLI_LOG_FILE");
    if (!v)
      return &std::cout; // enabled but no file named
    const std::string s(v);
    if (s == "stdout")
      return &std::cout;
    if (s == "stderr")
      return &std::cerr;
    file.open(s, std::ios::out);
    return file.is_open() ? static_cast<std::ostream *>(&file) : &std::cout;
  }();
  return *chosen;
}

inline std::ostream &getLogger() {
  static NullStream null;
  return isLoggingEnabled() ? getStream() : null;
}

} // namespace fusilli

#define FUSILLI_LOG(X) fusilli::getLogger() << X
#define FUSILLI_LOG_ENDL(X) fusilli::getLogger() << X << std::endl
#define FUSILLI_LOG_LABEL_ENDL(X)                                              \
  fusilli::getLogger() << "[FUSILLI] " << X << std::endl
#define FUSILLI_LOG_LABEL_RED(X)                                               \
  fusilli::getLogger() << "\033[31m[FUSILLI] " << X << "\033[0m"

// Returns error(code, message) from the enclosing function when cond holds.
#define FUSILLI_RETURN_ERROR_IF(cond, code, message)                           \
  do {                                                                         \
    if (cond) {                                                                \
      FUSILLI_LOG_LABEL_RED("ERROR: ");                                        \
      FUSILLI_LOG_ENDL(code << ": " << message << ": (" #cond ") at "          \
                            << __FILE__ << ":" << __LINE__);                   \
      return fusilli::error(code, message);                                    \
    }                                                                          \
  } while (false)

// Propagates a failed ErrorObject / ErrorOr out of the enclosing function.
#define FUSILLI_CHECK_ERROR(expr)                                              \
  do {                                                                         \
    fusilli::ErrorObject fusilliErr_ = (expr);                                 \
    if (fusilli::isError(fusilliErr_)) {                                       \
      FUSILLI_LOG_LABEL_RED("ERROR: " << fusilliErr_ << " ");                  \
      FUSILLI_LOG_ENDL(#expr << " at " << __FILE__ << ":" << __LINE__);        \
      return fusilliErr_;                                                      \
    }                                                                          \
  } while (false)

#define FUSILLI_CONCAT_INNER(a, b) a##b
#define FUSILLI_CONCAT2(a, b) FUSILLI_CONCAT_INNER(a, b)
#define FUSILLI_ASSIGN_OR_RETURN_AT(tmp, decl, expr)                           \
  auto tmp = (expr);                                                           \
  if (fusilli::isError(tmp)) {                                                 \
    FUSILLI_LOG_LABEL_RED("ERROR: " << fusilli::ErrorObject(tmp) << " ");      \
    FUSILLI_LOG_ENDL(#expr << " at " << __FILE__ << ":" << __LINE__);          \
    return fusilli::ErrorObject(tmp);                                          \
  }                                                                            \
  decl = std::move(*tmp);
// `decl` is a declaration or an lvalue: FUSILLI_ASSIGN_OR_RETURN(auto x, f());
#define FUSILLI_ASSIGN_OR_RETURN(decl, expr)                                   \
  FUSILLI_ASSIGN_OR_RETURN_AT(FUSILLI_CONCAT2(fusilliErrorOr_, __LINE__), decl, \
                              expr)

#endif // FUSILLI_ERRORS_H
