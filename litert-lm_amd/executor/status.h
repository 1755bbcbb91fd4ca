// Minimal stand-ins for absl::Status / absl::StatusOr and for the reference's
// status macros, so that this layer builds without abseil. Codes are the
// absl::StatusCode values; RET_CHECK defaults to kInternal and accepts
// .SetCode(), as in the reference (runtime/util/status_macros.h:15-62). When
// the executor is built inside the reference tree these aliases are replaced
// by the real absl types.
#ifndef LITERT_LM_AMD_EXECUTOR_STATUS_H_
#define LITERT_LM_AMD_EXECUTOR_STATUS_H_

#include <optional>
#include <sstream>
#include <string>
#include <string_view>
#include <utility>

namespace litert::lm {

// absl::string_view inside the reference tree (an alias of std::string_view in current abseil builds).
using string_view = std::string_view;

enum class StatusCode : int {
  kOk = 0,
  kCancelled = 1,
  kInvalidArgument = 3,
  kNotFound = 5,
  kAlreadyExists = 6,
  kResourceExhausted = 8,
  kFailedPrecondition = 9,
  kOutOfRange = 11,
  kUnimplemented = 12,
  kInternal = 13,
  kUnavailable = 14,
};

class Status {
 public:
  Status() = default;
  Status(StatusCode code, std::string message) : code_(code), message_(std::move(message)) {}
  bool ok() const { return code_ == StatusCode::kOk; }
  StatusCode code() const { return code_; }
  const std::string& message() const { return message_; }

 private:
  StatusCode code_ = StatusCode::kOk;
  std::string message_;
};

inline Status OkStatus() { return Status(); }
inline Status CancelledError(std::string m) { return Status(StatusCode::kCancelled, std::move(m)); }
inline Status InvalidArgumentError(std::string m) { return Status(StatusCode::kInvalidArgument, std::move(m)); }
inline Status InternalError(std::string m) { return Status(StatusCode::kInternal, std::move(m)); }
inline Status UnimplementedError(std::string m) { return Status(StatusCode::kUnimplemented, std::move(m)); }
inline Status FailedPreconditionError(std::string m) { return Status(StatusCode::kFailedPrecondition, std::move(m)); }
inline Status AlreadyExistsError(std::string m) { return Status(StatusCode::kAlreadyExists, std::move(m)); }
inline Status NotFoundError(std::string m) { return Status(StatusCode::kNotFound, std::move(m)); }
inline Status OutOfRangeError(std::string m) { return Status(StatusCode::kOutOfRange, std::move(m)); }
inline Status UnavailableError(std::string m) { return Status(StatusCode::kUnavailable, std::move(m)); }
inline Status ResourceExhaustedError(std::string m) { return Status(StatusCode::kResourceExhausted, std::move(m)); }

template <class T>
class StatusOr {
 public:
  StatusOr(Status s) : status_(std::move(s)) {}  // NOLINT: implicit like absl
  StatusOr(T v) : value_(std::move(v)) {}        // NOLINT
  bool ok() const { return status_.ok(); }
  const Status& status() const { return status_; }
  T& operator*() { return *value_; }
  const T& operator*() const { return *value_; }
  T* operator->() { return &*value_; }
  T& value() { return *value_; }
  const T& value() const { return *value_; }

 private:
  Status status_;
  std::optional<T> value_;
};

namespace internal {
class StreamToStatus {
 public:
  explicit StreamToStatus(const char* what) { stream_ << what << ": "; }
  StreamToStatus& SetCode(StatusCode c) {
    code_ = c;
    return *this;
  }
  template <class T>
  StreamToStatus& operator<<(const T& v) {
    stream_ << v;
    return *this;
  }
  operator Status() const { return Status(code_, stream_.str()); }  // NOLINT
  template <class T>
  operator StatusOr<T>() const { return Status(code_, stream_.str()); }  // NOLINT

 private:
  StatusCode code_ = StatusCode::kInternal;
  std::ostringstream stream_;
};
}  // namespace internal

}  // namespace litert::lm

#define LM_CONCAT_INNER(a, b) a##b
#define LM_CONCAT(a, b) LM_CONCAT_INNER(a, b)
#define RETURN_IF_ERROR(expr) \
  if (auto lm_status_ = (expr); !lm_status_.ok()) return lm_status_
#define ASSIGN_OR_RETURN(decl, expr) LM_ASSIGN_OR_RETURN_IMPL(LM_CONCAT(lm_statusor_, __LINE__), decl, expr)
#define LM_ASSIGN_OR_RETURN_IMPL(tmp, decl, expr) \
  auto&& tmp = (expr);                            \
  if (!tmp.ok()) return tmp.status();             \
  decl = std::move(*tmp)
#define RET_CHECK(cond) \
  if (!(cond)) return ::litert::lm::internal::StreamToStatus(#cond)
#define RET_CHECK_EQ(a, b) RET_CHECK((a) == (b))
#define RET_CHECK_GT(a, b) RET_CHECK((a) > (b))
#define RET_CHECK_GE(a, b) RET_CHECK((a) >= (b))
#define RET_CHECK_LE(a, b) RET_CHECK((a) <= (b))

#endif  // LITERT_LM_AMD_EXECUTOR_STATUS_H_
