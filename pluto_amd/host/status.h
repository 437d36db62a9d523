// Minimal Status / StatusOr / Span used by the host-side mirror of the
// reference's layer API.  The reference uses Abseil's types of the same names
// (absl::Status, absl::StatusOr, absl::Span); Abseil is not available where
// this library is built, so these carry exactly the subset the attention path
// uses: the canonical error codes, message(), ok(), value access and the two
// propagation macros of src/util/status_macros.h:11-39.  No exceptions.
#pragma once

#include <cstddef>
#include <cstdlib>
#include <initializer_list>
#include <iostream>
#include <optional>
#include <string>
#include <string_view>
#include <type_traits>
#include <utility>
#include <vector>

namespace pluto {

enum class StatusCode {
  kOk = 0,
  kCancelled = 1,
  kInvalidArgument = 3,
  kResourceExhausted = 8,
  kFailedPrecondition = 9,
  kUnimplemented = 12,
  kInternal = 13,
};

class [[nodiscard]] Status {
 public:
  Status() = default;
  Status(StatusCode code, std::string message) : code_(code), message_(std::move(message)) {}
  bool ok() const { return code_ == StatusCode::kOk; }
  StatusCode code() const { return code_; }
  std::string_view message() const { return message_; }
  std::string ToString() const;

 private:
  StatusCode code_ = StatusCode::kOk;
  std::string message_;
};

inline Status OkStatus() { return Status(); }
inline Status CancelledError(std::string m) { return {StatusCode::kCancelled, std::move(m)}; }
inline Status InvalidArgumentError(std::string m) { return {StatusCode::kInvalidArgument, std::move(m)}; }
inline Status ResourceExhaustedError(std::string m) { return {StatusCode::kResourceExhausted, std::move(m)}; }
inline Status UnimplementedError(std::string m) { return {StatusCode::kUnimplemented, std::move(m)}; }
inline Status InternalError(std::string m) { return {StatusCode::kInternal, std::move(m)}; }
inline Status FailedPreconditionError(std::string m) { return {StatusCode::kFailedPrecondition, std::move(m)}; }
inline bool IsInvalidArgument(const Status& s) { return s.code() == StatusCode::kInvalidArgument; }
inline bool IsResourceExhausted(const Status& s) { return s.code() == StatusCode::kResourceExhausted; }
inline bool IsUnimplemented(const Status& s) { return s.code() == StatusCode::kUnimplemented; }
inline bool IsFailedPrecondition(const Status& s) { return s.code() == StatusCode::kFailedPrecondition; }

inline const char* StatusCodeName(StatusCode code) {
  switch (code) {
    case StatusCode::kOk: return "OK";
    case StatusCode::kCancelled: return "CANCELLED";
    case StatusCode::kInvalidArgument: return "INVALID_ARGUMENT";
    case StatusCode::kResourceExhausted: return "RESOURCE_EXHAUSTED";
    case StatusCode::kFailedPrecondition: return "FAILED_PRECONDITION";
    case StatusCode::kUnimplemented: return "UNIMPLEMENTED";
    case StatusCode::kInternal: return "INTERNAL";
  }
  return "UNKNOWN";
}

inline std::string Status::ToString() const {
  if (ok()) return "OK";
  return std::string(StatusCodeName(code_)) + ": " + message_;
}

inline std::ostream& operator<<(std::ostream& os, const Status& s) { return os << s.ToString(); }

// Concatenates streamable pieces (the subset of absl::StrCat the path needs).
template <class... Pieces>
std::string StrCat(const Pieces&... pieces) {
  std::string out;
  auto add = [&out](const auto& piece) {
    using T = std::decay_t<decltype(piece)>;
    if constexpr (std::is_arithmetic_v<T>)
      out += std::to_string(piece);
    else
      out += std::string_view(piece);
  };
  (add(pieces), ...);
  return out;
}

template <class T>
class [[nodiscard]] StatusOr {
 public:
  StatusOr(Status status) : status_(std::move(status)) {  // NOLINT: implicit by design
    if (status_.ok()) status_ = InternalError("StatusOr constructed from OK without a value");
  }
  StatusOr(T value) : value_(std::move(value)) {}  // NOLINT: implicit by design
  template <class U, class = std::enable_if_t<std::is_constructible_v<T, U&&> &&
                                               !std::is_same_v<std::decay_t<U>, StatusOr> &&
                                               !std::is_same_v<std::decay_t<U>, Status> &&
                                               !std::is_same_v<std::decay_t<U>, T>>>
  StatusOr(U&& value) : value_(std::forward<U>(value)) {}  // NOLINT

  bool ok() const { return status_.ok(); }
  const Status& status() const { return status_; }
  T& value() & { Check(); return *value_; }
  const T& value() const& { Check(); return *value_; }
  T&& value() && { Check(); return std::move(*value_); }
  T& operator*() & { return value(); }
  const T& operator*() const& { return value(); }
  T&& operator*() && { return std::move(*this).value(); }
  T* operator->() { return &value(); }
  const T* operator->() const { return &value(); }

 private:
  void Check() const {
    if (!status_.ok()) {  // same policy as the reference build: no exceptions
      std::cerr << "StatusOr::value() on error: " << status_ << std::endl;
      std::abort();
    }
  }
  Status status_;
  std::optional<T> value_;
};

// Non-owning view of contiguous elements (subset of absl::Span).
template <class T>
class Span {
 public:
  using value_type = std::remove_cv_t<T>;
  Span() = default;
  Span(T* data, size_t size) : data_(data), size_(size) {}
  template <class V, class = std::enable_if_t<std::is_const_v<T> &&
                                               std::is_same_v<std::remove_cv_t<V>, value_type>>>
  Span(Span<V> other) : data_(other.data()), size_(other.size()) {}  // NOLINT
  template <size_t N>
  Span(T (&array)[N]) : data_(array), size_(N) {}  // NOLINT
  template <class V = T, class = std::enable_if_t<std::is_const_v<V>>>
  Span(const std::vector<value_type>& v) : data_(v.data()), size_(v.size()) {}  // NOLINT
  template <class V = T, class = std::enable_if_t<!std::is_const_v<V>>>
  Span(std::vector<value_type>& v) : data_(v.data()), size_(v.size()) {}  // NOLINT
  template <class V = T, class = std::enable_if_t<std::is_const_v<V>>>
  Span(std::initializer_list<value_type> list) : data_(list.begin()), size_(list.size()) {}  // NOLINT

  T* data() const { return data_; }
  size_t size() const { return size_; }
  bool empty() const { return size_ == 0; }
  T& operator[](size_t i) const { return data_[i]; }
  T* begin() const { return data_; }
  T* end() const { return data_ + size_; }
  T& front() const { return data_[0]; }

 private:
  T* data_ = nullptr;
  size_t size_ = 0;
};

template <class T>
Span<T> MakeSpan(std::vector<T>& v) { return Span<T>(v.data(), v.size()); }
template <class T>
Span<const T> MakeConstSpan(const std::vector<T>& v) { return Span<const T>(v.data(), v.size()); }

}  // namespace pluto

// src/util/status_macros.h:11-39
#define RETURN_IF_ERROR(expression)                                 \
  do {                                                              \
    ::pluto::Status pluto_status_macro_status = (expression);       \
    if (__builtin_expect(!pluto_status_macro_status.ok(), 0)) {     \
      return pluto_status_macro_status;                             \
    }                                                               \
  } while (false)

#define PLUTO_STATUS_CONCAT_INNER_(left, right) left##right
#define PLUTO_STATUS_CONCAT_(left, right) PLUTO_STATUS_CONCAT_INNER_(left, right)
#define PLUTO_ASSIGN_OR_RETURN_(status_or, lhs, expression)  \
  auto status_or = (expression);                             \
  if (__builtin_expect(!status_or.ok(), 0)) {                \
    return status_or.status();                               \
  }                                                          \
  lhs = std::move(status_or).value()
#define ASSIGN_OR_RETURN(lhs, expression) \
  PLUTO_ASSIGN_OR_RETURN_(PLUTO_STATUS_CONCAT_(pluto_status_or_, __COUNTER__), lhs, expression)
