// Error types of the host surface.
//
// DeviceError mirrors cuda-async/src/error.rs:12-33 (variants Driver, Context,
// KernelCache, Scheduling, Launch, Internal) plus the tensor/shape category of
// cutile/src/error.rs:43-56.  Result<T> stands in for Rust's
// Result<T, DeviceError>: operations return it instead of throwing, and
// .unwrap() throws like a Rust unwrap() panics.  Conditions the reference
// treats as programmer errors (panics) throw std::logic_error here.
#pragma once
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <variant>

#include "../cutile_hip.h"

namespace cutile {

struct DeviceError {
  enum class Kind { Driver, Context, KernelCache, Scheduling, Launch, Internal, Tensor };
  Kind kind = Kind::Internal;
  int code = 0;  // hipError_t for Driver, library status otherwise
  std::string message;

  const char* kind_name() const {
    switch (kind) {
      case Kind::Driver: return "Driver";
      case Kind::Context: return "Context";
      case Kind::KernelCache: return "KernelCache";
      case Kind::Scheduling: return "Scheduling";
      case Kind::Launch: return "Launch";
      case Kind::Tensor: return "Tensor";
      default: return "Internal";
    }
  }
  std::string to_string() const { return std::string(kind_name()) + "(" + message + ")"; }

  static DeviceError launch(std::string m) { return {Kind::Launch, CUTILE_ERR_KERNEL_LAUNCH, std::move(m)}; }
  static DeviceError internal(std::string m) { return {Kind::Internal, CUTILE_ERR_STATE, std::move(m)}; }
  static DeviceError tensor(std::string m) { return {Kind::Tensor, CUTILE_ERR_TENSOR, std::move(m)}; }
  static DeviceError scheduling(std::string m) { return {Kind::Scheduling, CUTILE_ERR_STATE, std::move(m)}; }

  // The calling thread's last C-ABI failure as a DeviceError.
  static DeviceError from_status(cutile_status_t s) {
    DeviceError e;
    e.code = s;
    e.message = cutile_last_error_message();
    if (s > 0 || s == CUTILE_ERR_LIBRARY_INIT)
      e.kind = Kind::Driver;
    else if (s == CUTILE_ERR_KERNEL_NOT_FOUND)
      e.kind = Kind::KernelCache;
    else if (s == CUTILE_ERR_KERNEL_LAUNCH)
      e.kind = Kind::Launch;
    else if (s == CUTILE_ERR_TENSOR)
      e.kind = Kind::Tensor;
    else
      e.kind = Kind::Internal;
    return e;
  }
};

struct Unit {};  // Rust's ()

template <class T>
class Result {
 public:
  Result(T v) : v_(std::in_place_index<0>, std::move(v)) {}
  Result(DeviceError e) : v_(std::in_place_index<1>, std::move(e)) {}
  bool is_ok() const { return v_.index() == 0; }
  bool is_err() const { return v_.index() == 1; }
  explicit operator bool() const { return is_ok(); }
  T& value() & { return std::get<0>(v_); }
  const T& value() const& { return std::get<0>(v_); }
  T&& value() && { return std::get<0>(std::move(v_)); }
  const DeviceError& error() const { return std::get<1>(v_); }
  T unwrap() && {
    if (is_err()) throw std::runtime_error("called unwrap() on an error: " + error().to_string());
    return std::get<0>(std::move(v_));
  }
  T unwrap() & { return std::move(*this).unwrap(); }
  template <class F>
  auto map(F&& f) && -> Result<decltype(f(std::declval<T>()))> {
    if (is_err()) return error();
    return f(std::get<0>(std::move(v_)));
  }

 private:
  std::variant<T, DeviceError> v_;
};

inline Result<Unit> ok() { return Unit{}; }
inline Result<Unit> check(cutile_status_t s) {
  if (s == CUTILE_SUCCESS) return Unit{};
  return DeviceError::from_status(s);
}

#define CUTILE_TRY(expr)                                  \
  do {                                                    \
    auto _r = (expr);                                     \
    if (_r.is_err()) return _r.error();                   \
  } while (0)

#define CUTILE_TRY_STATUS(expr)                                       \
  do {                                                                \
    cutile_status_t _s = (expr);                                      \
    if (_s != CUTILE_SUCCESS) return ::cutile::DeviceError::from_status(_s); \
  } while (0)

}  // namespace cutile
