// Test-only stand-in for xla/ffi/api/ffi.h.
//
// This is NOT XLA's header and holds none of its source: it declares, from the public description of the XLA FFI
// C++ binding API, just the names the handlers in ejkernel_amd/csrc/rpa_xla_ffi.cc use, so that the file can be
// type-checked where jaxlib (which ships the real header) is not installed.  Two things are checked by compiling
// against it: the handlers are well-formed C++ against that API surface, and every XLA_FFI_DEFINE_HANDLER_SYMBOL binding
// lists exactly the context, operands, results and attributes its implementation function takes, in order
// (Binding::To static_asserts that the function is callable with the bound types).  It proves nothing about the real
// header beyond that; nothing here can execute a handler.
#pragma once

#include <cstddef>
#include <cstdint>
#include <optional>
#include <string>
#include <type_traits>
#include <utility>

namespace xla::ffi {

enum DataType { PRED, S8, S16, S32, S64, U8, U16, U32, U64, F16, F32, F64, BF16, F8E5M2, F8E4M3FN };
enum class ErrorCode { kOk, kCancelled, kUnknown, kInvalidArgument, kInternal, kUnimplemented };

class Error {
 public:
  Error() = default;
  Error(ErrorCode code, std::string message) : code_(code), message_(std::move(message)) {}
  static Error Success() { return Error(); }
  bool success() const { return code_ == ErrorCode::kOk; }
  bool failure() const { return !success(); }
  const std::string& message() const { return message_; }

 private:
  ErrorCode code_ = ErrorCode::kOk;
  std::string message_;
};

template <typename T>
class Span {
 public:
  Span(const T* data, size_t size) : data_(data), size_(size) {}
  size_t size() const { return size_; }
  const T& operator[](size_t i) const { return data_[i]; }
  const T& back() const { return data_[size_ - 1]; }
  const T* begin() const { return data_; }
  const T* end() const { return data_ + size_; }

 private:
  const T* data_;
  size_t size_;
};

class AnyBuffer {
 public:
  void* untyped_data() const { return nullptr; }
  Span<int64_t> dimensions() const { return Span<int64_t>(nullptr, 0); }
  DataType element_type() const { return F32; }
  size_t element_count() const { return 0; }
  size_t size_bytes() const { return 0; }
};

template <DataType dtype> struct NativeType;
template <> struct NativeType<S32> { using type = int32_t; };
template <> struct NativeType<F32> { using type = float; };
template <> struct NativeType<BF16> { using type = uint16_t; };

template <DataType dtype>
class Buffer {
 public:
  typename NativeType<dtype>::type* typed_data() const { return nullptr; }
  void* untyped_data() const { return nullptr; }
  Span<int64_t> dimensions() const { return Span<int64_t>(nullptr, 0); }
  size_t element_count() const { return 0; }
};

template <typename T>
class Result {
 public:
  T* operator->() { return &value_; }
  T& operator*() { return value_; }

 private:
  T value_;
};

class RemainingArgs {
 public:
  size_t size() const { return 0; }
  template <typename T>
  std::optional<T> get(size_t) const { return std::nullopt; }  // the real one returns an ErrorOr<T>: has_value(), ->
};

template <typename T> struct PlatformStream {};

namespace internal {
template <typename... Ts> struct Types {};
template <typename F, typename L> struct Callable;
template <typename F, typename... Ts>
struct Callable<F, Types<Ts...>> : std::is_invocable_r<Error, F, Ts...> {};
}  // namespace internal

struct Handler {};

// Collects the types a handler function receives, in binding order.
template <typename... Ts>
class Binding {
 public:
  template <typename C> auto Ctx() const { return Next(static_cast<C*>(nullptr)); }
  template <typename T> Binding<Ts..., T> Arg() const { return {}; }
  template <typename T> Binding<Ts..., Result<T>> Ret() const { return {}; }
  Binding<Ts..., ::xla::ffi::RemainingArgs> RemainingArgs() const { return {}; }
  template <typename T> Binding<Ts..., T> Attr(const std::string&) const { return {}; }
  template <typename F>
  Handler To(F&&) const {
    static_assert(internal::Callable<F, internal::Types<Ts...>>::value,
                  "the handler function does not take the bound context, operands, results and attributes in order");
    return {};
  }

 private:
  template <typename S> Binding<Ts..., S> Next(PlatformStream<S>*) const { return {}; }
};

struct Ffi {
  static Binding<> Bind() { return {}; }
};

}  // namespace xla::ffi

#define XLA_FFI_DEFINE_HANDLER_SYMBOL(name, fn, binding) \
  extern "C" const void* name() {                        \
    static const ::xla::ffi::Handler handler = (binding).To(fn); \
    return &handler;                                     \
  }
