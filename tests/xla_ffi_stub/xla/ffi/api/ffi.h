// TEST INFRASTRUCTURE ONLY.  A minimal stand-in for the part of jaxlib's xla/ffi/api/ffi.h that
// maxdiffusion_amd/csrc/ffi/mdattn_ffi.cc uses, so that the shim can be type-checked on a machine without jaxlib
// (tests/test_ffi_shim.py compiles it with -fsyntax-only).  It follows the public typed-FFI interface: AnyBuffer with
// element_type / dimensions / untyped_data / element_count, Result<T>, Error, PlatformStream<T>, the
// Ffi::Bind().Ctx<>().Arg<>().Ret<>().Attr<>(name) builder and XLA_FFI_DEFINE_HANDLER_SYMBOL, which here checks at
// compile time that the handler function can be called with exactly the bound context, arguments, results and
// attributes, in that order (the real header performs the same check through its own templates).
// Never shipped, never linked into the product; a real build uses jax.ffi.include_dir().
#ifndef MDATTN_TEST_XLA_FFI_STUB_H_
#define MDATTN_TEST_XLA_FFI_STUB_H_

#include <cstddef>
#include <cstdint>
#include <string>
#include <type_traits>

namespace xla {
namespace ffi {

enum class DataType : uint8_t { INVALID = 0, PRED, S8, S16, S32, S64, U8, U16, U32, U64, F16, F32, F64, BF16, F8E5M2, F8E4M3FN };

template <typename T>
class Span {
 public:
  Span(T* data, size_t size) : data_(data), size_(size) {}
  T* begin() const { return data_; }
  T* end() const { return data_ + size_; }
  size_t size() const { return size_; }
  T& operator[](size_t i) const { return data_[i]; }

 private:
  T* data_;
  size_t size_;
};

class AnyBuffer {
 public:
  DataType element_type() const { return type_; }
  Span<const int64_t> dimensions() const { return Span<const int64_t>(dims_, rank_); }
  void* untyped_data() const { return data_; }
  size_t element_count() const {
    size_t n = 1;
    for (size_t i = 0; i < rank_; ++i) n *= (size_t)dims_[i];
    return n;
  }

 private:
  void* data_ = nullptr;
  DataType type_ = DataType::INVALID;
  const int64_t* dims_ = nullptr;
  size_t rank_ = 0;
};

template <typename T>
class Result {
 public:
  T* operator->() { return &value_; }
  T& operator*() { return value_; }

 private:
  T value_;
};

enum class ErrorCode { kOk = 0, kInvalidArgument = 3, kResourceExhausted = 8, kUnimplemented = 12, kInternal = 13 };

class Error {
 public:
  Error() = default;
  Error(ErrorCode code, std::string message) : code_(code), message_(std::move(message)) {}
  static Error Success() { return Error(); }
  static Error InvalidArgument(std::string message) { return Error(ErrorCode::kInvalidArgument, std::move(message)); }
  static Error Internal(std::string message) { return Error(ErrorCode::kInternal, std::move(message)); }
  bool success() const { return code_ == ErrorCode::kOk; }
  ErrorCode code() const { return code_; }
  const std::string& message() const { return message_; }

 private:
  ErrorCode code_ = ErrorCode::kOk;
  std::string message_;
};

template <typename T>
struct PlatformStream {};

template <typename... Ts>
struct Binding {
  template <typename C>
  struct CtxOf;
  template <typename S>
  struct CtxOf<PlatformStream<S>> {
    using type = S;
  };
  template <typename C>
  Binding<Ts..., typename CtxOf<C>::type> Ctx() const { return {}; }
  template <typename T>
  Binding<Ts..., T> Arg() const { return {}; }
  template <typename T>
  Binding<Ts..., Result<T>> Ret() const { return {}; }
  template <typename T>
  Binding<Ts..., T> Attr(const char*) const { return {}; }

  template <typename Fn>
  static constexpr bool Accepts() { return std::is_invocable_r_v<Error, Fn, Ts...>; }
};

struct Ffi {
  static Binding<> Bind() { return {}; }
};

}  // namespace ffi
}  // namespace xla

// The real macro defines an exported XLA_FFI_Handler; here: an exported symbol of the same name and the signature check.
#define XLA_FFI_DEFINE_HANDLER_SYMBOL(name, impl, binding)                                                         \
  static_assert(decltype(binding)::template Accepts<decltype(&impl)>(),                                            \
                #name ": the handler's parameters do not match the bound context/arguments/results/attributes");   \
  extern "C" int name(void*) { return 0; }

#endif  // MDATTN_TEST_XLA_FFI_STUB_H_
