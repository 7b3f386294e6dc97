// A minimal MODEL of the part of XLA's typed FFI API (xla/ffi/api/ffi.h, shipped inside jaxlib) that
// olmax_amd/ffi/olmax_ffi.cc uses.  Test infrastructure only: it lets the adapter be type-checked on
// a machine without jaxlib (tests/test_ffi_binding.py compiles the adapter against it with
// -fsyntax-only).  Nothing here executes; a binding's Ctx / Arg / Ret / Attr chain is folded into
// the parameter list its handler must accept, and XLA_FFI_DEFINE_HANDLER_SYMBOL asserts that the
// handler is callable with exactly that list and returns ffi::Error.  The real header decodes the
// same list from the call frame at run time.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <type_traits>

namespace xla::ffi {

enum class DataType { PRED, S8, S16, S32, S64, U8, U16, U32, U64, F16, F32, F64, BF16 };

template <class T>
class Span {
 public:
  constexpr Span(T* d = nullptr, size_t n = 0) : d_(d), n_(n) {}
  constexpr size_t size() const { return n_; }
  constexpr T* data() const { return d_; }
  constexpr T* begin() const { return d_; }
  constexpr T* end() const { return d_ + n_; }
  constexpr T& operator[](size_t i) const { return d_[i]; }
  constexpr T& front() const { return d_[0]; }
  constexpr T& back() const { return d_[n_ - 1]; }

 private:
  T* d_;
  size_t n_;
};

class Error {
 public:
  static Error Success() { return Error(); }
  static Error InvalidArgument(std::string) { return Error(); }
  static Error Internal(std::string) { return Error(); }
};

class AnyBuffer {
 public:
  DataType element_type() const { return DataType::F32; }
  Span<const int64_t> dimensions() const { return {}; }
  void* untyped_data() const { return nullptr; }
  size_t size_bytes() const { return 0; }
  size_t element_count() const { return 0; }
};

template <class T>
class Result {
 public:
  T* operator->() { return &v_; }
  T& operator*() { return v_; }

 private:
  T v_;
};

template <class T>
struct PlatformStream {};

namespace internal {
template <class T>
struct CtxDecode;
template <class T>
struct CtxDecode<PlatformStream<T>> {
  using type = T;
};
}  // namespace internal

template <class... Ts>
struct Binding {
  template <class T>
  Binding<Ts..., typename internal::CtxDecode<T>::type> Ctx() const { return {}; }
  template <class T>
  Binding<Ts..., T> Arg() const { return {}; }
  template <class T>
  Binding<Ts..., Result<T>> Ret() const { return {}; }
  template <class T>
  Binding<Ts..., T> Attr(const char*) const { return {}; }
  template <class Fn>
  static constexpr bool Accepts = std::is_invocable_r_v<Error, Fn, Ts...>;
};

struct Ffi {
  static Binding<> Bind() { return {}; }
};

}  // namespace xla::ffi

#define XLA_FFI_DEFINE_HANDLER_SYMBOL(symbol, fn, binding)                                       \
  static_assert(decltype(binding)::template Accepts<decltype(&fn)>,                              \
                #fn ": the handler's parameters do not match its Ctx/Arg/Ret/Attr binding");     \
  extern "C" void* symbol(void*) { return nullptr; }
