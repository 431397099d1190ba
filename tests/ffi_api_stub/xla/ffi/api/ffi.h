// A stand-in for jaxlib's xla/ffi/api/ffi.h with just the shape of the API that easydel_amd/csrc/rpa_ffi.cc uses, so that the file can be
// syntax- and type-checked where jax is not installed (tests/test_ffi_shim_source.py).  It is NOT the real header: it says
// nothing about whether the real one accepts the file, and nothing is ever linked against it.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <type_traits>
#include <vector>
namespace xla { namespace ffi {
enum DataType { PRED, S8, S16, S32, S64, U8, U16, U32, U64, F16, F32, F64, BF16, F8E4M3FN, F8E5M2 };
template <typename T> struct Span {
  const T* p; size_t n;
  size_t size() const { return n; }
  const T& operator[](size_t i) const { return p[i]; }
  const T* begin() const { return p; } const T* end() const { return p + n; }
  const T& front() const { return p[0]; } const T& back() const { return p[n - 1]; }
};
struct AnyBuffer {
  void* untyped_data() const { return nullptr; }
  Span<int64_t> dimensions() const { return {nullptr, 0}; }
  DataType element_type() const { return F32; }
  size_t element_count() const { return 0; }
  size_t size_bytes() const { return 0; }
};
template <DataType DT> struct NativeOf { using type = void; };
template <> struct NativeOf<S32> { using type = int32_t; };
template <> struct NativeOf<F32> { using type = float; };
template <> struct NativeOf<U8> { using type = uint8_t; };
template <DataType DT> struct Buffer {
  typename NativeOf<DT>::type* typed_data() const { return nullptr; }
  void* untyped_data() const { return nullptr; }
  Span<int64_t> dimensions() const { return {nullptr, 0}; }
  size_t element_count() const { return 0; }
  size_t size_bytes() const { return 0; }
};
template <typename T> struct Result { T v; T* operator->() { return &v; } T& operator*() { return v; } const T* operator->() const { return &v; } };
struct Error {
  static Error Success() { return {}; }
  static Error Internal(std::string) { return {}; }
  static Error InvalidArgument(std::string) { return {}; }
};
template <typename T> struct PlatformStream { using type = T; };
template <typename... Ts> struct Binding {
  template <typename T> Binding<Ts..., typename T::type> Ctx() const { return {}; }
  template <typename T> Binding<Ts..., T> Arg() const { return {}; }
  template <typename T> Binding<Ts..., Result<T>> Ret() const { return {}; }
  template <typename T> Binding<Ts..., T> Attr(const char*) const { return {}; }
  template <typename F> static constexpr bool Matches = std::is_invocable_r_v<Error, F, Ts...>;
};
struct Ffi { static Binding<> Bind() { return {}; } };
}}  // namespace xla::ffi
#define XLA_FFI_DEFINE_HANDLER_SYMBOL(name, impl, binding)                                              \
  static_assert(decltype(binding)::template Matches<decltype(&impl)>, #name ": handler and binding disagree"); \
  extern "C" void* name(void*) { return nullptr; }
