// A stand-in for the part of XLA's typed-FFI C++ API (xla/ffi/api/ffi.h, shipped inside jaxlib) that
// csrc/w8a8_xla_ffi.cc uses.  Test infrastructure only: it lets a machine without jaxlib run the shim
// through the compiler's front end, and it makes the binding of every handler a compile-time check --
// the sequence of .Ctx / .Arg / .Ret / .Attr calls must be invocable as the handler's parameter list, in
// order and by type -- which is what goes wrong when an argument is added to one and not the other.  It
// executes nothing and says nothing about the real library's behaviour.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <type_traits>

struct XLA_FFI_Error;
struct XLA_FFI_CallFrame;

namespace xla::ffi {

enum DataType { S8, U8, S32, F32, BF16 };

template <DataType D> struct NativeTypeOf { using type = void; };
template <> struct NativeTypeOf<S8> { using type = int8_t; };
template <> struct NativeTypeOf<U8> { using type = uint8_t; };
template <> struct NativeTypeOf<S32> { using type = int32_t; };
template <> struct NativeTypeOf<F32> { using type = float; };
template <> struct NativeTypeOf<BF16> { using type = uint16_t; };

template <class T>
class Span {
 public:
  Span(const T* d, size_t n) : d_(d), n_(n) {}
  size_t size() const { return n_; }
  const T& operator[](size_t i) const { return d_[i]; }
  const T& back() const { return d_[n_ - 1]; }
  const T* begin() const { return d_; }
  const T* end() const { return d_ + n_; }
 private:
  const T* d_;
  size_t n_;
};

template <DataType D>
class Buffer {
 public:
  using Native = typename NativeTypeOf<D>::type;
  Span<const int64_t> dimensions() const { return Span<const int64_t>(nullptr, 0); }
  size_t element_count() const { return 0; }
  size_t size_bytes() const { return 0; }
  void* untyped_data() const { return nullptr; }
  Native* typed_data() const { return nullptr; }
};

template <class T>
class Result {
 public:
  T* operator->() { return &v_; }
  T& operator*() { return v_; }
 private:
  T v_;
};
template <DataType D> using ResultBuffer = Result<Buffer<D>>;

class Error {
 public:
  static Error Success() { return Error(); }
  static Error Internal(std::string) { return Error(); }
  static Error InvalidArgument(std::string) { return Error(); }
};

template <class T> struct PlatformStream {};

template <class... Ts>
struct Binding {
  template <class C> struct CtxType;
  template <class T> struct CtxType<PlatformStream<T>> { using type = T; };
  template <class C> Binding<Ts..., typename CtxType<C>::type> Ctx() const { return {}; }
  template <class A> Binding<Ts..., A> Arg() const { return {}; }
  template <class R> Binding<Ts..., Result<R>> Ret() const { return {}; }
  template <class A> Binding<Ts..., A> Attr(const char*) const { return {}; }
  template <class F>
  static constexpr bool Matches() { return std::is_invocable_r_v<Error, F, Ts...>; }
};

struct Ffi {
  static Binding<> Bind() { return {}; }
};

}  // namespace xla::ffi

// The real macro defines an extern "C" symbol that decodes a call frame and invokes `fn`; the stand-in
// defines the symbol too (so that duplicate or misspelt names fail) and checks the binding against `fn`.
#define XLA_FFI_DEFINE_HANDLER_SYMBOL(symbol, fn, binding)                                                 \
  static_assert(decltype(binding)::template Matches<decltype(&fn)>(),                                      \
                #symbol ": the Bind() chain does not match the parameter list of " #fn);                   \
  extern "C" XLA_FFI_Error* symbol(XLA_FFI_CallFrame*) { return nullptr; }
