// Registration machinery of RAL: the memref ABI struct, the type-code mangling that
// turns a C++ signature into the symbol the DISC compiler emits, the global
// registry, and the type-erased invoker that rebuilds typed arguments from the
// compiler's void** slots.
//
// Public names and behaviour follow the reference's tao_compiler/mlir/ral/ral_helper.h
// (MemRefType :46-60, type codes :65-152, invoker :160-252, registry :254-285,
// driver wrapper :287-420) so kernel sources written against it register
// unchanged; the compiler side of the contract is disc/transforms/disc_to_llvm.cc
// :74-168 (signature encoding) and :302-365 (slot packing).
//
// Slot packing: args[i] points at the i-th scalar.  A scalar argument takes one
// slot; a MemRefType<T,N> takes 3+2N consecutive slots (basePtr, data, offset,
// sizes[N], strides[N]).  After the arguments come the result slots: one per
// result, each pointing at storage for the whole result value.
#ifndef RAL_RAL_HELPER_H_
#define RAL_RAL_HELPER_H_

#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

#include "mlir/ral/ral_base.h"

namespace tao {
namespace ral {

class Context;
class ExecutionContext;

struct bfloat16 {
  uint16_t value;
};

struct float16 {
  uint16_t value;
};

// How MLIR lowers a ranked memref to LLVM.
template <typename T, int N>
struct MemRefType {
  T* basePtr;
  T* data;
  int64_t offset;
  int64_t sizes[N];
  int64_t strides[N];
};

template <typename T>
struct MemRefType<T, 0> {
  T* basePtr;
  T* data;
  int64_t offset;
};

namespace detail {

template <typename T>
struct MemRefTraits : std::false_type {};
template <typename T, int N>
struct MemRefTraits<MemRefType<T, N>> : std::true_type {
  using elem = T;
  static constexpr int rank = N;
};

template <typename T>
using bare_t = std::remove_cv_t<std::remove_reference_t<T>>;

// number of void** slots one argument of type T occupies
template <typename T>
constexpr int slotsOf() {
  using U = bare_t<T>;
  if constexpr (MemRefTraits<U>::value)
    return 3 + 2 * MemRefTraits<U>::rank;
  else
    return 1;
}

template <typename... Ts>
struct SlotOffsets {
  static constexpr int count = sizeof...(Ts);
  // offsets[i] = first slot of argument i; offsets[count] = total
  static constexpr auto make() {
    struct R {
      int v[count + 1];
    } r{};
    constexpr int sizes[count + 1] = {slotsOf<Ts>()..., 0};
    int acc = 0;
    for (int i = 0; i < count; ++i) {
      r.v[i] = acc;
      acc += sizes[i];
    }
    r.v[count] = acc;
    return r;
  }
};

}  // namespace detail

// ---------------------------------------------------------------- type codes
template <typename T, typename Enable = void>
struct TaoTypeNameHelper;

#define DEFINE_TAO_TYPE_NAME_HELPER(type, name)  \
  template <>                                    \
  struct TaoTypeNameHelper<type, void> {         \
    static std::string Invoke() { return name; } \
  };

DEFINE_TAO_TYPE_NAME_HELPER(bool, "i1");
DEFINE_TAO_TYPE_NAME_HELPER(uint8_t, "ui8");
DEFINE_TAO_TYPE_NAME_HELPER(int8_t, "i8");
DEFINE_TAO_TYPE_NAME_HELPER(uint16_t, "ui16");
DEFINE_TAO_TYPE_NAME_HELPER(int16_t, "i16");
DEFINE_TAO_TYPE_NAME_HELPER(bfloat16, "bf16");
DEFINE_TAO_TYPE_NAME_HELPER(float16, "f16");
DEFINE_TAO_TYPE_NAME_HELPER(uint32_t, "ui32");
DEFINE_TAO_TYPE_NAME_HELPER(int32_t, "i32");
DEFINE_TAO_TYPE_NAME_HELPER(int64_t, "i64");
DEFINE_TAO_TYPE_NAME_HELPER(size_t, "i64");
DEFINE_TAO_TYPE_NAME_HELPER(float, "f32");
DEFINE_TAO_TYPE_NAME_HELPER(double, "f64");
DEFINE_TAO_TYPE_NAME_HELPER(void, "void");
// every context handle and untyped / character pointer is an opaque "pvoid"
DEFINE_TAO_TYPE_NAME_HELPER(const char*, "pvoid");
DEFINE_TAO_TYPE_NAME_HELPER(char*, "pvoid");
DEFINE_TAO_TYPE_NAME_HELPER(Context*, "pvoid");
DEFINE_TAO_TYPE_NAME_HELPER(ExecutionContext*, "pvoid");
DEFINE_TAO_TYPE_NAME_HELPER(const void*, "pvoid");

template <typename T, int N>
struct TaoTypeNameHelper<MemRefType<T, N>, void> {
  static std::string Invoke() {
    return "m" + std::to_string(N) + "d" + TaoTypeNameHelper<T>::Invoke();
  }
};

// other pointers: "p" + pointee code (void* -> "pvoid", void** -> "ppvoid")
template <typename T>
struct TaoTypeNameHelper<T*, void> {
  static std::string Invoke() { return "p" + TaoTypeNameHelper<T>::Invoke(); }
};

// references and cv-qualified values mangle like the value
template <typename T>
struct TaoTypeNameHelper<
    T, std::enable_if_t<!std::is_same<T, detail::bare_t<T>>::value>> {
  static std::string Invoke() {
    return TaoTypeNameHelper<detail::bare_t<T>>::Invoke();
  }
};

template <typename... Ts>
struct TaoVariadicTypeNameHelper {
  static std::string Invoke() {
    std::string out;
    const std::string codes[] = {TaoTypeNameHelper<Ts>::Invoke()..., ""};
    for (size_t i = 0; i < sizeof...(Ts); ++i) {
      if (i) out += "_";
      out += codes[i];
    }
    return out;
  }
};

template <typename... Ts>
struct TaoTypeNameHelper<std::tuple<Ts...>, void> {
  static std::string Invoke() { return TaoVariadicTypeNameHelper<Ts...>::Invoke(); }
};

// "<prefix>___<arg codes joined by _>___<result code>"
template <typename F>
struct TaoRalApiFuncNameHelper;

template <typename R, typename... Args>
struct TaoRalApiFuncNameHelper<R (*)(Args...)> {
  static std::string Invoke(const std::string& prefix) {
    return prefix + "___" + TaoVariadicTypeNameHelper<Args...>::Invoke() + "___" +
           TaoTypeNameHelper<R>::Invoke();
  }
};

template <typename R, typename... Args>
struct TaoRalApiFuncNameHelper<std::function<R(Args...)>>
    : TaoRalApiFuncNameHelper<R (*)(Args...)> {};

// ------------------------------------------------------------------- invoker
namespace detail {

// Rebuilds one typed argument from its slots.
template <typename T>
bare_t<T> decodeArg(void** slot) {
  using U = bare_t<T>;
  if constexpr (MemRefTraits<U>::value) {
    using E = typename MemRefTraits<U>::elem;
    constexpr int N = MemRefTraits<U>::rank;
    U m;
    m.basePtr = *static_cast<E**>(slot[0]);
    m.data = *static_cast<E**>(slot[1]);
    m.offset = *static_cast<int64_t*>(slot[2]);
    if constexpr (N > 0) {
      for (int i = 0; i < N; ++i) m.sizes[i] = *static_cast<int64_t*>(slot[3 + i]);
      for (int i = 0; i < N; ++i) m.strides[i] = *static_cast<int64_t*>(slot[3 + N + i]);
    }
    return m;
  } else {
    return *static_cast<U*>(slot[0]);
  }
}

template <typename R>
struct ResultWriter {
  static void write(void** slot, R&& r) { *static_cast<R*>(slot[0]) = std::move(r); }
};

template <typename... Rs>
struct ResultWriter<std::tuple<Rs...>> {
  template <size_t... I>
  static void each(void** slot, std::tuple<Rs...>& r, std::index_sequence<I...>) {
    ((*static_cast<Rs*>(slot[I]) = std::move(std::get<I>(r))), ...);
  }
  static void write(void** slot, std::tuple<Rs...>&& r) {
    each(slot, r, std::index_sequence_for<Rs...>{});
  }
};

template <typename R, typename... Args, size_t... I>
void invokeErased(R (*fn)(Args...), void** args, std::index_sequence<I...>) {
  constexpr auto off = SlotOffsets<Args...>::make();
  // decoded values live here so that reference parameters can bind to them
  std::tuple<bare_t<Args>...> decoded{decodeArg<Args>(args + off.v[I])...};
  if constexpr (std::is_void<R>::value) {
    fn(std::get<I>(decoded)...);
  } else {
    ResultWriter<R>::write(args + off.v[sizeof...(Args)], fn(std::get<I>(decoded)...));
  }
}

}  // namespace detail

template <typename F, F f>
struct TaoRalApiFuncInvoker;

template <typename R, typename... Args, R (*impl_fn)(Args...)>
struct TaoRalApiFuncInvoker<R (*)(Args...), impl_fn> {
  static void Invoke(void** args) {
    detail::invokeErased(impl_fn, args, std::index_sequence_for<Args...>{});
  }
};

// ------------------------------------------------------------------ registry
class TaoRalApiRegistry {
 public:
  ~TaoRalApiRegistry();
  using api_func_t = tao::ral::api_func_t;
  static TaoRalApiRegistry& Global();
  // Registers `api_func` under the full mangled `name`; `nickname` (the bare
  // target name) is bound to it too unless something already owns it.
  // Returns false when `name` was already registered (the first one is kept).
  bool Register(const std::string& name, const std::string& nickname,
                api_func_t api_func);
  api_func_t Find(const std::string& name);
  // All registered keys, sorted (introspection; not part of the reference API).
  std::vector<std::string> Names();

 private:
  TaoRalApiRegistry();
  struct Impl;
  std::unique_ptr<Impl> impl_;
};

#define TAO_RAL_API(name, device, ...) \
  TAO_RAL_API_UNIQ_HELPER(name, device, __COUNTER__, __VA_ARGS__)

#define TAO_RAL_API_UNIQ_HELPER(name, device, ctr, ...) \
  TAO_RAL_API_UNIQ(name, device, ctr, __VA_ARGS__)

#define TAO_RAL_API_UNIQ(name, device, ctr, ...)                               \
  static bool unused_ret_val_##ctr =                                           \
      ::tao::ral::TaoRalApiRegistry::Global().Register(                        \
          ::tao::ral::TaoRalApiFuncNameHelper<decltype(&__VA_ARGS__)>::Invoke( \
              std::string(name) + "___" + std::string(device)),                \
          std::string(name),                                                   \
          ::tao::ral::TaoRalApiFuncInvoker<decltype(&__VA_ARGS__),             \
                                           &__VA_ARGS__>::Invoke);

// ------------------------------------------------ typed view of an api_func_t
// Turns a type-erased registry entry back into a typed callable by packing the
// arguments into slots the way compiled code does.  Used by the driver facades,
// which resolve their implementation by name at construction.
using api_func_t = TaoRalApiRegistry::api_func_t;

namespace detail {

template <typename T>
void encodeArg(std::vector<void*>& slots, T& value) {
  using U = bare_t<T>;
  if constexpr (MemRefTraits<U>::value) {
    constexpr int N = MemRefTraits<U>::rank;
    slots.push_back(static_cast<void*>(&value.basePtr));
    slots.push_back(static_cast<void*>(&value.data));
    slots.push_back(static_cast<void*>(&value.offset));
    if constexpr (N > 0) {
      for (int i = 0; i < N; ++i) slots.push_back(static_cast<void*>(&value.sizes[i]));
      for (int i = 0; i < N; ++i) slots.push_back(static_cast<void*>(&value.strides[i]));
    }
  } else {
    slots.push_back(const_cast<void*>(static_cast<const void*>(&value)));
  }
}

}  // namespace detail

template <typename T>
struct DriverApiWrapper;

template <typename R, typename... Args>
struct DriverApiWrapper<std::function<R(Args...)>> {
  static std::function<R(Args...)> Wrapper(api_func_t func) {
    if (!func) return nullptr;
    return [func](Args... args) -> R {
      std::vector<void*> slots;
      (detail::encodeArg(slots, args), ...);
      if constexpr (std::is_void<R>::value) {
        func(slots.data());
      } else {
        R result{};
        slots.push_back(static_cast<void*>(&result));
        func(slots.data());
        return result;
      }
    };
  }
};

#define TAO_RAL_ASSIGN_TO_API_FUNC_WRAPPER(wrapper, api_func) \
  wrapper = ::tao::ral::DriverApiWrapper<decltype(wrapper)>::Wrapper(api_func);

}  // namespace ral
}  // namespace tao

#endif  // RAL_RAL_HELPER_H_
