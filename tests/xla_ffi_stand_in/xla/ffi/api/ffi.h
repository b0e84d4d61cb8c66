// A stand-in for jaxlib's xla/ffi/api/ffi.h, for tests only: the subset of the XLA FFI C++ API that
// axlearn_amd/csrc/ffi_shim.cc uses, written from that API's public documentation, so that the shim can
// be compiled and its handlers run where jaxlib is not installed.  It is NOT the real header: a handler
// defined with XLA_FFI_DEFINE_HANDLER_SYMBOL here is an `extern "C" int symbol(AxlStandInCallFrame*)`
// that a test fills by hand (tests/jax_stand_in.py), not an XLA_FFI_Handler.  What it keeps faithful is
// what the shim's source sees: the names, the accessors of AnyBuffer / Result / Span / Error, the
// binding chain Ffi::Bind().Ctx<>().Arg<>().Ret<>().Attr<T>("name"), operands and results decoded in
// binding order, attributes decoded by name and exact type.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

extern "C" {
struct AxlStandInBuffer {
  void* data;
  int32_t dtype;  // xla::ffi::DataType
  int32_t rank;
  const int64_t* dims;
};
struct AxlStandInAttr {
  const char* name;
  int32_t kind;  // 0: int32_t, 1: float
  int32_t i32;
  float f32;
};
struct AxlStandInCallFrame {
  void* stream;
  int32_t n_args;
  const AxlStandInBuffer* args;
  int32_t n_rets;
  const AxlStandInBuffer* rets;
  int32_t n_attrs;
  const AxlStandInAttr* attrs;
  int32_t error_code;  // out: xla::ffi::ErrorCode
  char error[1024];    // out: message
};
}

namespace xla::ffi {

enum class DataType : uint8_t {
  INVALID = 0, PRED = 1, S8 = 2, S16 = 3, S32 = 4, S64 = 5, U8 = 6, U16 = 7, U32 = 8, U64 = 9,
  F16 = 10, F32 = 11, F64 = 12, BF16 = 16,
};

inline size_t ByteWidth(DataType t) {
  switch (t) {
    case DataType::PRED: case DataType::S8: case DataType::U8: return 1;
    case DataType::S16: case DataType::U16: case DataType::F16: case DataType::BF16: return 2;
    case DataType::S32: case DataType::U32: case DataType::F32: return 4;
    case DataType::S64: case DataType::U64: case DataType::F64: return 8;
    default: return 0;
  }
}

enum class ErrorCode : uint8_t {
  kOk = 0, kCancelled = 1, kUnknown = 2, kInvalidArgument = 3, kDeadlineExceeded = 4, kNotFound = 5,
  kAlreadyExists = 6, kPermissionDenied = 7, kResourceExhausted = 8, kFailedPrecondition = 9, kAborted = 10,
  kOutOfRange = 11, kUnimplemented = 12, kInternal = 13, kUnavailable = 14, kDataLoss = 15, kUnauthenticated = 16,
};

class Error {
 public:
  Error() = default;
  Error(ErrorCode errc, std::string message) : errc_(errc), message_(std::move(message)) {}
  static Error Success() { return Error(); }
  bool success() const { return errc_ == ErrorCode::kOk; }
  bool failure() const { return !success(); }
  ErrorCode errc() const { return errc_; }
  const std::string& message() const { return message_; }

 private:
  ErrorCode errc_ = ErrorCode::kOk;
  std::string message_;
};

template <typename T>
class Span {
 public:
  constexpr Span(T* data, size_t size) : data_(data), size_(size) {}
  constexpr size_t size() const { return size_; }
  constexpr T& operator[](size_t i) const { return data_[i]; }
  constexpr T* begin() const { return data_; }
  constexpr T* end() const { return data_ + size_; }
  constexpr T& front() const { return data_[0]; }
  constexpr T& back() const { return data_[size_ - 1]; }

 private:
  T* data_;
  size_t size_;
};

class AnyBuffer {
 public:
  using Dimensions = Span<const int64_t>;
  explicit AnyBuffer(const AxlStandInBuffer* buf) : buf_(buf) {}
  DataType element_type() const { return static_cast<DataType>(buf_->dtype); }
  Dimensions dimensions() const { return Dimensions(buf_->dims, static_cast<size_t>(buf_->rank)); }
  void* untyped_data() const { return buf_->data; }
  size_t element_count() const {
    size_t n = 1;
    for (int i = 0; i < buf_->rank; i++) n *= static_cast<size_t>(buf_->dims[i]);
    return n;
  }
  size_t size_bytes() const { return element_count() * ByteWidth(element_type()); }

 private:
  const AxlStandInBuffer* buf_;
};

template <typename T>
class Result {
 public:
  explicit Result(T value) : value_(value) {}
  T* operator->() { return &value_; }
  T& operator*() { return value_; }

 private:
  T value_;
};

template <typename T>
struct PlatformStream {};

namespace stand_in {

template <typename T> struct CtxTag {};
template <typename T> struct ArgTag {};
template <typename T> struct RetTag {};
template <typename T> struct AttrTag {};

struct Cursor {
  int arg = 0, ret = 0, attr = 0;
  Error error;
};

template <typename Tag> struct Decode;
template <typename S>
struct Decode<CtxTag<PlatformStream<S>>> {
  static S Get(const AxlStandInCallFrame& f, const std::vector<std::string>&, Cursor&) { return static_cast<S>(f.stream); }
};
template <>
struct Decode<ArgTag<AnyBuffer>> {
  static AnyBuffer Get(const AxlStandInCallFrame& f, const std::vector<std::string>&, Cursor& c) {
    return AnyBuffer(&f.args[c.arg++]);
  }
};
template <>
struct Decode<RetTag<AnyBuffer>> {
  static Result<AnyBuffer> Get(const AxlStandInCallFrame& f, const std::vector<std::string>&, Cursor& c) {
    return Result<AnyBuffer>(AnyBuffer(&f.rets[c.ret++]));
  }
};
template <typename T>
struct Decode<AttrTag<T>> {
  static_assert(std::is_same_v<T, int32_t> || std::is_same_v<T, float>, "stand-in: int32_t and float attributes only");
  static T Get(const AxlStandInCallFrame& f, const std::vector<std::string>& names, Cursor& c) {
    const std::string& name = names[c.attr++];
    constexpr int kind = std::is_same_v<T, float> ? 1 : 0;
    for (int i = 0; i < f.n_attrs; i++) {
      if (name != f.attrs[i].name) continue;
      if (f.attrs[i].kind != kind) {
        c.error = Error(ErrorCode::kInvalidArgument, "attribute " + name + " has the wrong type");
        return T{};
      }
      if constexpr (kind == 1) return f.attrs[i].f32;
      else return f.attrs[i].i32;
    }
    c.error = Error(ErrorCode::kInvalidArgument, "attribute " + name + " is missing");
    return T{};
  }
};

template <typename Tag> struct Counts { static constexpr int args = 0, rets = 0, attrs = 0; };
template <typename T> struct Counts<ArgTag<T>> { static constexpr int args = 1, rets = 0, attrs = 0; };
template <typename T> struct Counts<RetTag<T>> { static constexpr int args = 0, rets = 1, attrs = 0; };
template <typename T> struct Counts<AttrTag<T>> { static constexpr int args = 0, rets = 0, attrs = 1; };

}  // namespace stand_in

template <typename... Tags>
class Binding {
 public:
  Binding() = default;
  explicit Binding(std::vector<std::string> attr_names) : attr_names_(std::move(attr_names)) {}
  template <typename T> Binding<Tags..., stand_in::CtxTag<T>> Ctx() && { return Binding<Tags..., stand_in::CtxTag<T>>(std::move(attr_names_)); }
  template <typename T> Binding<Tags..., stand_in::ArgTag<T>> Arg() && { return Binding<Tags..., stand_in::ArgTag<T>>(std::move(attr_names_)); }
  template <typename T> Binding<Tags..., stand_in::RetTag<T>> Ret() && { return Binding<Tags..., stand_in::RetTag<T>>(std::move(attr_names_)); }
  template <typename T> Binding<Tags..., stand_in::AttrTag<T>> Attr(std::string name) && {
    attr_names_.push_back(std::move(name));
    return Binding<Tags..., stand_in::AttrTag<T>>(std::move(attr_names_));
  }

  // Decodes the frame in binding order and calls fn; the error (if any) goes back through the frame.
  template <typename Fn>
  int Call(Fn&& fn, AxlStandInCallFrame* frame) const {
    constexpr int n_args = (0 + ... + stand_in::Counts<Tags>::args), n_rets = (0 + ... + stand_in::Counts<Tags>::rets),
                  n_attrs = (0 + ... + stand_in::Counts<Tags>::attrs);
    Error err;
    if (frame->n_args != n_args || frame->n_rets != n_rets || frame->n_attrs != n_attrs) {
      err = Error(ErrorCode::kInvalidArgument,
                  "wrong number of operands / results / attributes: expected " + std::to_string(n_args) + " / " +
                      std::to_string(n_rets) + " / " + std::to_string(n_attrs) + ", got " + std::to_string(frame->n_args) +
                      " / " + std::to_string(frame->n_rets) + " / " + std::to_string(frame->n_attrs));
    } else {
      stand_in::Cursor cursor;
      // braced initialisation: the decoders run left to right
      std::tuple<decltype(stand_in::Decode<Tags>::Get(*frame, attr_names_, cursor))...> decoded{
          stand_in::Decode<Tags>::Get(*frame, attr_names_, cursor)...};
      err = cursor.error.failure() ? cursor.error : std::apply(fn, std::move(decoded));
    }
    frame->error_code = static_cast<int32_t>(err.errc());
    std::strncpy(frame->error, err.message().c_str(), sizeof(frame->error) - 1);
    frame->error[sizeof(frame->error) - 1] = '\0';
    return frame->error_code;
  }

 private:
  std::vector<std::string> attr_names_;
};

struct Ffi {
  static Binding<> Bind() { return Binding<>(); }
};

}  // namespace xla::ffi

#define XLA_FFI_DEFINE_HANDLER_SYMBOL(symbol, impl, binding)            \
  extern "C" int symbol(AxlStandInCallFrame* frame) {                   \
    static const auto bound = (binding);                                \
    return bound.Call(impl, frame);                                     \
  }
