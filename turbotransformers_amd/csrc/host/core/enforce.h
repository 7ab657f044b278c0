// Error reporting of the host layer.  Same contract as the reference's TT_ENFORCE* / TT_THROW
// (turbo_transformers/core/enforce.h:41-85): a failed check throws EnforceNotMet, a
// std::exception that pybind11 surfaces as RuntimeError.  Device-API failures also throw
// (the reference prints and calls exit(0), cuda_enforce.cuh:57-64; throwing is strictly safer).
#pragma once

#include <cstdio>
#include <stdexcept>
#include <string>

namespace turbo_transformers {
namespace core {

class EnforceNotMet : public std::exception {
 public:
  explicit EnforceNotMet(std::string msg) : msg_(std::move(msg)) {}
  const char* what() const noexcept override { return msg_.c_str(); }

 private:
  std::string msg_;
};

namespace details {
template <typename... Args>
inline std::string Format(const char* fmt, Args... args) {
  int n = std::snprintf(nullptr, 0, fmt, args...);
  if (n <= 0) return std::string(fmt);
  std::string out((size_t)n + 1, '\0');
  std::snprintf(&out[0], out.size(), fmt, args...);
  out.resize((size_t)n);
  return out;
}
inline std::string Format() { return std::string(); }
inline std::string Format(const char* s) { return std::string(s); }
inline std::string Format(const std::string& s) { return s; }
}  // namespace details

#define TT_THROW(...)                                                                          \
  do {                                                                                         \
    throw ::turbo_transformers::core::EnforceNotMet(                                           \
        ::turbo_transformers::core::details::Format(__VA_ARGS__) + " (" + __FILE__ + ":" +     \
        std::to_string(__LINE__) + ")");                                                       \
  } while (false)

#define TT_ENFORCE(cond, ...)                                                                  \
  do {                                                                                         \
    if (!(cond)) {                                                                             \
      throw ::turbo_transformers::core::EnforceNotMet(                                         \
          std::string("enforce error " #cond " at ") + __FILE__ + ":" +                        \
          std::to_string(__LINE__) + "\n" +                                                    \
          ::turbo_transformers::core::details::Format(__VA_ARGS__));                           \
    }                                                                                          \
  } while (false)

#define TT_ENFORCE_EQ(a, b, ...) TT_ENFORCE((a) == (b), __VA_ARGS__)
#define TT_ENFORCE_NE(a, b, ...) TT_ENFORCE((a) != (b), __VA_ARGS__)
#define TT_ENFORCE_LT(a, b, ...) TT_ENFORCE((a) < (b), __VA_ARGS__)
#define TT_ENFORCE_LE(a, b, ...) TT_ENFORCE((a) <= (b), __VA_ARGS__)
#define TT_ENFORCE_GT(a, b, ...) TT_ENFORCE((a) > (b), __VA_ARGS__)
#define TT_ENFORCE_GE(a, b, ...) TT_ENFORCE((a) >= (b), __VA_ARGS__)

// Turn a C-ABI status into an exception carrying ttmi_last_error().
#define TT_DEVICE_CALL(expr)                                                                   \
  do {                                                                                         \
    int _tt_rc = (expr);                                                                       \
    if (_tt_rc != 0) {                                                                         \
      const char* _m = ttmi_last_error();                                                      \
      TT_THROW("%s failed (%d): %s", #expr, _tt_rc, _m ? _m : "?");                            \
    }                                                                                          \
  } while (false)

}  // namespace core
}  // namespace turbo_transformers
