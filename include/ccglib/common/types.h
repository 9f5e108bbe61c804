// Vocabulary types of the ccglib C++ API, as used by the drop-in classes in this
// directory tree. Enumerator names and integer values are those of the
// reference (they cross the C ABI as plain ints):
//   ValueType            include/ccglib/common/value_type.h:14-22
//   ComplexAxisLocation  include/ccglib/common/complex_order.h:12
//   Direction            include/ccglib/common/direction.h:6
//   mma::MemOrder        include/ccglib/gemm/mem_order.h:6
//   mma::Variant         include/ccglib/gemm/variant.h:6
//   ValuePrecision       include/ccglib/common/value_precision.h:10-33
//   Precision            include/ccglib/common/precision.h:13-37
//   helper::ceildiv      include/ccglib/common/helper.h:6-13
#ifndef CCGLIB_COMMON_TYPES_H_
#define CCGLIB_COMMON_TYPES_H_

#include <cstddef>

namespace ccglib {

enum ValueType { int1 = 0, int32 = 1, bfloat16 = 2, float8e4m3 = 3, float8e5m2 = 4, float16 = 5, float32 = 6 };
enum ComplexAxisLocation { complex_planar = 0, complex_interleaved = 1 };
enum Direction { forward = 0, backward = 1 };

namespace mma {
enum MemOrder { row_major = 0, col_major = 1 };
enum Variant { basic = 0, opt = 1 };
}  // namespace mma

constexpr std::size_t CalculateBitWidth(ValueType type) {
  return type == int1 ? 1
         : (type == float8e4m3 || type == float8e5m2) ? 8
         : (type == bfloat16 || type == float16) ? 16
         : (type == float32 || type == int32) ? 32
                                              : 0;
}

// A value type together with its width in bits.
struct ValuePrecision {
  constexpr ValuePrecision(ValueType t) : type(t), num_bits(CalculateBitWidth(t)) {}
  constexpr ValuePrecision(ValueType t, std::size_t bits) : type(t), num_bits(bits) {}
  constexpr bool operator==(const ValuePrecision &o) const { return type == o.type; }
  constexpr bool operator==(const ValueType &o) const { return type == o; }
  constexpr operator ValueType() const { return type; }
  constexpr std::size_t GetBitWidth() const { return num_bits; }

 private:
  ValueType type;
  std::size_t num_bits;
};

// Input and output value types of a GEMM; the output defaults to float32.
struct Precision {
  constexpr Precision(ValueType in) : input_type(in), output_type(float32) {}
  constexpr Precision(ValueType in, ValueType out) : input_type(in), output_type(out) {}
  constexpr Precision(ValuePrecision in) : input_type(in), output_type(float32) {}
  constexpr Precision(ValuePrecision in, ValuePrecision out) : input_type(in), output_type(out) {}
  constexpr std::size_t GetInputBits() const { return input_type.GetBitWidth(); }
  constexpr std::size_t GetOutputBits() const { return output_type.GetBitWidth(); }
  const ValuePrecision input_type;
  const ValuePrecision output_type;
};

namespace helper {
// Rounded-up quotient of two positive integers.
template <typename T> inline T ceildiv(T a, T b) { return a / b + (a % b != 0 ? 1 : 0); }
inline std::size_t ceildiv(std::size_t a, unsigned b) { return ceildiv(a, static_cast<std::size_t>(b)); }
}  // namespace helper

}  // namespace ccglib
#endif  // CCGLIB_COMMON_TYPES_H_
