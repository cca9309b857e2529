// Types and small helpers of the gfx950 code emitter.  The names follow the reference's generator
// (core/inc/SOFIE/utils/SOFIE_common.hxx) so that model-building code reads the same.
#ifndef SOFIE_HIP_COMMON
#define SOFIE_HIP_COMMON

#include <algorithm>
#include <cctype>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace SOFIE_HIP {

// ONNX TensorProto.DataType codes, as in the reference's ETensorType (SOFIE_common.hxx:29-32), extended by
// FLOAT8E4M3FN = 17, which the reference's enum stops short of.
enum class ETensorType {
   UNDEFINED = 0, FLOAT = 1, UINT8 = 2, INT8 = 3, UINT16 = 4, INT16 = 5, INT32 = 6, INT64 = 7, STRING = 8, BOOL = 9,
   FLOAT16 = 10, DOUBLE = 11, UINT32 = 12, UINT64 = 13, BFLOAT16 = 16, FLOAT8E4M3FN = 17
};

// the six activations a producer can take as its own, then the reference's other one-to-one float operators
// (EBasicUnaryOperator, core/inc/SOFIE/operators/ROperator_BasicUnary.hxx:11, and Clip)
enum class EActivationType {
   UNDEFINED, RELU, LEAKYRELU, SIGMOID, GELU, GELU_TANH, TANH,
   RECIPROCAL, SQRT, NEG, EXP, LOG, SIN, COS, ABS, SOFTPLUS, ATAN, FLOOR, ASINH, ACOSH, ATANH, CLIP, SELU, ELU, ERF, HARDSIGMOID, HARDSWISH, SWISH
};
enum class EBasicUnaryOperator { kReciprocal, kSqrt, kNeg, kExp, kLog, kSin, kCos, kAbs, kSoftplus, kAtan, kFloor, kAsinh, kAcosh, kAtanh };

// one link of a chain of one-to-one operators fused behind a producer (alpha: LeakyRelu slope or Clip minimum, beta: Clip maximum)
struct PostOp {
   EActivationType act = EActivationType::UNDEFINED;
   float alpha = 0.f, beta = 0.f;
};
constexpr std::size_t kMaxPostOps = 4; // SOFIE_MAX_POST_OPS of the runtime
constexpr std::size_t kMaxGemmChain = 16; // SOFIE_MAX_GEMM_CHAIN of the runtime

// Options of RModel::GenerateGPU_HIP: the subset of the reference's bit flags (core/inc/SOFIE/RModel_Base.hxx:19-33)
// that applies to this backend, with the reference's values.
enum class Options {
   kDefault = 0x0,
   kNoWeightFile = 0x2,
   kSafetensorsWeightFile = 0x100,
   kStridedInput = 0x200, // the Session's constructor takes the strides of the graph inputs (operands of Gemm)
   kExternalStream = 0x400,
   kCustomMemory = 0x800,
};
inline std::underlying_type_t<Options> operator|(Options a, Options b)
{
   return static_cast<std::underlying_type_t<Options>>(a) | static_cast<std::underlying_type_t<Options>>(b);
}

// Session member that holds the strides given for a graph input (the reference's name, core/inc/SOFIE/operators/ROperator.hxx:109)
inline std::string InputStrideMemberName(const std::string &inputName) { return "fInputStride_" + inputName; }

inline std::size_t GetTypeSize(ETensorType t)
{
   switch (t) {
   case ETensorType::FLOAT: case ETensorType::INT32: case ETensorType::UINT32: return 4;
   case ETensorType::INT8: case ETensorType::UINT8: case ETensorType::BOOL: case ETensorType::FLOAT8E4M3FN: return 1;
   case ETensorType::INT16: case ETensorType::UINT16: case ETensorType::FLOAT16: case ETensorType::BFLOAT16: return 2;
   case ETensorType::INT64: case ETensorType::UINT64: case ETensorType::DOUBLE: return 8;
   default: return 0;
   }
}

// C++ type of a tensor element in the emitted code (bf16 and e4m3 travel as raw bits)
inline std::string ConvertTypeToString(ETensorType t)
{
   switch (t) {
   case ETensorType::FLOAT: return "float";
   case ETensorType::INT8: return "int8_t";
   case ETensorType::UINT8: case ETensorType::BOOL: case ETensorType::FLOAT8E4M3FN: return "uint8_t";
   case ETensorType::INT32: return "int32_t";
   case ETensorType::INT64: return "int64_t";
   case ETensorType::BFLOAT16: return "uint16_t";
   case ETensorType::DOUBLE: return "double";
   default: return "other_" + std::to_string(static_cast<int>(t));
   }
}

inline std::size_t ConvertShapeToLength(const std::vector<std::size_t> &shape)
{
   std::size_t n = 1;
   for (auto d : shape)
      n *= d;
   return n;
}

// the same with a limit: a shape whose element count does not fit 2^40 is refused (a corrupt file, or a product that
// would overflow the byte arithmetic of the memory plan)
inline std::size_t CheckedShapeLength(const std::vector<std::size_t> &shape, const std::string &what)
{
   const std::size_t limit = std::size_t(1) << 40;
   std::size_t n = 1;
   for (auto d : shape) {
      if (d != 0 && n > limit / d)
         throw std::runtime_error("SOFIE: tensor " + what + " has more than 2^40 elements");
      n *= d;
   }
   return n;
}

inline std::string ConvertShapeToString(const std::vector<std::size_t> &shape)
{
   std::string s = "{ ";
   for (std::size_t i = 0; i < shape.size(); ++i)
      s += std::to_string(shape[i]) + (i + 1 < shape.size() ? " , " : "");
   return s + " }";
}

namespace UTILITY {
// '-' and '.' become '_', every other non-alphanumeric character is dropped (core/src/utils/SOFIE_common.cxx:509-516)
inline std::string Clean_name(std::string s)
{
   std::replace(s.begin(), s.end(), '-', '_');
   std::replace(s.begin(), s.end(), '.', '_');
   s.erase(std::remove_if(s.begin(), s.end(), [](char c) { return !std::isalnum(static_cast<unsigned char>(c)) && c != '_'; }), s.end());
   return s;
}
} // namespace UTILITY

// One dimension of an input shape: a number, or a named parameter that is fixed when the Session runs
// (the reference's Dim, core/inc/SOFIE/utils/SOFIE_common.hxx:64-89).  `dim` of a parameter is its default value.
struct Dim {
   bool isParam = false;
   std::size_t dim = 0;
   std::string param;
   Dim() = default;
   Dim(std::size_t d) : dim(d) {}
   Dim(const std::string &p, std::size_t d = 0) : isParam(true), dim(d), param(p)
   {
      if (!p.empty() && std::all_of(p.begin(), p.end(), [](unsigned char c) { return std::isdigit(c) != 0; })) {
         isParam = false;
         dim = std::stoull(p);
      }
   }
   std::string GetVal() const { return isParam ? param : std::to_string(dim); }
};

// Text of a count in the emitted code.  In a model with a run-time batch, tensors that carry the batch as
// their leading dimension are kept with that dimension = 1 and their counts are multiplied by the Session's
// `sofie_batch` when the code runs.
inline std::string BatchScaled(bool dynamic, std::size_t unit)
{
   return dynamic ? "sofie_batch * " + std::to_string(unit) : std::to_string(unit);
}

// the same for an argument or field of type int32_t
inline std::string BatchScaledInt(bool dynamic, std::size_t unit)
{
   return dynamic ? "static_cast<std::int32_t>(sofie_batch * " + std::to_string(unit) + ")" : std::to_string(unit);
}

struct InitializedTensor {
   ETensorType type = ETensorType::UNDEFINED;
   std::vector<std::size_t> shape;
   std::shared_ptr<void> data;
   bool constant = false; // folded at generation time: embedded in the header, not in the weight file
};

struct TensorInfo {
   ETensorType type = ETensorType::UNDEFINED;
   std::vector<std::size_t> shape;
};

} // namespace SOFIE_HIP
#endif
