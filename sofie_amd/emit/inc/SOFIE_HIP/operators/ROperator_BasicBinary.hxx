// The broadcasting binary operators Add, Sub, Mul, Div, Pow (core/inc/SOFIE/operators/ROperator_BasicBinary.hxx:22-53) and, as
// left folds of pairwise steps, the n-ary Max, Min, Sum, Mean (ROperator_BasicNary.hxx:19-100): one runtime call per step with
// the multidirectional broadcast resolved at generation time.
#ifndef SOFIE_HIP_ROPERATOR_BASICBINARY
#define SOFIE_HIP_ROPERATOR_BASICBINARY

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

#include <cmath>

namespace SOFIE_HIP {

// Add .. Pow as in the reference; the last three are the pairwise steps of the n-ary operators
enum EBasicBinaryOperator { Add, Sub, Mul, Div, Pow, PairMax, PairMin, AddThenDivide };

inline const char *BinaryRuntimeCode(EBasicBinaryOperator op)
{
   switch (op) {
   case Sub: return "SOFIE_BINARY_SUB";
   case Mul: return "SOFIE_BINARY_MUL";
   case Div: return "SOFIE_BINARY_DIV";
   case Pow: return "SOFIE_BINARY_POW";
   case PairMax: return "SOFIE_BINARY_MAX";
   case PairMin: return "SOFIE_BINARY_MIN";
   case AddThenDivide: return "SOFIE_BINARY_ADD_DIV";
   default: return "SOFIE_BINARY_ADD";
   }
}
inline const char *BinaryName(EBasicBinaryOperator op)
{
   switch (op) {
   case Sub: return "Sub";
   case Mul: return "Mul";
   case Div: return "Div";
   case Pow: return "Pow";
   case PairMax: return "Max";
   case PairMin: return "Min";
   case AddThenDivide: return "Mean (last step)";
   default: return "Add";
   }
}
// the value the generated code computes, for folding two constants (the host's arithmetic is the reference's)
inline float BinaryValue(EBasicBinaryOperator op, float a, float b, float param)
{
   switch (op) {
   case Sub: return a - b;
   case Mul: return a * b;
   case Div: return a / b;
   case Pow: return std::pow(a, b);
   case PairMax: return a < b ? b : a;
   case PairMin: return b < a ? b : a;
   case AddThenDivide: return (a + b) / param;
   default: return a + b;
   }
}

template <typename T, EBasicBinaryOperator Op>
class ROperator_BasicBinary final : public ROperator {
   static_assert(std::is_same<T, float>::value, "the float operators are on this backend's path");

public:
   ROperator_BasicBinary(std::string nameA, std::string nameB, std::string nameY, float param = 0.f)
      : fNA(UTILITY::Clean_name(nameA)), fNB(UTILITY::Clean_name(nameB)), fNY(UTILITY::Clean_name(nameY)), fParam(param)
   {
      fInputTensorNames = {fNA, fNB};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::BINARY;
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNA) || !model.CheckIfTensorAlreadyExist(fNB))
         throw std::runtime_error("SOFIE Binary Op Input Tensor " + fNA + " or " + fNB + " is not found in model");
      fShapeA = model.GetTensorShape(fNA);
      fShapeB = model.GetTensorShape(fNB);
      const std::size_t r = std::max(fShapeA.size(), fShapeB.size());
      // a batched operand's leading dimension must be the result's leading dimension
      fDynA = model.IsDynamicTensor(fNA);
      fDynB = model.IsDynamicTensor(fNB);
      if ((fDynA && fShapeA.size() != r) || (fDynB && fShapeB.size() != r))
         throw std::runtime_error("SOFIE Binary Op: with a run-time batch the batched operand must have the rank of the result");
      if ((fDynA && !fDynB && fShapeB.size() == r && fShapeB[0] != 1) || (fDynB && !fDynA && fShapeA.size() == r && fShapeA[0] != 1))
         throw std::runtime_error("SOFIE Binary Op: an operand without the batch cannot have a leading dimension above 1");
      if (r > 6)
         throw std::runtime_error("SOFIE Binary Op: rank above 6 is not supported");
      fShapeA.insert(fShapeA.begin(), r - fShapeA.size(), 1);
      fShapeB.insert(fShapeB.begin(), r - fShapeB.size(), 1);
      fShapeY.resize(r);
      for (std::size_t i = 0; i < r; ++i) {
         if (fShapeA[i] != fShapeB[i] && fShapeA[i] != 1 && fShapeB[i] != 1)
            throw std::runtime_error("SOFIE Binary Op: shapes " + ConvertShapeToString(fShapeA) + " and " + ConvertShapeToString(fShapeB) +
                                     " cannot be broadcast");
         fShapeY[i] = std::max(fShapeA[i], fShapeB[i]);
      }
      // two constants: the sum is computed now (core/inc/SOFIE/operators/ROperator_BasicBinary.hxx:191-257)
      if (model.IsConstantTensor(fNA) && model.IsConstantTensor(fNB) && model.GetTensorType(fNA) == ETensorType::FLOAT &&
          model.GetTensorType(fNB) == ETensorType::FLOAT) {
         const float *a = static_cast<const float *>(model.GetInitializedTensorData(fNA).get());
         const float *b = static_cast<const float *>(model.GetInitializedTensorData(fNB).get());
         std::vector<float> y(ConvertShapeToLength(fShapeY));
         std::vector<std::size_t> idx(r, 0);
         for (std::size_t i = 0; i < y.size(); ++i) {
            std::size_t ia = 0, ib = 0;
            for (std::size_t d = 0; d < r; ++d) {
               ia = ia * fShapeA[d] + (fShapeA[d] == 1 ? 0 : idx[d]);
               ib = ib * fShapeB[d] + (fShapeB[d] == 1 ? 0 : idx[d]);
            }
            y[i] = BinaryValue(Op, a[ia], b[ib], fParam);
            for (std::size_t d = r; d-- > 0;) {
               if (++idx[d] < fShapeY[d])
                  break;
               idx[d] = 0;
            }
         }
         model.AddConstantTensor(fNY, ETensorType::FLOAT, fShapeY, y.data());
         fIsOutputConstant = true;
         return;
      }
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShapeY, fDynA || fDynB);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      if (fIsOutputConstant)
         return "\n" + SP + "//------ " + BinaryName(Op) + " " + opName + " -> " + fNY + ": constants only, computed when the code was generated\n";
      std::stringstream out;
      auto list = [](const std::vector<std::size_t> &v, bool batched) {
         std::string s = "{";
         for (std::size_t i = 0; i < 6; ++i)
            s += BatchScaled(batched && i == 0, i < v.size() ? v[i] : 1) + (i < 5 ? ", " : "");
         return s + "}";
      };
      out << "\n" << SP << "//------ " << BinaryName(Op) << " " << opName << " --> " << ConvertShapeToString(fShapeY) << "\n";
      out << SP << "{\n";
      out << SP << "   " << "sofie_add_desc d{" << fShapeY.size() << ", " << list(fShapeY, fDynA || fDynB) << ", " << list(fShapeA, fDynA) << ", " << list(fShapeB, fDynB)
          << ", tensor_" << fNA << ", tensor_" << fNB << ", tensor_" << fNY << "};\n";
      if (Op == Add)
         out << SP << "   " << "detail::Check(sofie_hip_add_f32(fCtx, &d), \"" << opName << " Add\");\n";
      else
         out << SP << "   " << "detail::Check(sofie_hip_binary_f32(fCtx, &d, " << BinaryRuntimeCode(Op) << ", " << FloatLiteral(fParam) << "), \"" << opName << " "
             << BinaryName(Op) << "\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   std::string fNA, fNB, fNY;
   std::vector<std::size_t> fShapeA, fShapeB, fShapeY;
   float fParam = 0.f;
   bool fDynA = false, fDynB = false, fIsOutputConstant = false;
};

} // namespace SOFIE_HIP
#endif
