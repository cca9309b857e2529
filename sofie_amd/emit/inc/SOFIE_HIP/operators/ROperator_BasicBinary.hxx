// Broadcast Add (core/inc/SOFIE/operators/ROperator_BasicBinary.hxx, the Add instance): one
// sofie_hip_add_f32 call with the multidirectional broadcast resolved at generation time.
#ifndef SOFIE_HIP_ROPERATOR_BASICBINARY
#define SOFIE_HIP_ROPERATOR_BASICBINARY

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

enum EBasicBinaryOperator { Add };

template <typename T, EBasicBinaryOperator Op>
class ROperator_BasicBinary final : public ROperator {
   static_assert(std::is_same<T, float>::value && Op == Add, "only the float Add is on this backend's path");

public:
   ROperator_BasicBinary(std::string nameA, std::string nameB, std::string nameY)
      : fNA(UTILITY::Clean_name(nameA)), fNB(UTILITY::Clean_name(nameB)), fNY(UTILITY::Clean_name(nameY))
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
            y[i] = a[ia] + b[ib];
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
         return "\n" + SP + "//------ Add " + opName + " -> " + fNY + ": a sum of constants, computed when the code was generated\n";
      std::stringstream out;
      auto list = [](const std::vector<std::size_t> &v, bool batched) {
         std::string s = "{";
         for (std::size_t i = 0; i < 6; ++i)
            s += BatchScaled(batched && i == 0, i < v.size() ? v[i] : 1) + (i < 5 ? ", " : "");
         return s + "}";
      };
      out << "\n" << SP << "//------ Add " << opName << " --> " << ConvertShapeToString(fShapeY) << "\n";
      out << SP << "{\n";
      out << SP << "   " << "sofie_add_desc d{" << fShapeY.size() << ", " << list(fShapeY, fDynA || fDynB) << ", " << list(fShapeA, fDynA) << ", " << list(fShapeB, fDynB)
          << ", tensor_" << fNA << ", tensor_" << fNB << ", tensor_" << fNY << "};\n";
      out << SP << "   " << "detail::Check(sofie_hip_add_f32(fCtx, &d), \"" << opName << " Add\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   std::string fNA, fNB, fNY;
   std::vector<std::size_t> fShapeA, fShapeB, fShapeY;
   bool fDynA = false, fDynB = false, fIsOutputConstant = false;
};

} // namespace SOFIE_HIP
#endif
