// LayerNormalization (core/inc/SOFIE/operators/ROperator_LayerNormalization.hxx: constructor :54-64, the loops :247-312;
// attributes axis = -1, epsilon = 1e-5, stash_type = 1 as parsers/src/ParseLayerNormalization.cxx reads them).  The optional outputs
// Mean and InvStdDev are written when the node names them.
#ifndef SOFIE_HIP_ROPERATOR_LAYERNORMALIZATION
#define SOFIE_HIP_ROPERATOR_LAYERNORMALIZATION

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

template <typename T>
class ROperator_LayerNormalization final : public ROperator {
   static_assert(std::is_same<T, float>::value, "SOFIE Encountered unsupported type parsing a LayerNormalization operator");

public:
   ROperator_LayerNormalization(int axis, float epsilon, std::size_t stashType, const std::string &nameX, const std::string &nameScale,
                                const std::string &nameB, const std::string &nameY, const std::string &nameMean, const std::string &nameInvStdDev)
      : fAttrAxis(axis), fAttrEpsilon(epsilon), fAttrStashType(stashType), fNX(UTILITY::Clean_name(nameX)), fNScale(UTILITY::Clean_name(nameScale)),
        fNB(UTILITY::Clean_name(nameB)), fNY(UTILITY::Clean_name(nameY)), fNMean(UTILITY::Clean_name(nameMean)), fNInvStdDev(UTILITY::Clean_name(nameInvStdDev))
   {
      fInputTensorNames = {fNX, fNScale};
      if (!fNB.empty())
         fInputTensorNames.push_back(fNB);
      fOutputTensorNames = {fNY};
      if (!fNMean.empty())
         fOutputTensorNames.push_back(fNMean);
      if (!fNInvStdDev.empty())
         fOutputTensorNames.push_back(fNInvStdDev);
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE LayerNormalization Op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT || model.GetTensorLayout(fNX) != kLayoutNCHW)
         throw std::runtime_error("SOFIE LayerNormalization Op: input tensor " + fNX + " must be float in the ONNX layout");
      fShapeX = model.GetTensorShape(fNX);
      const int rank = static_cast<int>(fShapeX.size());
      if (fAttrAxis < -rank || fAttrAxis >= rank)
         throw std::runtime_error("SOFIE LayerNormalization Op: axis " + std::to_string(fAttrAxis) + " is out of range for " + fNX);
      fAxis = static_cast<std::size_t>(fAttrAxis < 0 ? fAttrAxis + rank : fAttrAxis);
      fDynamic = model.IsDynamicTensor(fNX);
      if (fDynamic && fAxis == 0)
         throw std::runtime_error("SOFIE LayerNormalization Op: the run-time batch of " + fNX + " cannot be normalised over");
      fRows = fLength = 1;
      for (std::size_t i = 0; i < fShapeX.size(); ++i)
         (i < fAxis ? fRows : fLength) *= fShapeX[i];
      if (fLength == 0 || fLength > 0x7fffffffu)
         throw std::runtime_error("SOFIE LayerNormalization Op: normalised length of " + fNX + " is out of range");
      // scale and bias cover the normalised dimensions element by element
      for (auto *n : {&fNScale, &fNB}) {
         if (n->empty())
            continue;
         if (!model.CheckIfTensorAlreadyExist(*n) || model.GetTensorType(*n) != ETensorType::FLOAT || model.IsDynamicTensor(*n) ||
             ConvertShapeToLength(model.GetTensorShape(*n)) != fLength)
            throw std::runtime_error("SOFIE LayerNormalization Op: " + *n + " must be a float tensor of the " + std::to_string(fLength) +
                                     " normalised elements (broadcast scale or bias is not supported)");
      }
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShapeX, fDynamic);
      // the statistics keep the leading dimensions and have 1 in the normalised ones
      std::vector<std::size_t> stat(fShapeX.size(), 1);
      for (std::size_t i = 0; i < fAxis; ++i)
         stat[i] = fShapeX[i];
      if (!fNMean.empty())
         model.AddIntermediateTensor(fNMean, ETensorType::FLOAT, stat, fDynamic);
      if (!fNInvStdDev.empty())
         model.AddIntermediateTensor(fNInvStdDev, ETensorType::FLOAT, stat, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- LayerNormalization " << opName << " " << ConvertShapeToString(fShapeX) << ", axis " << fAxis << "\n";
      out << SP << "detail::Check(sofie_hip_layernorm_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", tensor_" << fNScale << ", "
          << (fNB.empty() ? std::string("nullptr") : "tensor_" + fNB) << ", " << BatchScaled(fDynamic, fRows) << ", " << fLength << ", " << FloatLiteral(fAttrEpsilon)
          << ", " << (fNMean.empty() ? std::string("nullptr") : "tensor_" + fNMean) << ", " << (fNInvStdDev.empty() ? std::string("nullptr") : "tensor_" + fNInvStdDev)
          << "), \"" << opName << " LayerNormalization\");\n";
      return out.str();
   }

private:
   int fAttrAxis;
   float fAttrEpsilon;
   std::size_t fAttrStashType;
   std::string fNX, fNScale, fNB, fNY, fNMean, fNInvStdDev;
   std::vector<std::size_t> fShapeX;
   std::size_t fAxis = 0, fRows = 1, fLength = 1;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
