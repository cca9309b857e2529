// BatchNormalization at inference (core/inc/SOFIE/operators/ROperator_BatchNormalization.hxx: same constructor
// arguments; Initialize forms fused_scale = scale / sqrt(var + epsilon) as an extra initialized tensor, :92-109;
// the loop computes (x - mean) * fused_scale + bias, :139-158), with the reference's BN + Relu fusion as a flag.
#ifndef SOFIE_HIP_ROPERATOR_BATCHNORMALIZATION
#define SOFIE_HIP_ROPERATOR_BATCHNORMALIZATION

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

#include <cmath>

namespace SOFIE_HIP {

template <typename T>
class ROperator_BatchNormalization final : public ROperator {
   static_assert(std::is_same<T, float>::value, "SOFIE Encountered unsupported type parsing a BatchNormalization operator");

public:
   ROperator_BatchNormalization(float epsilon, float momentum, std::size_t training_mode, std::string nameX, std::string nameScale,
                                std::string nameB, std::string nameMean, std::string nameVar, std::string nameY,
                                EActivationType activation = EActivationType::UNDEFINED)
      : fepsilon(epsilon), fmomentum(momentum), ftraining_mode(training_mode), fNX(UTILITY::Clean_name(nameX)),
        fNScale(UTILITY::Clean_name(nameScale)), fNB(UTILITY::Clean_name(nameB)), fNMean(UTILITY::Clean_name(nameMean)),
        fNVar(UTILITY::Clean_name(nameVar)), fNY(UTILITY::Clean_name(nameY)), fActivation(activation)
   {
      fNFusedScale = fNScale + "_fused_inv_std_dev";
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      if (activation != EActivationType::UNDEFINED && activation != EActivationType::RELU)
         throw std::runtime_error("SOFIE BatchNormalization Op: only a Relu can be fused");
   }
   bool HasActivation() const { return fActivation != EActivationType::UNDEFINED; }
   void FuseRelu(const std::string &newOutput)
   {
      fActivation = EActivationType::RELU;
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   void Initialize(RModel &model) override
   {
      if (ftraining_mode)
         throw std::runtime_error("SOFIE BatchNormalization Op: training mode is not supported");
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE BatchNormalization op Input Tensor " + fNX + " fnx is not found in model");
      for (auto *n : {&fNScale, &fNB, &fNMean, &fNVar})
         if (!model.IsInitializedTensor(*n) || model.GetTensorType(*n) != ETensorType::FLOAT)
            throw std::runtime_error("SOFIE BatchNormalization op Input Tensor " + *n + " is not a float initializer of the model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE BatchNormalization Op: input tensor " + fNX + " is not float");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() < 2 || fShapeX.size() > 4)
         throw std::runtime_error("SOFIE BatchNormalization Op input tensor " + fNX + " has wrong shape : " + ConvertShapeToString(fShapeX));
      const std::size_t channels = fShapeX[1];
      for (auto *n : {&fNScale, &fNB, &fNMean, &fNVar})
         if (model.GetTensorShape(*n).size() != 1 || model.GetTensorShape(*n)[0] != channels)
            throw std::runtime_error("SOFIE BatchNormalization '" + *n + "' tensor must be 1D (per-channel) with " + std::to_string(channels) + " elements");
      const float *scale = static_cast<const float *>(model.GetInitializedTensorData(fNScale).get());
      const float *var = static_cast<const float *>(model.GetInitializedTensorData(fNVar).get());
      std::vector<float> fused(channels);
      for (std::size_t i = 0; i < channels; ++i) {
         volatile float shifted = var[i] + fepsilon;
         fused[i] = scale[i] / std::sqrt(shifted);
      }
      model.AddInitializedTensor(fNFusedScale, ETensorType::FLOAT, {channels}, fused.data());
      fDynamic = model.IsDynamicTensor(fNX);
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShapeX, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      if (fShapeX.empty())
         throw std::runtime_error("SOFIE Batch Normalization called to Generate without being initialized first");
      std::size_t spatial = 1;
      for (std::size_t i = 2; i < fShapeX.size(); ++i)
         spatial *= fShapeX[i];
      std::stringstream out;
      out << "\n" << SP << "//---- BatchNorm" << (fActivation == EActivationType::RELU ? " + ReLU " : " ") << opName << "\n";
      out << SP << "detail::Check(sofie_hip_batchnorm_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", tensor_" << fNFusedScale << ", tensor_"
          << fNMean << ", tensor_" << fNB << ", " << BatchScaledInt(fDynamic, fShapeX[0]) << ", " << fShapeX[1] << ", " << spatial << ", "
          << (fActivation == EActivationType::RELU ? 1 : 0) << "), \"" << opName << " BatchNormalization\");\n";
      return out.str();
   }

private:
   float fepsilon = 1e-05f, fmomentum = 0.9f;
   std::size_t ftraining_mode = 0;
   std::string fNX, fNScale, fNB, fNMean, fNVar, fNY, fNFusedScale;
   std::vector<std::size_t> fShapeX;
   EActivationType fActivation;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
