// Softmax and LogSoftmax along one axis (core/inc/SOFIE/operators/ROperator_Softmax.hxx: constructor :27-30, the last-axis
// loop :82-119, any other axis :121-198; the axis attribute defaults to -1, parsers/src/ParseSoftmax.cxx:22-26).
#ifndef SOFIE_HIP_ROPERATOR_SOFTMAX
#define SOFIE_HIP_ROPERATOR_SOFTMAX

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

class ROperator_Softmax final : public ROperator {
public:
   ROperator_Softmax(int64_t attr_axis, std::string nameX, std::string nameY, bool logSoftmax = false)
      : fLogSoftmax(logSoftmax), fAttrAxis(attr_axis), fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE Softmax Op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Softmax Op: input tensor " + fNX + " is not float");
      fShape = model.GetTensorShape(fNX);
      const int64_t rank = static_cast<int64_t>(fShape.size());
      if (rank == 0 || fAttrAxis < -rank || fAttrAxis >= rank)
         throw std::runtime_error("SOFIE Softmax Op: axis " + std::to_string(fAttrAxis) + " is out of range for tensor " + fNX + " of rank " +
                                  std::to_string(rank));
      fAxis = static_cast<std::size_t>(fAttrAxis < 0 ? fAttrAxis + rank : fAttrAxis);
      fDynamic = model.IsDynamicTensor(fNX);
      if (fDynamic && fAxis == 0)
         throw std::runtime_error("SOFIE Softmax Op: the axis of " + fNX + " is its run-time batch dimension");
      if (fShape[fAxis] == 0 || fShape[fAxis] > 0x7fffffffu)
         throw std::runtime_error("SOFIE Softmax Op: axis length of " + fNX + " is out of range");
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShape, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::size_t outer = 1, inner = 1;
      for (std::size_t i = 0; i < fAxis; ++i)
         outer *= fShape[i];
      for (std::size_t i = fAxis + 1; i < fShape.size(); ++i)
         inner *= fShape[i];
      std::stringstream out;
      out << "\n" << SP << "//------- " << (fLogSoftmax ? "LogSoftmax " : "Softmax ") << opName << " ---> " << ConvertShapeToString(fShape) << ", axis " << fAxis << "\n";
      out << SP << "detail::Check(sofie_hip_softmax_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << BatchScaled(fDynamic, outer) << ", " << fShape[fAxis]
          << ", " << inner << ", " << (fLogSoftmax ? 1 : 0) << "), \"" << opName << " Softmax\");\n";
      return out.str();
   }

private:
   bool fLogSoftmax;
   int64_t fAttrAxis;
   std::size_t fAxis = 0;
   std::string fNX, fNY;
   std::vector<std::size_t> fShape;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
