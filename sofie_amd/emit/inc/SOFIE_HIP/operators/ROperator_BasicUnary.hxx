// Stand-alone activation operators (Relu, LeakyRelu, Sigmoid, Gelu, Tanh): the emitters of
// core/inc/SOFIE/operators/ROperator_Relu.hxx, _LeakyRelu.hxx, _Sigmoid.hxx, _Gelu.hxx, _Tanh.hxx as one
// class; each emits one sofie_hip_unary_f32 call, unless the generator has fused it into the producing
// Gemm or Conv.
#ifndef SOFIE_HIP_ROPERATOR_BASICUNARY
#define SOFIE_HIP_ROPERATOR_BASICUNARY

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

class ROperator_Activation : public ROperator {
public:
   ROperator_Activation(EActivationType act, float alpha, std::string nameX, std::string nameY)
      : fAct(act), fAlpha(alpha), fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::UNARY;
   }
   EActivationType Activation() const { return fAct; }
   float Alpha() const { return fAlpha; }
   const std::string &OutputName() const { return fNY; }

   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE Activation Op Input Tensor " + fNX + " is not found in model");
      fType = model.GetTensorType(fNX);
      // a Relu on the int32 accumulator of a MatMulInteger only exists fused into that product's store
      if (fType != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Activation Op: input tensor " + fNX + " is not float (an integer Relu is only emitted fused "
                                  "into the MatMulInteger that produces its input)");
      fShape = model.GetTensorShape(fNX);
      fDynamic = model.IsDynamicTensor(fNX);
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShape, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//------ " << ActivationEnumName(fAct) << " " << opName << "\n";
      out << SP << "detail::Check(sofie_hip_unary_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << BatchScaled(fDynamic, ConvertShapeToLength(fShape))
          << ", " << ActivationEnumName(fAct) << ", " << FloatLiteral(fAlpha) << "), \"" << opName << " activation\");\n";
      return out.str();
   }

protected:
   EActivationType fAct;
   float fAlpha;
   std::string fNX, fNY;
   std::vector<std::size_t> fShape;
   ETensorType fType = ETensorType::FLOAT;
   bool fDynamic = false;
};

// the reference's class names
template <typename T>
struct ROperator_Relu : ROperator_Activation {
   ROperator_Relu(std::string x, std::string y) : ROperator_Activation(EActivationType::RELU, 0.f, x, y) {}
};
template <typename T>
struct ROperator_Sigmoid : ROperator_Activation {
   ROperator_Sigmoid(std::string x, std::string y) : ROperator_Activation(EActivationType::SIGMOID, 0.f, x, y) {}
};
template <typename T>
struct ROperator_Tanh : ROperator_Activation {
   ROperator_Tanh(std::string x, std::string y) : ROperator_Activation(EActivationType::TANH, 0.f, x, y) {}
};
template <typename T>
struct ROperator_LeakyRelu : ROperator_Activation {
   ROperator_LeakyRelu(float alpha, std::string x, std::string y) : ROperator_Activation(EActivationType::LEAKYRELU, alpha, x, y) {}
};
template <typename T>
struct ROperator_Gelu : ROperator_Activation {
   // approximate: "none" (erf form) or "tanh"
   ROperator_Gelu(std::string approximate, std::string x, std::string y)
      : ROperator_Activation(approximate == "tanh" ? EActivationType::GELU_TANH : EActivationType::GELU, 0.f, x, y)
   {
      if (approximate != "tanh" && approximate != "none")
         throw std::runtime_error("SOFIE Gelu Op: unknown approximation " + approximate);
   }
};

} // namespace SOFIE_HIP
#endif
