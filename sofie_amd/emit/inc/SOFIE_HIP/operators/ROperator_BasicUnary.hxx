// One-to-one float operators: the activations (core/inc/SOFIE/operators/ROperator_Relu.hxx, _LeakyRelu.hxx,
// _Sigmoid.hxx, _Gelu.hxx, _Tanh.hxx), the basic unary operators (ROperator_BasicUnary.hxx) and Clip
// (ROperator_Clip.hxx) as one class.  The generator folds such an operator into the Gemm or Conv that produces
// its input, or into the one-to-one operator before it (the reference's elementwise fusion,
// core/inc/SOFIE/operators/ROperator_ALPAKA.hxx:57-76); what remains emits one sofie_hip_unary_f32 or
// sofie_hip_unary_chain_f32 call.
#ifndef SOFIE_HIP_ROPERATOR_BASICUNARY
#define SOFIE_HIP_ROPERATOR_BASICUNARY

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

class ROperator_Activation : public ROperator {
public:
   ROperator_Activation(EActivationType act, float alpha, std::string nameX, std::string nameY, float beta = 0.f)
      : fAct(act), fAlpha(alpha), fBeta(beta), fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::UNARY;
   }
   EActivationType Activation() const { return fAct; }
   float Alpha() const { return fAlpha; }
   float Beta() const { return fBeta; }
   const std::string &OutputName() const { return fNY; }
   // this operator followed by the ones folded into it
   std::vector<PostOp> Chain() const
   {
      std::vector<PostOp> c{PostOp{fAct, fAlpha, fBeta}};
      c.insert(c.end(), fPost.begin(), fPost.end());
      return c;
   }
   void AddPostOp(const PostOp &op, const std::string &newOutput)
   {
      fPost.push_back(op);
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }

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
      out << "\n" << SP << "//------ " << ActivationEnumName(fAct);
      for (auto &p : fPost)
         out << " -> " << ActivationEnumName(p.act);
      out << " " << opName << "\n";
      if (fPost.empty() && fAct != EActivationType::CLIP && fAct != EActivationType::SELU) { // those two carry a second parameter
         out << SP << "detail::Check(sofie_hip_unary_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", "
             << BatchScaled(fDynamic, ConvertShapeToLength(fShape)) << ", " << ActivationEnumName(fAct) << ", " << FloatLiteral(fAlpha) << "), \""
             << opName << " activation\");\n";
         return out.str();
      }
      out << SP << "{\n";
      out << SP << "   " << PostOpsDeclaration("ops", Chain()) << "\n";
      out << SP << "   " << "detail::Check(sofie_hip_unary_chain_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", "
          << BatchScaled(fDynamic, ConvertShapeToLength(fShape)) << ", &ops), \"" << opName << " one-to-one chain\");\n";
      out << SP << "}\n";
      return out.str();
   }

protected:
   EActivationType fAct;
   float fAlpha, fBeta = 0.f;
   std::vector<PostOp> fPost;
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

// ROperator_BasicUnary<T, Op> of the reference (core/inc/SOFIE/operators/ROperator_BasicUnary.hxx:106-170)
inline EActivationType BasicUnaryActivation(EBasicUnaryOperator op)
{
   switch (op) {
   case EBasicUnaryOperator::kReciprocal: return EActivationType::RECIPROCAL;
   case EBasicUnaryOperator::kSqrt: return EActivationType::SQRT;
   case EBasicUnaryOperator::kNeg: return EActivationType::NEG;
   case EBasicUnaryOperator::kExp: return EActivationType::EXP;
   case EBasicUnaryOperator::kLog: return EActivationType::LOG;
   case EBasicUnaryOperator::kSin: return EActivationType::SIN;
   case EBasicUnaryOperator::kCos: return EActivationType::COS;
   case EBasicUnaryOperator::kAbs: return EActivationType::ABS;
   case EBasicUnaryOperator::kSoftplus: return EActivationType::SOFTPLUS;
   case EBasicUnaryOperator::kAtan: return EActivationType::ATAN;
   case EBasicUnaryOperator::kFloor: return EActivationType::FLOOR;
   case EBasicUnaryOperator::kAsinh: return EActivationType::ASINH;
   case EBasicUnaryOperator::kAcosh: return EActivationType::ACOSH;
   default: return EActivationType::ATANH;
   }
}
template <typename T, EBasicUnaryOperator Op>
struct ROperator_BasicUnary : ROperator_Activation {
   ROperator_BasicUnary(std::string x, std::string y) : ROperator_Activation(BasicUnaryActivation(Op), 0.f, x, y) {}
};
// Clip with constant bounds: Y = max(min, min(max, X)) (core/inc/SOFIE/operators/ROperator_Clip.hxx:18, 92-100)
template <typename T>
struct ROperator_Clip : ROperator_Activation {
   ROperator_Clip(std::string x, std::string y, T minVal, T maxVal) : ROperator_Activation(EActivationType::CLIP, minVal, x, y, maxVal) {}
};
// Selu: gamma * (max(0, x) + min(0, alpha * (exp(x) - 1))) (core/inc/SOFIE/operators/ROperator_Selu.hxx:16-62)
template <typename T>
struct ROperator_Selu : ROperator_Activation {
   ROperator_Selu(std::string x, std::string y) : ROperator_Selu(1.67326319217681884765625f, 1.05070102214813232421875f, x, y) {}
   ROperator_Selu(float alpha, float gamma, std::string x, std::string y) : ROperator_Activation(EActivationType::SELU, alpha, x, y, gamma) {}
};
// Elu: x >= 0 ? x : alpha * (exp(x) - 1) (core/inc/SOFIE/operators/ROperator_Elu.hxx:16-74)
template <typename T>
struct ROperator_Elu : ROperator_Activation {
   ROperator_Elu(float alpha, std::string x, std::string y) : ROperator_Activation(EActivationType::ELU, alpha, x, y) {}
};
// Erf: std::erf(x) (core/inc/SOFIE/operators/ROperator_Erf.hxx)
template <typename T>
struct ROperator_Erf : ROperator_Activation {
   ROperator_Erf(std::string x, std::string y) : ROperator_Activation(EActivationType::ERF, 0.f, x, y) {}
};
// HardSigmoid: max(0, min(1, alpha * x + beta)), alpha = 0.2, beta = 0.5 (core/inc/SOFIE/operators/ROperator_HardSigmoid.hxx:15-25, 71-74)
template <typename T>
struct ROperator_HardSigmoid : ROperator_Activation {
   ROperator_HardSigmoid(float alpha, float beta, std::string x, std::string y) : ROperator_Activation(EActivationType::HARDSIGMOID, alpha, x, y, beta) {}
};
// HardSwish: x * max(0, min(1, x / 6 + 1 / 2)) (core/inc/SOFIE/operators/ROperator_HardSwish.hxx:56-60)
template <typename T>
struct ROperator_HardSwish : ROperator_Activation {
   ROperator_HardSwish(std::string x, std::string y) : ROperator_Activation(EActivationType::HARDSWISH, 0.f, x, y) {}
};
// Swish: x / (1 + exp(-x)) (core/inc/SOFIE/operators/ROperator_Swish.hxx:54-56)
template <typename T>
struct ROperator_Swish : ROperator_Activation {
   ROperator_Swish(std::string x, std::string y) : ROperator_Activation(EActivationType::SWISH, 0.f, x, y) {}
};
// Identity: a copy that the generator folds away wherever it follows another operator
template <typename T>
struct ROperator_Identity : ROperator_Activation {
   ROperator_Identity(std::string x, std::string y) : ROperator_Activation(EActivationType::UNDEFINED, 0.f, x, y) {}
};

} // namespace SOFIE_HIP
#endif
