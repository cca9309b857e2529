// Quantised operators.  The reference has none (its operator registry, parsers/src/RModelParser_ONNX.cxx:279-367,
// and its float-only Gemm, core/inc/SOFIE/operators/ROperator_Gemm.hxx:67); these follow its operator
// contract and the ONNX definitions:
//   QuantizeLinear   q = sat8(rne(x / scale))                  per tensor, zero point 0
//   DequantizeLinear y = float(q) * scale                      int8 or int32 input
//   MatMulInteger    acc = A_i8 x B_i8 in int32
//   QGemm            MatMulInteger with the bias / Relu / DequantizeLinear / QuantizeLinear that follow it
//                    folded into the store of the matrix-core kernel (what the generator's fusion builds).
#ifndef SOFIE_HIP_ROPERATOR_QUANTIZED
#define SOFIE_HIP_ROPERATOR_QUANTIZED

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

class ROperator_QuantizeLinear final : public ROperator {
public:
   // scale: name of a float scalar initializer
   ROperator_QuantizeLinear(std::string nameX, std::string nameScale, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNS(UTILITY::Clean_name(nameScale)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::QUANTIZE;
   }
   const std::string &ScaleName() const { return fNS; }
   const std::string &OutputName() const { return fNY; }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE QuantizeLinear Op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE QuantizeLinear Op: input tensor " + fNX + " is not float");
      fScale = model.GetScalarInitializer(fNS);
      if (!(fScale > 0))
         throw std::runtime_error("SOFIE QuantizeLinear Op: scale " + fNS + " must be positive");
      fShape = model.GetTensorShape(fNX);
      fDynamic = model.IsDynamicTensor(fNX);
      model.AddIntermediateTensor(fNY, ETensorType::INT8, fShape, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//------ QuantizeLinear " << opName << "\n";
      out << SP << "detail::Check(sofie_hip_quantize_linear(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << BatchScaled(fDynamic, ConvertShapeToLength(fShape))
          << ", " << FloatLiteral(fScale) << "), \"" << opName << " QuantizeLinear\");\n";
      return out.str();
   }

private:
   std::string fNX, fNS, fNY;
   float fScale = 0;
   std::vector<std::size_t> fShape;
   bool fDynamic = false;
};

class ROperator_DequantizeLinear final : public ROperator {
public:
   ROperator_DequantizeLinear(std::string nameX, std::string nameScale, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNS(UTILITY::Clean_name(nameScale)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::DEQUANTIZE;
   }
   const std::string &ScaleName() const { return fNS; }
   const std::string &OutputName() const { return fNY; }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE DequantizeLinear Op Input Tensor " + fNX + " is not found in model");
      fType = model.GetTensorType(fNX);
      if (fType != ETensorType::INT8 && fType != ETensorType::INT32)
         throw std::runtime_error("SOFIE DequantizeLinear Op: input tensor " + fNX + " is neither int8 nor int32");
      fScale = model.GetScalarInitializer(fNS);
      fShape = model.GetTensorShape(fNX);
      fDynamic = model.IsDynamicTensor(fNX);
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShape, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//------ DequantizeLinear " << opName << "\n";
      out << SP << "detail::Check(sofie_hip_dequantize_linear_" << (fType == ETensorType::INT8 ? "i8" : "i32") << "(fCtx, tensor_" << fNY
          << ", tensor_" << fNX << ", " << BatchScaled(fDynamic, ConvertShapeToLength(fShape)) << ", " << FloatLiteral(fScale) << "), \"" << opName
          << " DequantizeLinear\");\n";
      return out.str();
   }

private:
   std::string fNX, fNS, fNY;
   float fScale = 0;
   ETensorType fType = ETensorType::INT8;
   std::vector<std::size_t> fShape;
   bool fDynamic = false;
};

// int8 x int8 -> int32 product with everything that can ride on its store.  As a plain MatMulInteger the
// output is int32; the generator's fusion (or a model builder) may attach, in this order:
//   bias (int32 [N], added to the accumulator) -> Relu on the accumulator -> DequantizeLinear(scale)
//   -> QuantizeLinear(q_scale) of the next layer, or a per-channel requantisation scale[N] (+ Relu after it).
class ROperator_QGemm final : public ROperator {
public:
   enum class Out { I32, F32, I8_REQUANT, I8_DQQ };
   // A [M,K] int8 activations, B [K,N] int8 weights (an initializer: re-laid out once to [N,K])
   ROperator_QGemm(std::string nameA, std::string nameB, std::string nameY)
      : fNA(UTILITY::Clean_name(nameA)), fNB(UTILITY::Clean_name(nameB)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNA, fNB};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::QGEMM;
   }
   void SetBias(const std::string &nameBias)
   {
      fNBias = UTILITY::Clean_name(nameBias);
      fInputTensorNames.push_back(fNBias);
   }
   void SetReluOnAccumulator() { fReluAcc = true; }
   void SetDequantize(float scale) { fOut = Out::F32; fScale = scale; }
   void SetDequantizeQuantize(float scale, float qscale) { fOut = Out::I8_DQQ; fScale = scale; fQScale = qscale; }
   // per-output-channel requantisation: scale tensor [N] float; relu after the rounding
   void SetRequantize(const std::string &nameScale, bool reluOut)
   {
      fOut = Out::I8_REQUANT;
      fNScale = UTILITY::Clean_name(nameScale);
      fInputTensorNames.push_back(fNScale);
      fReluOut = reluOut;
   }
   void SetOutputName(const std::string &name)
   {
      fNY = UTILITY::Clean_name(name);
      fOutputTensorNames = {fNY};
   }
   void SetReluOnOutput() { fReluOut = true; }
   bool ReluOnOutput() const { return fReluOut; }
   Out OutputKind() const { return fOut; }
   float DequantScale() const { return fScale; }
   bool ReluOnAccumulator() const { return fReluAcc; }

   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNA) || !model.CheckIfTensorAlreadyExist(fNB))
         throw std::runtime_error("SOFIE QGemm Op Input Tensor " + fNA + " or " + fNB + " is not found in model");
      if (model.GetTensorType(fNA) != ETensorType::INT8 || model.GetTensorType(fNB) != ETensorType::INT8)
         throw std::runtime_error("SOFIE QGemm Op: both operands must be int8");
      auto sA = model.GetTensorShape(fNA), sB = model.GetTensorShape(fNB);
      if (sA.size() != 2 || sB.size() != 2 || sA[1] != sB[0])
         throw std::runtime_error("SOFIE QGemm Op: shapes " + ConvertShapeToString(sA) + " and " + ConvertShapeToString(sB) + " do not form a product");
      fM = sA[0];
      fK = sA[1];
      fN = sB[1];
      fWeightIsInitializer = model.IsInitializedTensor(fNB);
      fDynamic = model.IsDynamicTensor(fNA);
      if (model.IsDynamicTensor(fNB))
         throw std::runtime_error("SOFIE QGemm Op: a run-time batch must be the row dimension of A");
      if (!fNBias.empty()) {
         if (!model.CheckIfTensorAlreadyExist(fNBias) || model.GetTensorType(fNBias) != ETensorType::INT32 ||
             ConvertShapeToLength(model.GetTensorShape(fNBias)) != fN)
            throw std::runtime_error("SOFIE QGemm Op: bias " + fNBias + " must be an int32 tensor of " + std::to_string(fN) + " elements");
      }
      if (!fNScale.empty()) {
         if (!model.CheckIfTensorAlreadyExist(fNScale) || model.GetTensorType(fNScale) != ETensorType::FLOAT ||
             ConvertShapeToLength(model.GetTensorShape(fNScale)) != fN)
            throw std::runtime_error("SOFIE QGemm Op: scale " + fNScale + " must be a float tensor of " + std::to_string(fN) + " elements");
      }
      const ETensorType ty = fOut == Out::I32 ? ETensorType::INT32 : fOut == Out::F32 ? ETensorType::FLOAT : ETensorType::INT8;
      model.AddIntermediateTensor(fNY, ty, {fM, fN}, fDynamic);
   }
   // a constant B is re-laid out once into [N,K] (K contiguous, what the matrix-core kernel reads)
   std::vector<std::pair<std::string, std::size_t>> GetPersistentBuffers() override
   {
      if (!fWeightIsInitializer)
         return {};
      return {{"packed_" + fNB, fK * fN}};
   }
   std::string GenerateInitCode_GPU_HIP() override
   {
      if (!fWeightIsInitializer)
         return "";
      std::stringstream out;
      out << SP << "   " << "detail::Check(sofie_hip_transpose_i8(fCtx, packed_" << fNB << ", tensor_" << fNB << ", " << fK << ", " << fN
          << ", 0, 0), \"re-layout of " << fNB << "\");\n";
      return out.str();
   }
   std::size_t GetWorkspaceBytes() override { return fWeightIsInitializer ? 0 : ((fK * fN + 255) / 256) * 256; }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      const std::string ws = "workspace_op_" + opName;
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//--------- QGemm " << opName << " int8 { " << fM << " , " << fK << " } * { " << fK << " , " << fN << " } -> " << fNY << "\n";
      out << SP << "{\n";
      out << SP << "   " << "sofie_gemm_i8_desc d{};\n";
      out << SP << "   " << "d.M = " << BatchScaledInt(fDynamic, fM) << "; d.N = " << fN << "; d.K = " << fK << ";\n";
      if (fWeightIsInitializer)
         out << SP << "   " << "d.A = tensor_" << fNA << "; d.B = packed_" << fNB << "; d.transB = 1;\n";
      else
         out << SP << "   " << "d.A = tensor_" << fNA << "; d.B = tensor_" << fNB << "; d.transB = 0; d.workspace = " << ws
             << "; d.workspace_bytes = " << GetWorkspaceBytes() << ";\n";
      out << SP << "   " << "d.bias = " << (fNBias.empty() ? "nullptr" : "tensor_" + fNBias) << "; d.scale = "
          << (fNScale.empty() ? "nullptr" : "tensor_" + fNScale) << "; d.scale_scalar = " << FloatLiteral(fScale) << "; d.q_scale = "
          << FloatLiteral(fQScale) << ";\n";
      const char *outName = fOut == Out::I32 ? "SOFIE_I8OUT_I32" : fOut == Out::F32 ? "SOFIE_I8OUT_F32" : fOut == Out::I8_REQUANT ? "SOFIE_I8OUT_I8" : "SOFIE_I8OUT_I8_DQQ";
      out << SP << "   " << "d.relu_acc = " << (fReluAcc ? 1 : 0) << "; d.relu_out = " << (fReluOut ? 1 : 0) << "; d.out = " << outName
          << "; d.Y = tensor_" << fNY << ";\n";
      out << SP << "   " << "detail::Check(sofie_hip_gemm_i8(fCtx, &d), \"" << opName << " QGemm\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   std::string fNA, fNB, fNY, fNBias, fNScale;
   std::size_t fM = 0, fN = 0, fK = 0;
   bool fWeightIsInitializer = false, fReluAcc = false, fReluOut = false, fDynamic = false;
   Out fOut = Out::I32;
   float fScale = 1.0f, fQScale = 1.0f;
};

// ONNX MatMulInteger (zero points 0): the plain int32 product
inline std::unique_ptr<ROperator_QGemm> MakeMatMulInteger(std::string nameA, std::string nameB, std::string nameY)
{
   return std::make_unique<ROperator_QGemm>(nameA, nameB, nameY);
}

// FP8 (OCP e4m3fn) Gemm: the fp32 activation is quantised per tensor at run time, the weight is an e4m3 initializer,
// the matrix cores accumulate in fp32, and scale, bias, activation and the fp32 / bf16 conversion are fused into the store:
//   Y = act( (e4m3(X / x_scale) x W_e4m3) * (x_scale * w_scale) + bias )
// The reference has no 8-bit floating type (core/inc/SOFIE/SOFIE_common.hxx:29-54 stops at BFLOAT16).
class ROperator_Fp8Gemm final : public ROperator {
public:
   ROperator_Fp8Gemm(float xScale, float wScale, int transB, std::string nameX, std::string nameW, std::string nameBias,
                     EActivationType act, ETensorType outType, std::string nameY)
      : fXScale(xScale), fWScale(wScale), fTransB(transB), fNX(UTILITY::Clean_name(nameX)), fNW(UTILITY::Clean_name(nameW)),
        fNBias(UTILITY::Clean_name(nameBias)), fAct(act), fOutType(outType), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX, fNW};
      if (!fNBias.empty())
         fInputTensorNames.push_back(fNBias);
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::QGEMM;
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX) || !model.CheckIfTensorAlreadyExist(fNW))
         throw std::runtime_error("SOFIE Fp8Gemm Op Input Tensor " + fNX + " or " + fNW + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Fp8Gemm Op: input tensor " + fNX + " is not float");
      if (!model.IsInitializedTensor(fNW) || model.GetTensorType(fNW) != ETensorType::FLOAT8E4M3FN)
         throw std::runtime_error("SOFIE Fp8Gemm Op: weight tensor " + fNW + " must be an e4m3 initializer");
      if (!(fXScale > 0) || !(fWScale > 0))
         throw std::runtime_error("SOFIE Fp8Gemm Op: scales must be positive");
      if (fOutType != ETensorType::FLOAT && fOutType != ETensorType::BFLOAT16)
         throw std::runtime_error("SOFIE Fp8Gemm Op: the output is float or bfloat16");
      const auto sx = model.GetTensorShape(fNX), sw = model.GetTensorShape(fNW);
      if (sx.size() != 2 || sw.size() != 2)
         throw std::runtime_error("SOFIE Fp8Gemm Op: 2-D operands only");
      fM = sx[0];
      fK = sx[1];
      fN = fTransB ? sw[0] : sw[1];
      if ((fTransB ? sw[1] : sw[0]) != fK)
         throw std::runtime_error("SOFIE Fp8Gemm Op: shapes " + ConvertShapeToString(sx) + " and " + ConvertShapeToString(sw) + " do not agree");
      if (!fNBias.empty() && (!model.CheckIfTensorAlreadyExist(fNBias) || model.GetTensorType(fNBias) != ETensorType::FLOAT ||
                              ConvertShapeToLength(model.GetTensorShape(fNBias)) != fN))
         throw std::runtime_error("SOFIE Fp8Gemm Op: bias " + fNBias + " must be a float tensor of " + std::to_string(fN) + " elements");
      fDynamic = model.IsDynamicTensor(fNX);
      model.AddIntermediateTensor(fNY, fOutType, {fM, fN}, fDynamic);
   }
   std::vector<std::pair<std::string, std::size_t>> GetPersistentBuffers() override
   {
      if (fTransB)
         return {};
      return {{"packed_" + fNW, fK * fN}};
   }
   std::string GenerateInitCode_GPU_HIP() override
   {
      if (fTransB)
         return "";
      std::stringstream out;
      out << SP << "   " << "detail::Check(sofie_hip_transpose_i8(fCtx, packed_" << fNW << ", reinterpret_cast<const int8_t *>(tensor_" << fNW << "), "
          << fK << ", " << fN << ", 0, 0), \"re-layout of " << fNW << "\");\n";
      return out.str();
   }
   // the e4m3 copy of the activations: K bytes per row
   std::size_t GetWorkspaceBytes() override { return fDynamic ? fM * fK : ((fM * fK + 255) / 256) * 256; }
   bool WorkspacePerBatchEntry() const override { return fDynamic; }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      const std::string ws = "workspace_op_" + opName;
      opName = "op_" + opName;
      volatile float prod = fXScale * fWScale;
      std::stringstream out;
      out << "\n" << SP << "//--------- Fp8Gemm " << opName << " e4m3 { " << fM << " , " << fK << " } * { " << fK << " , " << fN << " } -> " << fNY << "\n";
      out << SP << "{\n";
      out << SP << "   " << "detail::Check(sofie_hip_quantize_fp8(fCtx, reinterpret_cast<uint8_t *>(" << ws << "), tensor_" << fNX << ", " << BatchScaled(fDynamic, fM * fK)
          << ", " << FloatLiteral(fXScale) << "), \"" << opName << " quantisation\");\n";
      out << SP << "   " << "sofie_gemm_fp8_desc d{};\n";
      out << SP << "   " << "d.M = " << BatchScaledInt(fDynamic, fM) << "; d.N = " << fN << "; d.K = " << fK << "; d.transB = 1;\n";
      out << SP << "   " << "d.A = reinterpret_cast<const uint8_t *>(" << ws << "); d.B = "
          << (fTransB ? "tensor_" + fNW : "reinterpret_cast<const uint8_t *>(packed_" + fNW + ")") << ";\n";
      out << SP << "   " << "d.bias = " << (fNBias.empty() ? "nullptr" : "tensor_" + fNBias) << "; d.scale = " << FloatLiteral(prod)
          << "; d.act = " << ActivationEnumName(fAct) << "; d.out = " << (fOutType == ETensorType::FLOAT ? "SOFIE_F8OUT_F32" : "SOFIE_F8OUT_BF16")
          << "; d.Y = tensor_" << fNY << ";\n";
      out << SP << "   " << "detail::Check(sofie_hip_gemm_fp8(fCtx, &d), \"" << opName << " Fp8Gemm\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   float fXScale, fWScale;
   int fTransB;
   std::string fNX, fNW, fNBias;
   EActivationType fAct;
   ETensorType fOutType;
   std::string fNY;
   std::size_t fM = 0, fN = 0, fK = 0;
   bool fDynamic = false;
};

// int8 Relu on an int32 accumulator tensor is only meaningful fused; as a stand-alone operator on int32 it
// is not emitted (the fusion always removes it).

} // namespace SOFIE_HIP
#endif
