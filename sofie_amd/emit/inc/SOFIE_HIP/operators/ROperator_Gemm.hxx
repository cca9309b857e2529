// Gemm / MatMul emitter for the gfx950 backend: the operator of core/inc/SOFIE/operators/ROperator_Gemm.hxx
// (same constructor arguments, same shape and bias rules), emitting one sofie_hip_gemm_f32 call with the
// bias broadcast and the activation fused into the kernel's store instead of Copy/Fill + Gemm_Call + Relu.
#ifndef SOFIE_HIP_ROPERATOR_GEMM
#define SOFIE_HIP_ROPERATOR_GEMM

#include "SOFIE_HIP/RModel.hxx"

#include <iomanip>
#include <limits>
#include <sstream>

namespace SOFIE_HIP {

inline const char *ActivationEnumName(EActivationType a)
{
   switch (a) {
   case EActivationType::RELU: return "SOFIE_ACT_RELU";
   case EActivationType::LEAKYRELU: return "SOFIE_ACT_LEAKYRELU";
   case EActivationType::SIGMOID: return "SOFIE_ACT_SIGMOID";
   case EActivationType::GELU: return "SOFIE_ACT_GELU";
   case EActivationType::GELU_TANH: return "SOFIE_ACT_GELU_TANH";
   case EActivationType::TANH: return "SOFIE_ACT_TANH";
   case EActivationType::RECIPROCAL: return "SOFIE_ACT_RECIPROCAL";
   case EActivationType::SQRT: return "SOFIE_ACT_SQRT";
   case EActivationType::NEG: return "SOFIE_ACT_NEG";
   case EActivationType::EXP: return "SOFIE_ACT_EXP";
   case EActivationType::LOG: return "SOFIE_ACT_LOG";
   case EActivationType::SIN: return "SOFIE_ACT_SIN";
   case EActivationType::COS: return "SOFIE_ACT_COS";
   case EActivationType::ABS: return "SOFIE_ACT_ABS";
   case EActivationType::SOFTPLUS: return "SOFIE_ACT_SOFTPLUS";
   case EActivationType::ATAN: return "SOFIE_ACT_ATAN";
   case EActivationType::FLOOR: return "SOFIE_ACT_FLOOR";
   case EActivationType::ASINH: return "SOFIE_ACT_ASINH";
   case EActivationType::ACOSH: return "SOFIE_ACT_ACOSH";
   case EActivationType::ATANH: return "SOFIE_ACT_ATANH";
   case EActivationType::CLIP: return "SOFIE_ACT_CLIP";
   case EActivationType::SELU: return "SOFIE_ACT_SELU";
   case EActivationType::ELU: return "SOFIE_ACT_ELU";
   case EActivationType::ERF: return "SOFIE_ACT_ERF";
   case EActivationType::HARDSIGMOID: return "SOFIE_ACT_HARDSIGMOID";
   case EActivationType::HARDSWISH: return "SOFIE_ACT_HARDSWISH";
   case EActivationType::SWISH: return "SOFIE_ACT_SWISH";
   default: return "SOFIE_ACT_NONE";
   }
}

// true for the activations an operator's own `act` field can hold (one parameter at most)
inline bool IsProducerActivation(EActivationType a) { return a >= EActivationType::RELU && a <= EActivationType::TANH; }

inline std::string FloatLiteral(float v)
{
   std::ostringstream s;
   s << std::setprecision(std::numeric_limits<float>::max_digits10) << v;
   std::string t = s.str();
   if (t.find_first_of(".eEn") == std::string::npos)
      t += ".0";
   return t + "f";
}

// `sofie_post_ops <name>{...};` for a chain of fused one-to-one operators
inline std::string PostOpsDeclaration(const std::string &name, const std::vector<PostOp> &ops)
{
   std::ostringstream s;
   s << "sofie_post_ops " << name << "{" << ops.size() << ", {";
   for (std::size_t i = 0; i < kMaxPostOps; ++i)
      s << (i < ops.size() ? ActivationEnumName(ops[i].act) : "SOFIE_ACT_NONE") << (i + 1 < kMaxPostOps ? ", " : "");
   s << "}, {";
   for (std::size_t i = 0; i < kMaxPostOps; ++i)
      s << FloatLiteral(i < ops.size() ? ops[i].alpha : 0.f) << (i + 1 < kMaxPostOps ? ", " : "");
   s << "}, {";
   for (std::size_t i = 0; i < kMaxPostOps; ++i)
      s << FloatLiteral(i < ops.size() ? ops[i].beta : 0.f) << (i + 1 < kMaxPostOps ? ", " : "");
   s << "}};";
   return s.str();
}

template <typename T>
class ROperator_Gemm final : public ROperator {
   static_assert(std::is_same<T, float>::value, "SOFIE - Unsupported type parsing a Gemm operator");

public:
   ROperator_Gemm(float alpha, float beta, int64_t transA, int64_t transB, std::string nameA, std::string nameB, std::string nameY,
                  EActivationType activation = EActivationType::UNDEFINED)
      : fAttrAlpha(alpha), fAttrBeta(beta), fAttrTransA(transA), fAttrTransB(transB), fNA(UTILITY::Clean_name(nameA)),
        fNB(UTILITY::Clean_name(nameB)), fNY(UTILITY::Clean_name(nameY)), fActivation(activation)
   {
      fInputTensorNames = {fNA, fNB};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::GEMM;
   }
   ROperator_Gemm(float alpha, float beta, int64_t transA, int64_t transB, std::string nameA, std::string nameB, std::string nameC,
                  std::string nameY, EActivationType activation = EActivationType::UNDEFINED)
      : fAttrAlpha(alpha), fAttrBeta(beta), fAttrTransA(transA), fAttrTransB(transB), fNA(UTILITY::Clean_name(nameA)),
        fNB(UTILITY::Clean_name(nameB)), fNC(UTILITY::Clean_name(nameC)), fNY(UTILITY::Clean_name(nameY)), fActivation(activation)
   {
      fInputTensorNames = {fNA, fNB, fNC};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::GEMM;
   }

   // used by the activation fusion of the generator (the reference's FuseGemmActivations,
   // core/src/RModel_Fusion_ALPAKA.cxx:367-416)
   bool HasActivation() const { return fActivation != EActivationType::UNDEFINED; }
   void FuseActivation(EActivationType a, float alpha, const std::string &newOutput)
   {
      fActivation = a;
      fActAlpha = alpha;
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   // further one-to-one operators behind the activation, applied in the kernel's store in this order
   std::size_t PostOpCount() const { return fPost.size(); }
   void AddPostOp(const PostOp &op, const std::string &newOutput)
   {
      fPost.push_back(op);
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }

   // A tensor of the product's shape that an Add behind this operator adds to it (a residual connection): it joins
   // the kernel's store, before the activation.  The generator calls this when the shapes agree (OutputShape below).
   bool HasResidual() const { return !fNR.empty(); }
   void SetResidual(const std::string &name, const std::string &newOutput)
   {
      fNR = UTILITY::Clean_name(name);
      fInputTensorNames.push_back(fNR);
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   const std::vector<std::size_t> &OutputShape() const { return fShapeY; }
   bool IsBatched() const { return fDynamic; }

   bool SupportsStridedInput() const override { return true; }

   void Initialize(RModel &model) override
   {
      ResolveShapes(model);
      // The operands A and B can be graph inputs read through the strides given to the Session (Options::kStridedInput).  A
      // matrix is described to the kernels by a row stride and a transpose flag, so one of an operand's two strides must be
      // 1; the plain 2-D product only (core/inc/SOFIE/operators/ROperator_Gemm.hxx:388-399 of the reference).
      fStridedA = model.IsStridedInputTensor(fNA);
      fStridedB = model.IsStridedInputTensor(fNB);
      if ((!fNC.empty() && model.IsStridedInputTensor(fNC)) || (!fNR.empty() && model.IsStridedInputTensor(fNR)))
         throw std::runtime_error("SOFIE Gemm Op - strided input is not supported for the bias (C)");
      if ((fStridedA || fStridedB) && (model.GetTensorShape(fNA).size() != 2 || model.GetTensorShape(fNB).size() != 2))
         throw std::runtime_error("SOFIE Gemm Op - strided input is only supported for a plain 2D Gemm "
                                  "(no MatMul batching, no low rank factorization)");
      fStoredA = model.GetTensorShape(fNA);
      fStoredB = model.GetTensorShape(fNB);
      if (!fNR.empty() && (!model.CheckIfTensorAlreadyExist(fNR) || model.GetTensorType(fNR) != ETensorType::FLOAT ||
                           model.GetTensorShape(fNR) != fShapeY || model.IsDynamicTensor(fNR) != fDynamic))
         throw std::runtime_error("SOFIE Gemm Op: residual tensor " + fNR + " does not have the shape of the product");
      // A product of weights only is computed now and becomes a constant of the model, with the loops of the reference
      // (core/inc/SOFIE/operators/ROperator_Gemm.hxx:317-373: plain 2-D operands, C of the product's own shape, Relu at most)
      const bool canFold = !fDynamic && fShapeA.size() <= 2 && fBatch == 1 && model.IsInitializedTensor(fNA) && model.IsInitializedTensor(fNB) &&
                           (fNC.empty() || (model.IsInitializedTensor(fNC) && fBiasMode == std::string("SOFIE_BIAS_FULL"))) && fNR.empty() &&
                           fPost.empty() && (fActivation == EActivationType::UNDEFINED || fActivation == EActivationType::RELU);
      if (canFold) {
         const float *dataA = static_cast<const float *>(model.GetInitializedTensorData(fNA).get());
         const float *dataB = static_cast<const float *>(model.GetInitializedTensorData(fNB).get());
         const std::size_t m = fM, n = fN, k = fK;
         std::vector<float> dataY(m * n, 0.f);
         for (std::size_t i = 0; i < m; i++) {
            for (std::size_t j = 0; j < n; j++) {
               float sum = 0.f;
               for (std::size_t p = 0; p < k; p++) {
                  const float aVal = fAttrTransA ? dataA[p * m + i] : dataA[i * k + p];
                  const float bVal = fAttrTransB ? dataB[j * k + p] : dataB[p * n + j];
                  volatile float prod = aVal * bVal; // one rounding per operation, no fused multiply-add
                  sum += prod;
               }
               dataY[i * n + j] = fAttrAlpha * sum;
            }
         }
         if (!fNC.empty()) {
            const float *dataC = static_cast<const float *>(model.GetInitializedTensorData(fNC).get());
            for (std::size_t idx = 0; idx < dataY.size(); idx++) {
               volatile float scaled = fAttrBeta * dataC[idx];
               dataY[idx] += scaled;
            }
         }
         if (fActivation == EActivationType::RELU)
            for (auto &v : dataY)
               v = std::max(v, 0.f);
         model.AddConstantTensor(fNY, ETensorType::FLOAT, fShapeY, dataY.data());
         fIsOutputConstant = true;
         return;
      }
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShapeY, fDynamic);
   }
   bool IsOutputConstant() const { return fIsOutputConstant; }
   // shape inference only (registers nothing): sets M, N, K, the bias mode and OutputShape()
   void ResolveShapes(RModel &model)
   {
      if (!model.CheckIfTensorAlreadyExist(fNA) || !model.CheckIfTensorAlreadyExist(fNB))
         throw std::runtime_error("SOFIE Gemm Op Input Tensor " + fNA + " or " + fNB + " is not found in model");
      if (!fNC.empty() && !model.CheckIfTensorAlreadyExist(fNC))
         throw std::runtime_error("SOFIE Gemm Op Input Tensor " + fNC + " is not found in model");
      if (model.GetTensorType(fNA) != ETensorType::FLOAT || model.GetTensorType(fNB) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Gemm Op: only float tensors; quantised products use ROperator_QGemm");
      fShapeA = model.GetTensorShape(fNA);
      fShapeB = model.GetTensorShape(fNB);
      // a run-time batch is the leading dimension of the operand (kept as 1 in its shape)
      const bool dynA = model.IsDynamicTensor(fNA), dynB = model.IsDynamicTensor(fNB);
      fDynamic = dynA || dynB;
      if (fDynamic && (fShapeA.size() < 2 || fShapeB.size() < 2 || (dynA && fShapeA.size() < fShapeB.size()) ||
                       (dynB && fShapeB.size() < fShapeA.size())))
         throw std::runtime_error("SOFIE Gemm Op: with a run-time batch the batched operand must have the full rank of the product");
      // MatMul conventions of the reference (ROperator_Gemm.hxx:183-215): a 1-D A gets a leading 1, a 1-D B a
      // trailing 1, and the shorter shape is padded with leading 1s
      bool prependOne = false, appendOne = false;
      if (fShapeA.size() == 1) {
         fShapeA.insert(fShapeA.begin(), 1);
         prependOne = true;
      }
      if (fShapeB.size() == 1) {
         fShapeB.push_back(1);
         appendOne = true;
      }
      if (fShapeA.size() < 2 || fShapeB.size() < 2)
         throw std::runtime_error("SOFIE Gemm Op Shape Inference only accept input tensor with >=2 dimensions");
      while (fShapeA.size() < fShapeB.size())
         fShapeA.insert(fShapeA.begin(), 1);
      while (fShapeB.size() < fShapeA.size())
         fShapeB.insert(fShapeB.begin(), 1);
      const std::size_t r = fShapeA.size();
      fM = fAttrTransA ? fShapeA[r - 1] : fShapeA[r - 2];
      fK = fAttrTransA ? fShapeA[r - 2] : fShapeA[r - 1];
      const std::size_t kB = fAttrTransB ? fShapeB[r - 1] : fShapeB[r - 2];
      fN = fAttrTransB ? fShapeB[r - 2] : fShapeB[r - 1];
      if (kB != fK)
         throw std::runtime_error("SOFIE Gemm Op: the inner dimensions of " + fNA + " " + ConvertShapeToString(fShapeA) + " and " + fNB +
                                  " " + ConvertShapeToString(fShapeB) + " do not agree");
      // stacked MatMul: leading dims broadcast (1 or equal)
      std::vector<std::size_t> shapeY;
      fBatch = 1;
      fStrideA = fStrideB = 0;
      std::size_t leadA = 1, leadB = 1;
      for (std::size_t i = 0; i + 2 < r; ++i) {
         const std::size_t a = fShapeA[i], b = fShapeB[i];
         if (a != b && a != 1 && b != 1)
            throw std::runtime_error("SOFIE Gemm(MatMul) has invalid shape for inputs or output");
         shapeY.push_back(std::max(a, b));
         fBatch *= std::max(a, b);
         leadA *= a;
         leadB *= b;
      }
      if (fBatch > 1) {
         if ((leadA != 1 && leadA != fBatch) || (leadB != 1 && leadB != fBatch))
            throw std::runtime_error("SOFIE Gemm(MatMul): mixed broadcasting of the stacked dimensions is not supported");
         fStrideA = leadA == 1 ? 0 : fM * fK;
         fStrideB = leadB == 1 ? 0 : fK * fN;
      }
      fDynamicRows = fDynamicStack = false;
      if (fDynamic && r == 2) {
         // Y[batch, N] = A[batch, K] * B: the rows of the product grow with the batch
         if (dynB || fAttrTransA)
            throw std::runtime_error("SOFIE Gemm Op: a run-time batch must be the row dimension of A");
         fDynamicRows = true;
      } else if (fDynamic) {
         // stacked product: the number of stacked matrices grows with the batch; an operand without the batch
         // must be one matrix shared by all
         if ((!dynA && leadA != 1) || (!dynB && leadB != 1))
            throw std::runtime_error("SOFIE Gemm(MatMul): with a run-time batch the other operand must be a single matrix");
         fDynamicStack = true;
         fStrideA = dynA ? fM * fK : 0;
         fStrideB = dynB ? fK * fN : 0;
      }
      shapeY.push_back(fM);
      shapeY.push_back(fN);

      // bias: the four broadcast cases of the reference (ROperator_Gemm.hxx:578-617) or a Y-shaped C
      fBiasMode = "SOFIE_BIAS_NONE";
      if (!fNC.empty()) {
         if (model.GetTensorType(fNC) != ETensorType::FLOAT)
            throw std::runtime_error("SOFIE Gemm Op: bias tensor " + fNC + " is not float");
         auto shapeC = model.GetTensorShape(fNC);
         std::vector<std::size_t> c2 = shapeC;
         while (c2.size() > 2 && c2.front() == 1)
            c2.erase(c2.begin());
         if (c2.size() == 1)
            c2.insert(c2.begin(), 1);
         if (c2.empty())
            c2 = {1, 1};
         // a C with exactly Y's shape goes to the kernel as C with the operator's beta; anything else is a
         // broadcast, for which the reference forces beta = 1 (ROperator_Gemm.hxx:580)
         // (with a run-time batch only a C that carries the batch itself can have Y's shape)
         if (shapeC == shapeY && (!fDynamic || model.IsDynamicTensor(fNC)))
            fBiasMode = "SOFIE_BIAS_FULL";
         else if (fDynamic && model.IsDynamicTensor(fNC))
            throw std::runtime_error("SOFIE Gemm Op - a batched bias tensor must have the shape of the product");
         else if (c2.size() == 2 && c2[0] == 1 && c2[1] == fN)
            fBiasMode = "SOFIE_BIAS_ROW";
         else if (c2.size() == 2 && c2[1] == 1 && c2[0] == fM && !fDynamicRows)
            fBiasMode = "SOFIE_BIAS_COL";
         else if (c2.size() == 2 && c2[0] == 1 && c2[1] == 1)
            fBiasMode = "SOFIE_BIAS_SCALAR";
         else
            throw std::runtime_error("SOFIE Gemm Op - bias tensor of shape " + ConvertShapeToString(shapeC) +
                                     " cannot be uni-directional broadcasted to " + ConvertShapeToString(shapeY));
         if (fBiasMode == std::string("SOFIE_BIAS_FULL") && (fBatch > 1 || fDynamicStack))
            fStrideC = fM * fN;
      } else if (fAttrBeta != 0) {
         fAttrBeta = 0; // no bias: beta is forced to zero as in the reference (ROperator_Gemm.hxx:491-499)
      }
      if (prependOne)
         shapeY.erase(shapeY.end() - 2);
      if (appendOne)
         shapeY.pop_back();
      fShapeY = shapeY;
   }

   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      if (fM == 0)
         throw std::runtime_error("SOFIE Gemm Op called to Generate without being initialized first");
      if (fIsOutputConstant)
         return "\n" + SP + "//--------- Gemm " + opName + " -> " + fNY + ": a product of weights, computed when the code was generated\n";
      std::stringstream out;
      out << "\n" << SP << "//--------- Gemm " << opName << " " << Title() << "\n";
      out << SP << "{\n";
      out << SP << "   " << "sofie_gemm_f32_desc d{};\n";
      out << DescriptorStatements("d", "post");
      out << SP << "   " << "detail::Check(sofie_hip_gemm_f32(fCtx, &d), \"" << opName << " Gemm\");\n";
      out << SP << "}\n";
      return out.str();
   }
   std::string Title() const { return ConvertShapeToString(fShapeA) + " * " + ConvertShapeToString(fShapeB) + " -> " + fNY; }
   // the statements that fill the sofie_gemm_f32_desc named `d` (a post-operator block, if any, is declared as `post`)
   std::string DescriptorStatements(const std::string &d, const std::string &post) const
   {
      std::stringstream out;
      out << SP << "   " << d << ".M = " << BatchScaledInt(fDynamicRows, fM) << "; " << d << ".N = " << fN << "; " << d << ".K = " << fK << "; " << d
          << ".transA = " << (fAttrTransA ? 1 : 0) << "; " << d << ".transB = " << (fAttrTransB ? 1 : 0) << ";\n";
      out << SP << "   " << d << ".alpha = " << FloatLiteral(fAttrAlpha) << "; " << d << ".beta = " << FloatLiteral(fAttrBeta) << ";\n";
      out << SP << "   " << d << ".A = tensor_" << fNA << "; " << d << ".B = tensor_" << fNB << "; " << d << ".C = " << (fNC.empty() ? "nullptr" : "tensor_" + fNC)
          << "; " << d << ".bias_mode = " << fBiasMode << ";\n";
      out << SP << "   " << d << ".act = " << ActivationEnumName(fActivation) << "; " << d << ".act_alpha = " << FloatLiteral(fActAlpha) << ";\n";
      out << SP << "   " << d << ".Y = tensor_" << fNY << "; " << d << ".batch = " << BatchScaledInt(fDynamicStack, fBatch) << "; " << d << ".strideA = " << fStrideA
          << "; " << d << ".strideB = " << fStrideB << "; " << d << ".strideC = " << fStrideC << "; " << d << ".strideY = "
          << (fBatch > 1 || fDynamicStack ? fM * fN : 0) << ";\n";
      if (!fPost.empty())
         out << SP << "   " << PostOpsDeclaration(post, fPost) << " " << d << ".post = &" << post << ";\n";
      if (!fNR.empty())
         out << SP << "   " << d << ".residual = tensor_" << fNR << ";\n";
      // An operand read through strides {s0, s1}: element (i, j) of the stored matrix is at i * s0 + j * s1.  Row-major with
      // s1 == 1: row stride s0.  Column-major with s0 == 1: row stride s1 and the transpose flag flipped.  Without a unit
      // stride the matrix cannot be described (ROperator_Gemm.hxx:644-668 and 898-927 of the reference).
      auto resolve = [&](const char *tag, const std::string &name, const std::vector<std::size_t> &stored, bool batchedRows) {
         const std::string member = "this->" + InputStrideMemberName(name);
         const std::string rows = batchedRows ? "static_cast<std::size_t>(sofie_batch)" : "static_cast<std::size_t>(" + std::to_string(stored[0]) + ")";
         const std::string cols = "static_cast<std::size_t>(" + std::to_string(stored[1]) + ")";
         out << SP << "   " << "if (!" << member << ".empty()) {\n";
         out << SP << "      " << "if (" << member << "[1] == 1) {\n";
         out << SP << "         " << d << ".ld" << (tag[0] == 'A' ? "a" : "b") << " = static_cast<std::int32_t>(std::max<std::size_t>(" << member << "[0], " << cols << "));\n";
         out << SP << "      " << "} else if (" << member << "[0] == 1) {\n";
         out << SP << "         " << d << ".trans" << tag << " = !" << d << ".trans" << tag << ";\n";
         out << SP << "         " << d << ".ld" << (tag[0] == 'A' ? "a" : "b") << " = static_cast<std::int32_t>(std::max<std::size_t>(" << member << "[1], " << rows << "));\n";
         out << SP << "      " << "} else {\n";
         out << SP << "         " << "throw std::runtime_error(\"SOFIE Gemm Op - input tensor " << name << " has strides {\" + std::to_string(" << member
             << "[0]) + \", \" + std::to_string(" << member << "[1]) + \"} without a unit stride, which BLAS cannot handle\");\n";
         out << SP << "      " << "}\n";
         out << SP << "   " << "}\n";
      };
      if (fStridedA)
         resolve("A", fNA, fStoredA, fDynamicRows);
      if (fStridedB)
         resolve("B", fNB, fStoredB, false);
      return out.str();
   }
   // Can this product stand in a chain handed to sofie_hip_gemm_chain_f32 (it exists at run time and is a plain 2-D product)?
   // (an operand read through strides may turn out transposed at run time: such a product stays on its own)
   bool IsChainLink() const { return fM != 0 && !fIsOutputConstant && fBatch == 1 && !fDynamicStack && !fAttrTransA && !fStridedA && !fStridedB; }
   const std::string &NameA() const { return fNA; }
   const std::string &NameY() const { return fNY; }

private:
   float fAttrAlpha = 1.0, fAttrBeta = 1.0;
   int64_t fAttrTransA = 0, fAttrTransB = 0;
   std::string fNA, fNB, fNC, fNY, fNR;
   std::vector<std::size_t> fShapeY;
   EActivationType fActivation = EActivationType::UNDEFINED;
   float fActAlpha = 0.01f;
   std::vector<PostOp> fPost;
   std::vector<std::size_t> fShapeA, fShapeB;
   std::size_t fM = 0, fN = 0, fK = 0, fBatch = 1, fStrideA = 0, fStrideB = 0, fStrideC = 0;
   std::string fBiasMode;
   bool fDynamic = false, fDynamicRows = false, fDynamicStack = false, fIsOutputConstant = false;
   bool fStridedA = false, fStridedB = false; // graph inputs read through the strides given to the Session
   std::vector<std::size_t> fStoredA, fStoredB; // the operands' shapes as stored
};

} // namespace SOFIE_HIP
#endif
