// Conv emitter for the gfx950 backend: the operator of core/inc/SOFIE/operators/ROperator_Conv.hxx (same
// constructor arguments, same padding / stride / dilation / autopad rules), emitting ONE implicit-GEMM
// launch over the whole batch (sofie_hip_conv_f32) instead of a per-image Im2col + Gemm_Call loop and a
// per-call weight re-layout.  1-D convolutions run as 2-D with H = 1; 3-D convolutions (the reference's Im2col_3d path) go to
// sofie_hip_conv3d_f32, the same implicit GEMM with the reduction over (channel, kd, kh, kw).
#ifndef SOFIE_HIP_ROPERATOR_CONV
#define SOFIE_HIP_ROPERATOR_CONV

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

struct ConvGeometry {
   std::size_t N = 0, C = 0, H = 1, W = 0, Cout = 0, kh = 1, kw = 1, OH = 1, OW = 0, group = 1;
   // three spatial dimensions: depth first; the pads in the attribute's order {d0, h0, w0, d1, h1, w1}
   std::size_t D = 1, kd = 1, OD = 1;
   std::vector<std::size_t> pads3, strides3, dils3;
   std::size_t pad_h0 = 0, pad_w0 = 0, pad_h1 = 0, pad_w1 = 0, stride_h = 1, stride_w = 1, dil_h = 1, dil_w = 1;
   std::size_t dim = 2;

   // ROperator_Conv::DoShapeInference (ROperator_Conv.hxx:123-262): default dilations/strides of 1; with auto_pad
   // NOTSET and no pads attribute the pads are 1 (:172-175); SAME_UPPER / SAME_LOWER split the total padding
   // (:176-197); the effective kernel is k + (d-1)(k-1); output = (in + pads - kernel) / stride + 1.
   void Resolve(const std::string &autopad, std::vector<std::size_t> dilations, std::size_t grp, std::vector<std::size_t> kernelShape,
                std::vector<std::size_t> pads, std::vector<std::size_t> strides, const std::vector<std::size_t> &shapeX,
                const std::vector<std::size_t> &shapeW)
   {
      if (shapeX.size() < 3 || shapeX.size() > 5)
         throw std::runtime_error("SOFIE Conv Op: the input must have 3, 4 or 5 dimensions (1-D, 2-D or 3-D convolution)");
      dim = shapeX.size() - 2;
      if (shapeW.size() != shapeX.size())
         throw std::runtime_error("SOFIE Conv Op Shape inference - invalid weights ");
      if (grp == 0)
         grp = shapeX[1] / shapeW[1];
      group = grp;
      if (kernelShape.empty())
         kernelShape.assign(shapeW.begin() + 2, shapeW.end());
      if (dilations.empty())
         dilations.assign(dim, 1);
      if (strides.empty())
         strides.assign(dim, 1);
      std::vector<std::size_t> ek(dim);
      for (std::size_t d = 0; d < dim; ++d)
         ek[d] = kernelShape[d] + (dilations[d] - 1) * (kernelShape[d] - 1);
      if (autopad == "NOTSET") {
         if (pads.empty())
            pads.assign(2 * dim, 1);
      } else if (autopad == "SAME_UPPER" || autopad == "SAME_LOWER") {
         pads.assign(2 * dim, 0);
         for (std::size_t d = 0; d < dim; ++d) {
            const std::size_t in = shapeX[d + 2], out = (in + strides[d] - 1) / strides[d];
            const int total = std::max(0, (int)((out - 1) * strides[d] + ek[d]) - (int)in);
            if (autopad == "SAME_UPPER") {
               pads[d] = total / 2;
               pads[d + dim] = total - total / 2;
            } else {
               pads[d] = total - total / 2;
               pads[d + dim] = total / 2;
            }
         }
      } else if (autopad == "VALID") {
         pads.assign(2 * dim, 0);
      } else {
         throw std::runtime_error("SOFIE Conv Op invalid fAutopad");
      }
      if (pads.size() != 2 * dim || kernelShape.size() != dim || strides.size() != dim || dilations.size() != dim)
         throw std::runtime_error("SOFIE Conv Op: attribute lengths do not match the number of spatial dimensions");
      N = shapeX[0];
      C = shapeX[1];
      Cout = shapeW[0];
      if (C % group != 0 || Cout % group != 0 || shapeW[1] != C / group)
         throw std::runtime_error("SOFIE Conv Op: channels, groups and weight shape do not agree");
      if (dim == 3) {
         D = shapeX[2]; H = shapeX[3]; W = shapeX[4]; kd = kernelShape[0]; kh = kernelShape[1]; kw = kernelShape[2];
         pads3 = pads; strides3 = strides; dils3 = dilations;
         std::size_t out[3];
         for (std::size_t d = 0; d < 3; ++d) {
            if (shapeX[2 + d] + pads[d] + pads[d + 3] < ek[d])
               throw std::runtime_error("SOFIE Conv Op: kernel larger than the padded input");
            out[d] = (shapeX[2 + d] + pads[d] + pads[d + 3] - ek[d]) / strides[d] + 1;
         }
         OD = out[0]; OH = out[1]; OW = out[2];
         return;
      }
      if (dim == 1) {
         H = 1; W = shapeX[2]; kh = 1; kw = kernelShape[0];
         pad_h0 = pad_h1 = 0; pad_w0 = pads[0]; pad_w1 = pads[1];
         stride_h = 1; stride_w = strides[0]; dil_h = 1; dil_w = dilations[0];
      } else {
         H = shapeX[2]; W = shapeX[3]; kh = kernelShape[0]; kw = kernelShape[1];
         pad_h0 = pads[0]; pad_w0 = pads[1]; pad_h1 = pads[2]; pad_w1 = pads[3];
         stride_h = strides[0]; stride_w = strides[1]; dil_h = dilations[0]; dil_w = dilations[1];
      }
      const std::size_t ekh = kh + (dil_h - 1) * (kh - 1), ekw = kw + (dil_w - 1) * (kw - 1);
      if (H + pad_h0 + pad_h1 < ekh || W + pad_w0 + pad_w1 < ekw)
         throw std::runtime_error("SOFIE Conv Op: kernel larger than the padded input");
      OH = (H + pad_h0 + pad_h1 - ekh) / stride_h + 1;
      OW = (W + pad_w0 + pad_w1 - ekw) / stride_w + 1;
   }
   std::vector<std::size_t> OutputShape() const
   {
      if (dim == 1)
         return {N, Cout, OW};
      if (dim == 3)
         return {N, Cout, OD, OH, OW};
      return {N, Cout, OH, OW};
   }
   // statement that scales the descriptor's image count by the run-time batch
   std::string BatchLine(bool dynamic, const std::string &indent) const
   {
      return dynamic ? indent + "d.N = static_cast<std::int32_t>(sofie_batch * " + std::to_string(N) + ");\n" : std::string();
   }
   std::string DescInitializer() const
   {
      std::stringstream s;
      if (dim == 3) {
         s << "{" << N << ", " << C << ", " << D << ", " << H << ", " << W << ", " << Cout << ", " << kd << ", " << kh << ", " << kw << ", {"
           << pads3[0] << ", " << pads3[1] << ", " << pads3[2] << ", " << pads3[3] << ", " << pads3[4] << ", " << pads3[5] << "}, {" << strides3[0]
           << ", " << strides3[1] << ", " << strides3[2] << "}, {" << dils3[0] << ", " << dils3[1] << ", " << dils3[2] << "}, " << group << ", " << OD
           << ", " << OH << ", " << OW << "}";
         return s.str();
      }
      s << "{" << N << ", " << C << ", " << H << ", " << W << ", " << Cout << ", " << kh << ", " << kw << ", " << pad_h0 << ", " << pad_w0 << ", "
        << pad_h1 << ", " << pad_w1 << ", " << stride_h << ", " << stride_w << ", " << dil_h << ", " << dil_w << ", " << group << ", " << OH
        << ", " << OW << "}";
      return s.str();
   }
};

template <typename T>
class ROperator_Conv final : public ROperator {
   static_assert(std::is_same<T, float>::value, "SOFIE Encountered unsupported type parsing a Conv operator");

public:
   ROperator_Conv(std::string autopad, std::vector<std::size_t> dilations, std::size_t group, std::vector<std::size_t> kernelShape,
                  std::vector<std::size_t> pads, std::vector<std::size_t> strides, std::string nameX, std::string nameW, std::string nameB,
                  std::string nameY)
      : fAttrAutopad(autopad), fAttrDilations(dilations), fAttrGroup(group), fAttrKernelShape(kernelShape), fAttrPads(pads),
        fAttrStrides(strides), fNX(UTILITY::Clean_name(nameX)), fNW(UTILITY::Clean_name(nameW)), fNB(UTILITY::Clean_name(nameB)),
        fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX, fNW};
      if (!fNB.empty())
         fInputTensorNames.push_back(fNB);
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::CONV;
   }
   ROperator_Conv(std::string autopad, std::vector<std::size_t> dilations, std::size_t group, std::vector<std::size_t> kernelShape,
                  std::vector<std::size_t> pads, std::vector<std::size_t> strides, std::string nameX, std::string nameW, std::string nameY)
      : ROperator_Conv(autopad, dilations, group, kernelShape, pads, strides, nameX, nameW, "", nameY)
   {
   }
   bool HasActivation() const { return fActivation != EActivationType::UNDEFINED; }
   void FuseActivation(EActivationType a, float alpha, const std::string &newOutput)
   {
      fActivation = a;
      fActAlpha = alpha;
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   std::size_t PostOpCount() const { return fPost.size(); }
   void AddPostOp(const PostOp &op, const std::string &newOutput)
   {
      fPost.push_back(op);
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   // see ROperator_Gemm::SetResidual
   bool HasResidual() const { return !fNR.empty(); }
   void SetResidual(const std::string &name, const std::string &newOutput)
   {
      fNR = UTILITY::Clean_name(name);
      fInputTensorNames.push_back(fNR);
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   std::vector<std::size_t> OutputShape() const { return fGeo.OutputShape(); }
   bool IsBatched() const { return fDynamic; }

   void Initialize(RModel &model) override
   {
      ResolveShapes(model);
      if (!fNR.empty() && (!model.CheckIfTensorAlreadyExist(fNR) || model.GetTensorType(fNR) != ETensorType::FLOAT ||
                           model.GetTensorShape(fNR) != fGeo.OutputShape() || model.IsDynamicTensor(fNR) != fDynamic))
         throw std::runtime_error("SOFIE Conv Op: residual tensor " + fNR + " does not have the shape of the output");
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fGeo.OutputShape(), fDynamic);
   }
   void ResolveShapes(RModel &model)
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE Conv op Input Tensor " + fNX + " is not found in model");
      if (!model.CheckIfTensorAlreadyExist(fNW))
         throw std::runtime_error("SOFIE Conv op Input weight Tensor " + fNW + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Conv Op: only float tensors; quantised convolutions use ROperator_QConv");
      fGeo.Resolve(fAttrAutopad, fAttrDilations, fAttrGroup, fAttrKernelShape, fAttrPads, fAttrStrides, model.GetTensorShape(fNX),
                   model.GetTensorShape(fNW));
      if (!fNB.empty()) {
         if (!model.CheckIfTensorAlreadyExist(fNB))
            throw std::runtime_error("SOFIE Conv op Input Tensor " + fNB + " is not found in model");
         auto shapeB = model.GetTensorShape(fNB);
         if (shapeB.size() != 1 || shapeB[0] != fGeo.Cout)
            throw std::runtime_error("SOFIE Conv op " + fNY + " : invalid shape for Bias tensor " + fNB + " : " + ConvertShapeToString(shapeB));
      }
      fDynamic = model.IsDynamicTensor(fNX);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      if (fGeo.Cout == 0)
         throw std::runtime_error("SOFIE Conv Op called to Generate without being initialized first");
      std::stringstream out;
      out << "\n" << SP << "//----  operator Conv " << opName << " --> " << ConvertShapeToString(fGeo.OutputShape()) << "\n";
      out << SP << "{\n";
      const bool threeD = fGeo.dim == 3;
      out << SP << "   " << (threeD ? "sofie_conv3d_desc d" : "sofie_conv_desc d") << fGeo.DescInitializer() << ";\n" << fGeo.BatchLine(fDynamic, SP + "   ");
      if (!fPost.empty())
         out << SP << "   " << PostOpsDeclaration("post", fPost) << "\n";
      out << SP << "   " << "detail::Check(" << (threeD ? "sofie_hip_conv3d_f32" : "sofie_hip_conv_f32") << "(fCtx, &d, tensor_" << fNX << ", tensor_" << fNW << ", "
          << (fNB.empty() ? "nullptr" : "tensor_" + fNB) << ", " << ActivationEnumName(fActivation) << ", " << FloatLiteral(fActAlpha)
          << ", tensor_" << fNY << ", " << (fPost.empty() ? "nullptr" : "&post") << ", " << (fNR.empty() ? "nullptr" : "tensor_" + fNR) << "), \""
          << opName << " Conv\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   std::string fAttrAutopad;
   std::vector<std::size_t> fAttrDilations;
   std::size_t fAttrGroup;
   std::vector<std::size_t> fAttrKernelShape, fAttrPads, fAttrStrides;
   std::string fNX, fNW, fNB, fNY, fNR;
   EActivationType fActivation = EActivationType::UNDEFINED;
   float fActAlpha = 0.01f;
   std::vector<PostOp> fPost;
   ConvGeometry fGeo;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
