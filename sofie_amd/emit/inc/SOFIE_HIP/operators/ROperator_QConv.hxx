// Quantised convolution chain of the gfx950 backend.  The reference has no quantised operator
// (parsers/src/RModelParser_ONNX.cxx:279-367); these follow its operator contract
// (core/inc/SOFIE/operators/ROperator.hxx:111-147), the geometry rules of its Conv
// (core/inc/SOFIE/operators/ROperator_Conv.hxx:123-262) and the ONNX definitions:
//   QLinearConv  acc = conv_i32(x_i8, w_i8) + B_i32[co];  y_i8 = sat8(rne(float(acc) * m[co])),
//                m[co] = (x_scale * w_scale[co]) / y_scale formed once in fp32 by the generator; zero points 0.
//                A Relu that follows is folded into the store.  Between two quantised convolutions the
//                activation is kept NHWC (channels fastest), which is what the matrix-core kernel reads in place.
//   DequantizeLinear + GlobalAveragePool on an int8 map  ->  one kernel: exact int32 sum, then * scale / HW.
//                When that map comes from a QLinearConv which nothing else reads, and the runtime can do it (planes of a
//                multiple of 256 pixels, no column matrix), the convolution adds the planes up in its own store: the map
//                is neither written nor read back, and a small kernel turns the sums into the average.
#ifndef SOFIE_HIP_ROPERATOR_QCONV
#define SOFIE_HIP_ROPERATOR_QCONV

#include "SOFIE_HIP/operators/ROperator_Conv.hxx"

#include <cmath>

namespace SOFIE_HIP {

class ROperator_QConv final : public ROperator {
public:
   // the nine inputs of ONNX QLinearConv (nameB may be empty)
   ROperator_QConv(std::string autopad, std::vector<std::size_t> dilations, std::size_t group, std::vector<std::size_t> kernelShape,
                   std::vector<std::size_t> pads, std::vector<std::size_t> strides, std::string nameX, std::string nameXScale,
                   std::string nameXZero, std::string nameW, std::string nameWScale, std::string nameWZero, std::string nameYScale,
                   std::string nameYZero, std::string nameB, std::string nameY)
      : fAttrAutopad(autopad), fAttrDilations(dilations), fAttrGroup(group), fAttrKernelShape(kernelShape), fAttrPads(pads),
        fAttrStrides(strides), fNX(UTILITY::Clean_name(nameX)), fNXS(UTILITY::Clean_name(nameXScale)), fNXZ(UTILITY::Clean_name(nameXZero)),
        fNW(UTILITY::Clean_name(nameW)), fNWS(UTILITY::Clean_name(nameWScale)), fNWZ(UTILITY::Clean_name(nameWZero)),
        fNYS(UTILITY::Clean_name(nameYScale)), fNYZ(UTILITY::Clean_name(nameYZero)), fNB(UTILITY::Clean_name(nameB)),
        fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX, fNW};
      if (!fNB.empty())
         fInputTensorNames.push_back(fNB);
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::QCONV;
   }
   // ONNX ConvInteger: the plain int32 accumulator is the output (no scales, no bias), NCHW
   static std::unique_ptr<ROperator_QConv> MakeConvInteger(std::string autopad, std::vector<std::size_t> dilations, std::size_t group,
                                                            std::vector<std::size_t> kernelShape, std::vector<std::size_t> pads,
                                                            std::vector<std::size_t> strides, std::string nameX, std::string nameW,
                                                            std::string nameXZero, std::string nameWZero, std::string nameY)
   {
      auto op = std::make_unique<ROperator_QConv>(autopad, dilations, group, kernelShape, pads, strides, nameX, "", nameXZero, nameW, "", nameWZero,
                                                  "", "", "", nameY);
      op->fInt32Out = true;
      return op;
   }
   bool HasRelu() const { return fRelu; }
   void FuseRelu(const std::string &newOutput)
   {
      fRelu = true;
      fNY = newOutput;
      fOutputTensorNames = {fNY};
   }
   const std::string &OutputName() const { return fNY; }

   // Whether the runtime would add the output planes up in the kernel's store (sofie_hip_conv_i8 with
   // SOFIE_I8OUT_I8_PLANE_SUMS): callable before Initialize, once the input's shape and layout are known.
   bool CanSumPlanes(RModel &model)
   {
      if (fInt32Out || !model.CheckIfTensorAlreadyExist(fNX) || !model.CheckIfTensorAlreadyExist(fNW))
         return false;
      try {
         fGeo.Resolve(fAttrAutopad, fAttrDilations, fAttrGroup, fAttrKernelShape, fAttrPads, fAttrStrides, model.GetTensorShape(fNX),
                      model.GetTensorShape(fNW));
      if (fGeo.dim == 3)
         throw std::runtime_error("SOFIE quantised Conv Op: 3-D convolutions are emitted for float tensors only");
      } catch (const std::exception &) {
         return false; // Initialize reports the problem
      }
      fXLayout = model.GetTensorLayout(fNX);
      return (fGeo.OH * fGeo.OW) % 256 == 0 && (ImplicitGemm() || GatheredGemm());
   }
   // The GlobalAveragePool(DequantizeLinear(Y, scale)) that was the only reader of Y becomes this operator's output.
   void SumPlanes(float dequantScale, const std::string &pooledOutput)
   {
      fSumPlanes = true;
      fPoolScale = dequantScale;
      fNPooled = pooledOutput;
      fOutputTensorNames = {fNPooled};
   }
   bool SumsPlanes() const { return fSumPlanes; }

   void Initialize(RModel &model) override
   {
      for (auto *n : {&fNX, &fNW})
         if (!model.CheckIfTensorAlreadyExist(*n))
            throw std::runtime_error("SOFIE QLinearConv Op Input Tensor " + *n + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::INT8)
         throw std::runtime_error("SOFIE QLinearConv Op: input tensor " + fNX + " is not int8");
      if (!model.IsInitializedTensor(fNW) || model.GetTensorType(fNW) != ETensorType::INT8)
         throw std::runtime_error("SOFIE QLinearConv Op: weight tensor " + fNW + " must be an int8 initializer");
      for (auto *z : {&fNXZ, &fNWZ, &fNYZ}) {
         if (z->empty())
            continue;
         if (!model.IsInitializedTensor(*z) || model.GetTensorType(*z) != ETensorType::INT8)
            throw std::runtime_error("SOFIE QLinearConv Op: zero point " + *z + " must be an int8 initializer");
         const auto *p = static_cast<const int8_t *>(model.GetInitializedTensorData(*z).get());
         for (std::size_t i = 0; i < ConvertShapeToLength(model.GetTensorShape(*z)); ++i)
            if (p[i] != 0)
               throw std::runtime_error("SOFIE QLinearConv Op: zero point " + *z + " is not 0; this backend emits symmetric quantisation only");
      }
      fGeo.Resolve(fAttrAutopad, fAttrDilations, fAttrGroup, fAttrKernelShape, fAttrPads, fAttrStrides, model.GetTensorShape(fNX),
                   model.GetTensorShape(fNW));
      fXLayout = model.GetTensorLayout(fNX);
      fDynamic = model.IsDynamicTensor(fNX);
      if (fInt32Out) {
         fYLayout = kLayoutNCHW;
         model.AddIntermediateTensor(fNY, ETensorType::INT32, fGeo.OutputShape(), fDynamic);
         return;
      }
      const float xs = model.GetScalarInitializer(fNXS), ys = model.GetScalarInitializer(fNYS);
      if (!(xs > 0) || !(ys > 0))
         throw std::runtime_error("SOFIE QLinearConv Op: scales of " + fNX + " and " + fNY + " must be positive");
      if (!model.IsInitializedTensor(fNWS) || model.GetTensorType(fNWS) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE QLinearConv Op: weight scale " + fNWS + " must be a float initializer");
      const std::size_t nws = ConvertShapeToLength(model.GetTensorShape(fNWS));
      if (nws != 1 && nws != fGeo.Cout)
         throw std::runtime_error("SOFIE QLinearConv Op: weight scale " + fNWS + " must have 1 or " + std::to_string(fGeo.Cout) + " elements");
      const float *ws = static_cast<const float *>(model.GetInitializedTensorData(fNWS).get());
      std::vector<float> m(fGeo.Cout);
      for (std::size_t co = 0; co < fGeo.Cout; ++co) {
         volatile float prod = xs * ws[nws == 1 ? 0 : co]; // two fp32 roundings, in this order
         m[co] = prod / ys;
      }
      fNM = fNY + "_requant_scale";
      model.AddInitializedTensor(fNM, ETensorType::FLOAT, {fGeo.Cout}, m.data());
      if (!fNB.empty()) {
         if (!model.IsInitializedTensor(fNB) || model.GetTensorType(fNB) != ETensorType::INT32 ||
             ConvertShapeToLength(model.GetTensorShape(fNB)) != fGeo.Cout)
            throw std::runtime_error("SOFIE QLinearConv Op: bias " + fNB + " must be an int32 initializer of " + std::to_string(fGeo.Cout) + " elements");
      }
      if (fSumPlanes) {
         if (!((fGeo.OH * fGeo.OW) % 256 == 0 && (ImplicitGemm() || GatheredGemm())))
            throw std::runtime_error("SOFIE QLinearConv Op: " + fNY + " cannot be summed plane by plane in the convolution");
         model.AddIntermediateTensor(fNPooled, ETensorType::FLOAT, {fGeo.N, fGeo.Cout, 1, 1}, fDynamic);
         return;
      }
      // channels-last output when every reader understands it
      fYLayout = kLayoutNHWC;
      if (model.IsOutputTensor(fNY))
         fYLayout = kLayoutNCHW;
      for (OperatorKind k : model.ConsumerKinds(fNY))
         if (k != OperatorKind::QCONV && k != OperatorKind::QPOOL)
            fYLayout = kLayoutNCHW;
      model.AddIntermediateTensor(fNY, ETensorType::INT8, fGeo.OutputShape(), fDynamic);
      model.SetTensorLayout(fNY, fYLayout);
   }
   std::size_t PackedK() const { return ((fGeo.C / fGeo.group) * fGeo.kh * fGeo.kw + 15) / 16 * 16; }
   // The int32 plane sums [N][Cout] of a convolution that feeds a GlobalAveragePool.  With a fixed batch they have a buffer of
   // their own, cleared once at construction: the averaging call clears them again behind its read, so no inference starts
   // with a clearing launch.  With a run-time batch (N is 1 here and the bytes are per batch entry) they are a workspace,
   // cleared by every inference.
   bool KeepsPlaneSums() const { return fSumPlanes && !fDynamic; }
   std::size_t PlaneSumBytes() const { return (fGeo.N * fGeo.Cout * 4 + 255) / 256 * 256; }
   std::vector<std::pair<std::string, std::size_t>> GetPersistentBuffers() override
   {
      std::vector<std::pair<std::string, std::size_t>> b = {{"packed_" + fNW, (fGeo.Cout * PackedK() + 255) / 256 * 256}};
      if (KeepsPlaneSums())
         b.emplace_back("planesums_" + fNY, PlaneSumBytes());
      return b;
   }
   std::string GenerateInitCode_GPU_HIP() override
   {
      std::stringstream out;
      out << SP << "   " << "{\n";
      out << SP << "      " << "sofie_conv_desc d" << fGeo.DescInitializer() << ";\n";
      out << SP << "      " << "detail::Check(sofie_hip_pack_conv_weight_i8(fCtx, &d, packed_" << fNW << ", tensor_" << fNW << "), \"re-layout of "
          << fNW << "\");\n";
      if (KeepsPlaneSums())
         out << SP << "      " << "detail::Check(sofie_hip_fill_zero(fCtx, planesums_" << fNY << ", " << PlaneSumBytes() << "), \"clearing of the plane sums of "
             << fNY << "\");\n";
      out << SP << "   " << "}\n";
      return out.str();
   }
   // the runtime's rule for reading the activations in place (no column matrix): NHWC, channels per group a power
   // of two >= 64, at most 32 taps, 32-bit offsets
   bool ImplicitGemm() const
   {
      const std::size_t cg = fGeo.C / fGeo.group, taps = fGeo.kh * fGeo.kw;
      const double xbytes = (double)fGeo.N * fGeo.H * fGeo.W * fGeo.C;
      return fXLayout == kLayoutNHWC && (cg & (cg - 1)) == 0 && cg >= 64 && taps <= 32 && fGeo.C % 16 == 0 && xbytes < 2.0e9 &&
             (double)fGeo.N * fGeo.OH * fGeo.OW < 2.0e9 && taps <= 32;
   }
   // the runtime's rule for gathering the rows inside the kernel: the whole reduction fits one 64-byte slab
   bool GatheredGemm() const
   {
      return (fGeo.C / fGeo.group) * fGeo.kh * fGeo.kw <= 64 && (fGeo.kh - 1) * fGeo.dil_h <= 127 && (fGeo.kw - 1) * fGeo.dil_w <= 127 &&
             (double)fGeo.C * fGeo.H * fGeo.W < 2.0e9 && (double)fGeo.N * fGeo.OH * fGeo.OW < 2.0e9;
   }
   std::size_t GetWorkspaceBytes() override
   {
      if (fSumPlanes)
         return KeepsPlaneSums() ? 0 : PlaneSumBytes();
      if (ImplicitGemm() || GatheredGemm())
         return 0;
      const std::size_t per_image = (fGeo.OH * fGeo.OW * PackedK() + 255) / 256 * 256;
      std::size_t images = std::max<std::size_t>(1, (std::size_t(64) << 20) / per_image);
      return per_image * std::min(images, fGeo.N); // with a run-time batch N is 1: the column matrix of one image per batch entry
   }
   bool WorkspacePerBatchEntry() const override { return fDynamic; }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      const std::string ws = KeepsPlaneSums() ? "planesums_" + fNY : "workspace_op_" + opName;
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//----  operator " << (fInt32Out ? "ConvInteger " : "QLinearConv ") << opName << " --> " << ConvertShapeToString(fGeo.OutputShape())
          << (fSumPlanes ? " (not stored: planes summed for the GlobalAveragePool)" : fYLayout == kLayoutNHWC ? " (stored NHWC)" : "")
          << (ImplicitGemm() ? ", implicit GEMM" : GatheredGemm() ? ", rows gathered in the kernel" : ", column matrix") << "\n";
      out << SP << "{\n";
      out << SP << "   " << "sofie_conv_desc d" << fGeo.DescInitializer() << ";\n" << fGeo.BatchLine(fDynamic, SP + "   ");
      out << SP << "   " << "sofie_conv_i8_args a{};\n";
      out << SP << "   " << "a.X = tensor_" << fNX << "; a.W = packed_" << fNW << "; a.w_is_packed = 1; a.bias = "
          << (fNB.empty() ? "nullptr" : "tensor_" + fNB) << "; a.scale = " << (fInt32Out ? std::string("nullptr") : "tensor_" + fNM) << ";\n";
      out << SP << "   " << "a.relu = " << (fRelu ? 1 : 0) << "; a.out = " << (fSumPlanes ? "SOFIE_I8OUT_I8_PLANE_SUMS" : fInt32Out ? "SOFIE_I8OUT_I32" : "SOFIE_I8OUT_I8")
          << "; a.x_layout = " << (fXLayout == kLayoutNHWC ? "SOFIE_LAYOUT_NHWC" : "SOFIE_LAYOUT_NCHW") << "; a.y_layout = "
          << (fYLayout == kLayoutNHWC ? "SOFIE_LAYOUT_NHWC" : "SOFIE_LAYOUT_NCHW") << "; a.Y = " << (fSumPlanes ? ws : "tensor_" + fNY) << ";\n";
      if (fSumPlanes) {
         // rows of Cout int32 sums, one per image; zero before, filled by the convolution's store, then averaged
         const std::string count = BatchScaledInt(fDynamic, fGeo.N * fGeo.Cout);
         if (!KeepsPlaneSums())
            out << SP << "   " << "detail::Check(sofie_hip_fill_zero(fCtx, " << ws << ", static_cast<std::size_t>(" << count << ") * 4), \"" << opName
                << " clear plane sums\");\n";
         out << SP << "   " << "detail::Check(sofie_hip_conv_i8(fCtx, &d, &a), \"" << opName << " QLinearConv\");\n";
         if (KeepsPlaneSums())
            out << SP << "   " << "detail::Check(sofie_hip_plane_sums_take_average(fCtx, tensor_" << fNPooled << ", static_cast<int32_t *>(static_cast<void *>(" << ws
                << ")), " << count << ", " << fGeo.OH * fGeo.OW << ", " << FloatLiteral(fPoolScale) << "), \"" << opName << " GlobalAveragePool\");\n";
         else
            out << SP << "   " << "detail::Check(sofie_hip_plane_sums_to_average(fCtx, tensor_" << fNPooled << ", static_cast<const int32_t *>(static_cast<const void *>(" << ws
                << ")), " << count << ", " << fGeo.OH * fGeo.OW << ", " << FloatLiteral(fPoolScale) << "), \"" << opName << " GlobalAveragePool\");\n";
         out << SP << "}\n";
         return out.str();
      }
      if (GetWorkspaceBytes())
         out << SP << "   " << "a.workspace = " << ws << "; a.workspace_bytes = " << BatchScaled(fDynamic, GetWorkspaceBytes()) << ";\n";
      out << SP << "   " << "detail::Check(sofie_hip_conv_i8(fCtx, &d, &a), \"" << opName << " QLinearConv\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   std::string fAttrAutopad;
   std::vector<std::size_t> fAttrDilations;
   std::size_t fAttrGroup;
   std::vector<std::size_t> fAttrKernelShape, fAttrPads, fAttrStrides;
   std::string fNX, fNXS, fNXZ, fNW, fNWS, fNWZ, fNYS, fNYZ, fNB, fNY, fNM;
   bool fRelu = false, fInt32Out = false, fDynamic = false, fSumPlanes = false;
   float fPoolScale = 1.0f;
   std::string fNPooled;
   int fXLayout = kLayoutNCHW, fYLayout = kLayoutNCHW;
   ConvGeometry fGeo;
};

// DequantizeLinear(int8 feature map) followed by GlobalAveragePool, as one kernel over either layout
class ROperator_QGlobalAveragePool final : public ROperator {
public:
   ROperator_QGlobalAveragePool(std::string nameX, std::string nameScale, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNS(UTILITY::Clean_name(nameScale)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::QPOOL;
   }
   const std::string &ScaleName() const { return fNS; }
   const std::string &OutputName() const { return fNY; }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE GlobalAveragePool op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::INT8)
         throw std::runtime_error("SOFIE quantised GlobalAveragePool Op: input tensor " + fNX + " is not int8");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() < 3)
         throw std::runtime_error("SOFIE Pool Op input data tensor" + fNX + " has fewer than 3 dimensions");
      fScale = model.GetScalarInitializer(fNS);
      fLayout = model.GetTensorLayout(fNX);
      std::vector<std::size_t> shapeY(fShapeX.size(), 1);
      shapeY[0] = fShapeX[0];
      shapeY[1] = fShapeX[1];
      fDynamic = model.IsDynamicTensor(fNX);
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, shapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::size_t hw = 1;
      for (std::size_t i = 2; i < fShapeX.size(); ++i)
         hw *= fShapeX[i];
      std::stringstream out;
      out << "\n" << SP << "//----  DequantizeLinear + GlobalAveragePool " << opName << "\n";
      out << SP << "detail::Check(sofie_hip_global_avg_pool_i8(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << BatchScaledInt(fDynamic, fShapeX[0]) << ", " << fShapeX[1]
          << ", " << hw << ", " << (fLayout == kLayoutNHWC ? "SOFIE_LAYOUT_NHWC" : "SOFIE_LAYOUT_NCHW") << ", " << FloatLiteral(fScale) << "), \""
          << opName << " GlobalAveragePool\");\n";
      return out.str();
   }

private:
   std::string fNX, fNS, fNY;
   std::vector<std::size_t> fShapeX;
   float fScale = 1.0f;
   int fLayout = kLayoutNCHW;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
