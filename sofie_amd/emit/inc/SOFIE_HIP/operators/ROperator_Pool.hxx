// MaxPool, AveragePool and GlobalAveragePool over one, two or three spatial dimensions
// (core/inc/SOFIE/operators/ROperator_Pool.hxx: attributes :17-26, shape inference :89-189, generated loops :286-475).
// The operator resolves attributes to one window description per spatial axis and emits one runtime call; the runtime
// kernel visits the window in the order of the reference's generated loops.
#ifndef SOFIE_HIP_ROPERATOR_POOL
#define SOFIE_HIP_ROPERATOR_POOL

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

#include <algorithm>

namespace SOFIE_HIP {

enum PoolOpMode { InvalidPoolOp, MaxPool, AveragePool, GlobalAveragePool };

// Same members as the reference's attribute block (ROperator_Pool.hxx:17-26).
struct RAttributes_Pool {
   std::string auto_pad = "NOTSET";
   int ceil_mode = 0;
   int count_include_pad = 0;
   int storage_order = 0;
   std::vector<std::size_t> dilations;
   std::vector<std::size_t> kernel_shape;
   std::vector<std::size_t> pads;
   std::vector<std::size_t> strides;
};

template <typename T>
class ROperator_Pool final : public ROperator {
public:
   ROperator_Pool(PoolOpMode mode, std::string nameX, std::string nameY) : ROperator_Pool(mode, RAttributes_Pool{}, nameX, nameY) {}
   ROperator_Pool(PoolOpMode mode, RAttributes_Pool attr, std::string nameX, std::string nameY)
      : fMode(mode), fAttr(std::move(attr)), fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      static_assert(std::is_same<T, float>::value, "SOFIE Encountered unsupported type parsing a Pool operator");
      if (mode == InvalidPoolOp)
         throw std::runtime_error("SOFIE Pool Op: invalid pooling mode");
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::POOL;
   }
   std::string Name() const { return fMode == MaxPool ? "MaxPool" : fMode == AveragePool ? "AveragePool" : "GlobalAveragePool"; }

   // One spatial axis after the attributes are resolved.
   struct Axis {
      std::size_t in = 1, out = 1, window = 1, stride = 1, padBegin = 0, padEnd = 0;
   };

   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE Pool op Input Tensor " + fNX + " is not found in model");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() < 3)
         throw std::runtime_error("SOFIE Pool Op input data tensor" + fNX + " has fewer than 3 dimensions");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Pool Op: input tensor " + fNX + " is not float");
      fDynamic = model.IsDynamicTensor(fNX);
      std::vector<std::size_t> shapeY(fShapeX.begin(), fShapeX.begin() + 2);
      if (fMode == GlobalAveragePool) {
         // the kernel is the image, no padding, no strides (ROperator_Pool.hxx:225-237)
         shapeY.resize(fShapeX.size(), 1);
      } else {
         const std::size_t nd = fShapeX.size() - 2;
         if (nd > 3)
            throw std::runtime_error("SOFIE " + Name() + " Op : pooling over 1, 2 or 3 spatial dimensions, tensor " + fNX + " has " +
                                     std::to_string(nd));
         if (fAttr.storage_order != 0)
            throw std::runtime_error("SOFIE " + Name() + " Op : storage_order = 1 is not supported");
         ResolveAxes(nd);
         for (std::size_t d = 0; d < nd; ++d)
            shapeY.push_back(fAxes[d].out);
      }
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, shapeY, fDynamic);
   }

   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//----  operator " << Name() << " " << opName << "\n";
      const std::string planes = BatchScaledInt(fDynamic, fShapeX[0] * fShapeX[1]);
      if (fMode == GlobalAveragePool) {
         std::size_t hw = 1;
         for (std::size_t i = 2; i < fShapeX.size(); ++i)
            hw *= fShapeX[i];
         out << SP << "detail::Check(sofie_hip_global_avg_pool_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << planes << ", " << hw << "), \""
             << opName << " GlobalAveragePool\");\n";
         return out.str();
      }
      // the divisor of an average follows the window over the border whenever there is padding or ceil_mode
      // (ROperator_Pool.hxx:323-327)
      bool dynamicDivisor3 = fAttr.ceil_mode != 0;
      for (auto &a : fAxes)
         dynamicDivisor3 |= a.padBegin > 0 || a.padEnd > 0;
      if (fAxes.size() == 3) {
         auto triple = [&](auto field) {
            return "{" + std::to_string(field(fAxes[0])) + ", " + std::to_string(field(fAxes[1])) + ", " + std::to_string(field(fAxes[2])) + "}";
         };
         out << SP << "{\n";
         out << SP << "   " << "sofie_pool3d_desc d{" << planes << ", " << triple([](const Axis &a) { return a.in; }) << ", " << triple([](const Axis &a) { return a.out; })
             << ", " << triple([](const Axis &a) { return a.window; }) << ", " << triple([](const Axis &a) { return a.padBegin; }) << ", "
             << triple([](const Axis &a) { return a.padEnd; }) << ", " << triple([](const Axis &a) { return a.stride; }) << ", "
             << (fMode == MaxPool ? "SOFIE_POOL_MAX" : "SOFIE_POOL_AVERAGE") << ", " << (fAttr.count_include_pad ? 1 : 0) << ", " << (dynamicDivisor3 ? 1 : 0) << "};\n";
         out << SP << "   " << "detail::Check(sofie_hip_pool3d_f32(fCtx, &d, tensor_" << fNY << ", tensor_" << fNX << "), \"" << opName << " " << Name() << "\");\n";
         out << SP << "}\n";
         return out.str();
      }
      // 1-D pooling runs as a 2-D pooling over images of one row
      const Axis one;
      const Axis &h = fAxes.size() == 2 ? fAxes[0] : one, &w = fAxes.size() == 2 ? fAxes[1] : fAxes[0];
      // the divisor of an average follows the window over the border whenever there is padding or ceil_mode
      // (ROperator_Pool.hxx:323-327)
      bool dynamicDivisor = fAttr.ceil_mode != 0;
      for (auto &a : fAxes)
         dynamicDivisor |= a.padBegin > 0 || a.padEnd > 0;
      out << SP << "{\n";
      out << SP << "   " << "sofie_pool_desc d{};\n";
      out << SP << "   " << "d.planes = " << planes << ";\n";
      out << SP << "   " << "d.H = " << h.in << "; d.W = " << w.in << "; d.OH = " << h.out << "; d.OW = " << w.out << ";\n";
      out << SP << "   " << "d.kh = " << h.window << "; d.kw = " << w.window << ";\n";
      out << SP << "   " << "d.pad_h0 = " << h.padBegin << "; d.pad_w0 = " << w.padBegin << "; d.pad_h1 = " << h.padEnd << "; d.pad_w1 = " << w.padEnd << ";\n";
      out << SP << "   " << "d.stride_h = " << h.stride << "; d.stride_w = " << w.stride << ";\n";
      out << SP << "   " << "d.mode = " << (fMode == MaxPool ? "SOFIE_POOL_MAX" : "SOFIE_POOL_AVERAGE") << ";\n";
      out << SP << "   " << "d.count_include_pad = " << (fAttr.count_include_pad ? 1 : 0) << "; d.dynamic_divisor = " << (dynamicDivisor ? 1 : 0) << ";\n";
      out << SP << "   " << "detail::Check(sofie_hip_pool_f32(fCtx, &d, tensor_" << fNY << ", tensor_" << fNX << "), \"" << opName << " " << Name() << "\");\n";
      out << SP << "}\n";
      return out.str();
   }

   const std::vector<Axis> &Axes() const { return fAxes; }

private:
   // Attribute defaults, auto_pad and the output extent, axis by axis (ROperator_Pool.hxx:107-171).
   void ResolveAxes(std::size_t nd)
   {
      auto &a = fAttr;
      if (!a.kernel_shape.empty() && a.kernel_shape.size() != nd)
         throw std::runtime_error("SOFIE " + Name() + " Op : kernel_shape has " + std::to_string(a.kernel_shape.size()) + " entries for " + std::to_string(nd) +
                                  " spatial dimensions");
      if ((!a.strides.empty() && a.strides.size() < nd) || (!a.dilations.empty() && a.dilations.size() < nd) || (!a.pads.empty() && a.pads.size() != 2 * nd))
         throw std::runtime_error("SOFIE " + Name() + " Op : strides, dilations or pads do not match the " + std::to_string(nd) + " spatial dimensions");
      if (a.auto_pad != "NOTSET" && a.auto_pad != "VALID" && a.auto_pad != "SAME_UPPER" && a.auto_pad != "SAME_LOWER")
         throw std::runtime_error("SOFIE" + Name() + "Op invalid Autopad value : " + a.auto_pad);
      fAxes.assign(nd, Axis{});
      for (std::size_t d = 0; d < nd; ++d) {
         Axis &x = fAxes[d];
         x.in = fShapeX[d + 2];
         const std::size_t k = a.kernel_shape.empty() ? x.in : a.kernel_shape[d];
         const std::size_t dil = a.dilations.empty() ? 1 : a.dilations[d];
         x.stride = a.strides.empty() ? 1 : a.strides[d];
         if (k == 0 || dil == 0 || x.stride == 0)
            throw std::runtime_error("SOFIE " + Name() + " Op : kernel, dilation and stride must be positive");
         // the reference pools over the whole dilated extent (:125-128)
         x.window = k + (dil - 1) * (k - 1);
         if (a.auto_pad == "NOTSET" && !a.pads.empty()) {
            x.padBegin = a.pads[d];
            x.padEnd = a.pads[d + nd];
         } else if (a.auto_pad == "SAME_UPPER" || a.auto_pad == "SAME_LOWER") {
            const std::size_t outSame = (x.in + x.stride - 1) / x.stride;
            const long long total = std::max(0LL, (long long)((outSame - 1) * x.stride + x.window) - (long long)x.in);
            const std::size_t small = (std::size_t)(total / 2), large = (std::size_t)(total - total / 2);
            x.padBegin = a.auto_pad == "SAME_UPPER" ? small : large;
            x.padEnd = a.auto_pad == "SAME_UPPER" ? large : small;
         }
         if (x.in + x.padBegin + x.padEnd < x.window)
            throw std::runtime_error("SOFIE " + Name() + " Op : the window (" + std::to_string(x.window) + ") is larger than the padded input of tensor " + fNX);
         const std::size_t n = x.in + x.padBegin + x.padEnd - x.window;
         // ceil_mode drops a last window that would begin beyond the input (:161-166)
         x.out = a.ceil_mode ? std::min((n + x.stride - 1) / x.stride, (x.in - 1 + x.padBegin) / x.stride) + 1 : n / x.stride + 1;
      }
   }

   PoolOpMode fMode;
   RAttributes_Pool fAttr;
   std::string fNX, fNY;
   std::vector<std::size_t> fShapeX;
   std::vector<Axis> fAxes;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
