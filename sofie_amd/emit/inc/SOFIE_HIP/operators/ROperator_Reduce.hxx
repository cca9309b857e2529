// ReduceSum / ReduceMean / ReduceSumSquare / ReduceProd / ReduceL2 / ReduceMax / ReduceMin
// (core/inc/SOFIE/operators/ROperator_Reduce.hxx: constructor :88-99, output shape :102-127, axes from the second input or the
// attribute, all axes when neither is given :136-148, the loops :349-400; parsers/src/ParseReduce.cxx:51-62 for keepdims = 1 and axes).
// The reduced axes must be adjacent: they then fold into the middle dimension of [outer, A, inner], which one launch reduces.
#ifndef SOFIE_HIP_ROPERATOR_REDUCE
#define SOFIE_HIP_ROPERATOR_REDUCE

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

enum EReduceOpMode { ReduceMean, ReduceSum, ReduceSumSquare, ReduceProd, ReduceL2, ReduceMax, ReduceMin, InvalidReduceOp };

template <EReduceOpMode Op>
class ROperator_Reduce final : public ROperator {
public:
   ROperator_Reduce(int keepdims, std::vector<int64_t> attrAxes, std::string nameX, std::string nameAxes, std::string nameY)
      : fkeepdims(keepdims), fAttrAxes(std::move(attrAxes)), fNX(UTILITY::Clean_name(nameX)), fNAxes(UTILITY::Clean_name(nameAxes)),
        fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   static std::string Name()
   {
      switch (Op) {
      case ReduceMean: return "ReduceMean";
      case ReduceSum: return "ReduceSum";
      case ReduceSumSquare: return "ReduceSumSquare";
      case ReduceProd: return "ReduceProd";
      case ReduceL2: return "ReduceL2";
      case ReduceMax: return "ReduceMax";
      case ReduceMin: return "ReduceMin";
      default: return "Invalid";
      }
   }
   // the SOFIE_REDUCE_* name of sofie_hip.h
   static std::string RuntimeCode()
   {
      switch (Op) {
      case ReduceMean: return "SOFIE_REDUCE_MEAN";
      case ReduceSum: return "SOFIE_REDUCE_SUM";
      case ReduceSumSquare: return "SOFIE_REDUCE_SUM_SQUARE";
      case ReduceProd: return "SOFIE_REDUCE_PROD";
      case ReduceL2: return "SOFIE_REDUCE_L2";
      case ReduceMax: return "SOFIE_REDUCE_MAX";
      default: return "SOFIE_REDUCE_MIN";
      }
   }
   void Initialize(RModel &model) override
   {
      static_assert(Op != InvalidReduceOp, "SOFIE - Reduce op mode not supported.");
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE Reduce Op Input Tensor " + fNX + " is not found in model");
      if (model.GetTensorType(fNX) != ETensorType::FLOAT || model.GetTensorLayout(fNX) != kLayoutNCHW)
         throw std::runtime_error("SOFIE " + Name() + " Op: input tensor " + fNX + " must be float in the ONNX layout");
      fShapeX = model.GetTensorShape(fNX);
      const int64_t rank = static_cast<int64_t>(fShapeX.size());
      if (!fNAxes.empty()) {
         if (!model.IsInitializedTensor(fNAxes) || model.GetTensorType(fNAxes) != ETensorType::INT64)
            throw std::runtime_error("SOFIE " + Name() + " Op: " + fNAxes + " must be an int64 initializer (axes computed at run time are not supported)");
         const int64_t *p = static_cast<const int64_t *>(model.GetInitializedTensorData(fNAxes).get());
         fAttrAxes.assign(p, p + ConvertShapeToLength(model.GetTensorShape(fNAxes)));
      }
      if (fAttrAxes.empty()) { // neither input nor attribute: everything is reduced
         for (int64_t i = 0; i < rank; ++i)
            fAttrAxes.push_back(i);
      }
      std::vector<bool> reduced(fShapeX.size(), false);
      for (int64_t &a : fAttrAxes) {
         if (a < 0)
            a += rank;
         if (a < 0 || a >= rank)
            throw std::runtime_error("SOFIE Reduce Op - invalid axes values " + std::to_string(a));
         reduced[a] = true;
      }
      std::size_t first = fShapeX.size(), last = 0;
      for (std::size_t i = 0; i < fShapeX.size(); ++i) {
         if (reduced[i]) {
            first = std::min(first, i);
            last = i;
         }
      }
      if (first == fShapeX.size()) { // a scalar input: the loop runs over its one element
         first = 0;
         last = 0;
      }
      for (std::size_t i = first; i <= last && i < fShapeX.size(); ++i) {
         if (!reduced[i] && fShapeX[i] != 1)
            throw std::runtime_error("SOFIE " + Name() + " Op: the reduced axes of " + fNX + " are not adjacent (" + ConvertShapeToString(fShapeX) + ")");
      }
      fOuter = fLength = fInner = 1;
      for (std::size_t i = 0; i < fShapeX.size(); ++i)
         (i < first ? fOuter : i <= last ? fLength : fInner) *= fShapeX[i];
      if (fLength == 0 || fLength > 0x7fffffffu)
         throw std::runtime_error("SOFIE " + Name() + " Op: reduced length of " + fNX + " is out of range");
      // a run-time batch in front: kept (it multiplies `outer`) or reduced away (it multiplies the reduced length)
      const bool dynamicX = model.IsDynamicTensor(fNX);
      fDynamicLength = dynamicX && first == 0 && !fShapeX.empty() && reduced[0];
      fDynamicOuter = dynamicX && !fDynamicLength;
      std::vector<std::size_t> shapeY;
      for (std::size_t i = 0; i < fShapeX.size(); ++i) {
         if (!reduced[i])
            shapeY.push_back(fShapeX[i]);
         else if (fkeepdims)
            shapeY.push_back(1);
      }
      if (fDynamicOuter && (shapeY.empty() || reduced[0]))
         throw std::runtime_error("SOFIE " + Name() + " Op: " + fNX + " loses its run-time batch dimension");
      fShapeY = shapeY;
      model.AddIntermediateTensor(fNY, ETensorType::FLOAT, fShapeY, fDynamicOuter);
   }
   bool ConsumesBatch() const override { return fDynamicLength; }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- " << Name() << " " << opName << " " << ConvertShapeToString(fShapeX) << " -> " << ConvertShapeToString(fShapeY) << "\n";
      out << SP << "detail::Check(sofie_hip_reduce_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << BatchScaled(fDynamicOuter, fOuter) << ", "
          << BatchScaledInt(fDynamicLength, fLength) << ", " << fInner << ", " << RuntimeCode() << "), \"" << opName << " " << Name() << "\");\n";
      return out.str();
   }

private:
   int fkeepdims = 1;
   std::vector<int64_t> fAttrAxes;
   std::string fNX, fNAxes, fNY;
   std::vector<std::size_t> fShapeX, fShapeY;
   std::size_t fOuter = 1, fLength = 1, fInner = 1;
   bool fDynamicOuter = false, fDynamicLength = false;
};

} // namespace SOFIE_HIP
#endif
