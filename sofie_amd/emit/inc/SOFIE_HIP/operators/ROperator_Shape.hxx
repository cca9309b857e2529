// Operators that only move data: Reshape / Flatten / Squeeze / Unsqueeze (core/inc/SOFIE/operators/ROperator_Reshape.hxx: the four
// modes of one operator, :14, shape rules :95-215), Transpose (ROperator_Transpose.hxx: default perm reverses the axes) and Concat
// (ROperator_Concat.hxx: equal shapes but for the axis, :43-75).  The reshapes are device copies of the same bytes, the transpose one
// gather kernel, the concatenation one pitched copy per input.
#ifndef SOFIE_HIP_ROPERATOR_SHAPE
#define SOFIE_HIP_ROPERATOR_SHAPE

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

#include <numeric>

namespace SOFIE_HIP {

enum ReshapeOpMode { Reshape, Flatten, Squeeze, Unsqueeze };

class ROperator_Reshape final : public ROperator {
public:
   // Reshape: attr_value = allowzero, nameInput2 = the shape (an int64 initializer).  Flatten: attr_value = axis.
   // Squeeze / Unsqueeze from opset 13 on: nameInput2 = the axes (an int64 initializer; may be empty for Squeeze).
   ROperator_Reshape(ReshapeOpMode opMode, int attr_value, std::string nameData, std::string nameInput2, std::string nameOutput)
      : fOpMode(opMode), fNData(UTILITY::Clean_name(nameData)), fNInput2(UTILITY::Clean_name(nameInput2)), fNOutput(UTILITY::Clean_name(nameOutput))
   {
      if (opMode == Reshape)
         fAllowZero = attr_value;
      if (opMode == Flatten)
         fAxis = attr_value;
      fInputTensorNames = {fNData};
      fOutputTensorNames = {fNOutput};
   }
   // Squeeze / Unsqueeze with the axes as an attribute (before opset 13)
   ROperator_Reshape(ReshapeOpMode opMode, std::vector<int64_t> attrAxes, std::string nameData, std::string nameOutput)
      : fOpMode(opMode), fNData(UTILITY::Clean_name(nameData)), fNOutput(UTILITY::Clean_name(nameOutput)), fAttrAxes(std::move(attrAxes))
   {
      fInputTensorNames = {fNData};
      fOutputTensorNames = {fNOutput};
   }
   std::string Name() const { return fOpMode == Reshape ? "Reshape" : fOpMode == Flatten ? "Flatten" : fOpMode == Squeeze ? "Squeeze" : "Unsqueeze"; }

   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNData))
         throw std::runtime_error("SOFIE Reshape Op Input Tensor " + fNData + "  is not found in model");
      if (model.GetTensorLayout(fNData) != kLayoutNCHW)
         throw std::runtime_error("SOFIE " + Name() + " Op: input tensor " + fNData + " is stored channels-last");
      const std::vector<std::size_t> in = model.GetTensorShape(fNData);
      fType = model.GetTensorType(fNData);
      fDynamic = model.IsDynamicTensor(fNData);
      const std::size_t length = ConvertShapeToLength(in);
      std::vector<int64_t> param = fAttrAxes;
      if (!fNInput2.empty()) {
         if (!model.IsInitializedTensor(fNInput2) || model.GetTensorType(fNInput2) != ETensorType::INT64)
            throw std::runtime_error("SOFIE " + Name() + " Op: " + fNInput2 + " must be an int64 initializer (shapes computed at run time are not supported)");
         const int64_t *p = static_cast<const int64_t *>(model.GetInitializedTensorData(fNInput2).get());
         param.assign(p, p + ConvertShapeToLength(model.GetTensorShape(fNInput2)));
      }
      std::vector<std::size_t> out;
      const int64_t rank = static_cast<int64_t>(in.size());
      auto axisOf = [&](int64_t a, int64_t r) {
         if (a < -r || a >= r)
            throw std::runtime_error("SOFIE " + Name() + " Op: axis " + std::to_string(a) + " is out of range for " + fNData);
         return static_cast<std::size_t>(a < 0 ? a + r : a);
      };
      switch (fOpMode) {
      case Reshape: {
         // 0 copies the input's dimension (unless allowzero), one -1 takes what is left (ROperator_Reshape.hxx:100-150)
         std::size_t known = 1;
         int64_t free = -1;
         for (std::size_t i = 0; i < param.size(); ++i) {
            int64_t d = param[i];
            if (d == 0 && !fAllowZero) {
               if (i >= in.size())
                  throw std::runtime_error("SOFIE Reshape Op: a 0 in the shape of " + fNOutput + " has no input dimension to copy");
               d = static_cast<int64_t>(in[i]);
            }
            if (d == -1) {
               if (free >= 0)
                  throw std::runtime_error("SOFIE Reshape Op: more than one -1 in the shape of " + fNOutput);
               free = static_cast<int64_t>(i);
               out.push_back(1);
               continue;
            }
            if (d < 0)
               throw std::runtime_error("SOFIE Reshape Op: negative dimension in the shape of " + fNOutput);
            // with a run-time batch the leading dimension is the batch whatever the file wrote there
            if (fDynamic && i == 0)
               d = 1;
            out.push_back(static_cast<std::size_t>(d));
            known *= static_cast<std::size_t>(d);
         }
         if (free >= 0) {
            if (known == 0 || length % known != 0)
               throw std::runtime_error("SOFIE Reshape Op: the -1 in the shape of " + fNOutput + " does not divide " + std::to_string(length) + " elements");
            out[free] = length / known;
         }
         if (fDynamic && (free == 0 || out.empty()))
            throw std::runtime_error("SOFIE Reshape Op: the run-time batch of " + fNData + " must stay the leading dimension of " + fNOutput);
         break;
      }
      case Flatten: {
         const std::size_t axis = fAxis < 0 ? axisOf(fAxis, rank) : static_cast<std::size_t>(fAxis);
         if (axis > in.size())
            throw std::runtime_error("SOFIE Flatten Op: axis out of range for " + fNData);
         if (fDynamic && axis < 1)
            throw std::runtime_error("SOFIE Flatten Op: axis 0 would fold the run-time batch of " + fNData + " into the second dimension");
         std::size_t a = 1, b = 1;
         for (std::size_t i = 0; i < in.size(); ++i)
            (i < axis ? a : b) *= in[i];
         out = {a, b};
         break;
      }
      case Squeeze: {
         std::vector<bool> drop(in.size(), false);
         if (param.empty()) {
            for (std::size_t i = 0; i < in.size(); ++i)
               drop[i] = in[i] == 1 && !(fDynamic && i == 0);
         } else {
            for (int64_t a : param) {
               const std::size_t ax = axisOf(a, rank);
               if (in[ax] != 1 || (fDynamic && ax == 0))
                  throw std::runtime_error("SOFIE Squeeze Op: axis " + std::to_string(a) + " of " + fNData + " does not have length 1");
               drop[ax] = true;
            }
         }
         for (std::size_t i = 0; i < in.size(); ++i)
            if (!drop[i])
               out.push_back(in[i]);
         break;
      }
      case Unsqueeze: {
         const int64_t outRank = rank + static_cast<int64_t>(param.size());
         std::vector<bool> fresh(outRank, false);
         for (int64_t a : param) {
            const std::size_t ax = axisOf(a, outRank);
            if (fresh[ax])
               throw std::runtime_error("SOFIE Unsqueeze Op: axis " + std::to_string(a) + " is given twice");
            fresh[ax] = true;
         }
         if (fDynamic && fresh[0])
            throw std::runtime_error("SOFIE Unsqueeze Op: the run-time batch of " + fNData + " must stay the leading dimension");
         std::size_t next = 0;
         for (int64_t i = 0; i < outRank; ++i)
            out.push_back(fresh[i] ? 1 : in[next++]);
         break;
      }
      }
      if (ConvertShapeToLength(out) != length)
         throw std::runtime_error("SOFIE " + Name() + " Op: " + ConvertShapeToString(in) + " cannot become " + ConvertShapeToString(out));
      fBytes = length * GetTypeSize(fType);
      fShapeOut = out;
      model.AddIntermediateTensor(fNOutput, fType, out, fDynamic);
   }
   bool CanBeView() const override { return true; }
   void SetView(bool v) override { fIsView = v; }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//----  " << Name() << " " << opName << " --> " << ConvertShapeToString(fShapeOut) << "\n";
      if (fIsView) {
         out << SP << "// tensor_" << fNOutput << " is a view of tensor_" << fNData << " (same arena offset): nothing to copy\n";
         return out.str();
      }
      out << SP << "detail::Check(sofie_hip_copy(fCtx, tensor_" << fNOutput << ", tensor_" << fNData << ", " << BatchScaled(fDynamic, fBytes) << "), \"" << opName << " "
          << Name() << "\");\n";
      return out.str();
   }

private:
   ReshapeOpMode fOpMode;
   int fAllowZero = 0, fAxis = 1;
   std::string fNData, fNInput2, fNOutput;
   std::vector<int64_t> fAttrAxes;
   std::vector<std::size_t> fShapeOut;
   ETensorType fType = ETensorType::FLOAT;
   std::size_t fBytes = 0;
   bool fDynamic = false;
   bool fIsView = false;
};

template <typename T>
class ROperator_Transpose final : public ROperator {
   static_assert(sizeof(T) == 4, "the transpose kernel moves 4-byte elements");

public:
   ROperator_Transpose(std::vector<int64_t> attr_perm, std::string nameData, std::string nameOutput)
      : fAttrPerm(std::move(attr_perm)), fNData(UTILITY::Clean_name(nameData)), fNOutput(UTILITY::Clean_name(nameOutput))
   {
      fInputTensorNames = {fNData};
      fOutputTensorNames = {fNOutput};
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNData))
         throw std::runtime_error("SOFIE Tranpose Op Input Tensor " + fNData + " is not found in model");
      if (GetTypeSize(model.GetTensorType(fNData)) != 4 || model.GetTensorLayout(fNData) != kLayoutNCHW)
         throw std::runtime_error("SOFIE Transpose Op: input tensor " + fNData + " must hold 4-byte elements in the ONNX layout");
      fShapeX = model.GetTensorShape(fNData);
      const std::size_t rank = fShapeX.size();
      if (rank < 1 || rank > 6)
         throw std::runtime_error("SOFIE Transpose Op: rank " + std::to_string(rank) + " of " + fNData + " is not in [1, 6]");
      if (fAttrPerm.empty()) // the default reverses the axes (ROperator_Transpose.hxx:77-81)
         for (std::size_t i = 0; i < rank; ++i)
            fAttrPerm.push_back(static_cast<int64_t>(rank - 1 - i));
      if (fAttrPerm.size() != rank)
         throw std::runtime_error("SOFIE Transpose Op: perm has " + std::to_string(fAttrPerm.size()) + " entries for a tensor of rank " + std::to_string(rank));
      std::vector<bool> seen(rank, false);
      std::vector<std::size_t> shapeY(rank);
      for (std::size_t k = 0; k < rank; ++k) {
         if (fAttrPerm[k] < 0 || fAttrPerm[k] >= (int64_t)rank || seen[fAttrPerm[k]])
            throw std::runtime_error("SOFIE Transpose Op: perm of " + fNData + " is not a permutation");
         seen[fAttrPerm[k]] = true;
         shapeY[k] = fShapeX[fAttrPerm[k]];
      }
      fDynamic = model.IsDynamicTensor(fNData);
      if (fDynamic && fAttrPerm[0] != 0)
         throw std::runtime_error("SOFIE Transpose Op: the run-time batch of " + fNData + " must stay the leading dimension");
      model.AddIntermediateTensor(fNOutput, model.GetTensorType(fNData), shapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//----  Transpose " << opName << " " << ConvertShapeToString(fShapeX) << "\n";
      out << SP << "{\n";
      out << SP << "   " << "const std::int64_t shape[6] = {";
      for (std::size_t i = 0; i < 6; ++i)
         out << (i < fShapeX.size() ? BatchScaled(fDynamic && i == 0, fShapeX[i]) : std::string("1")) << (i < 5 ? ", " : "");
      out << "};\n";
      out << SP << "   " << "const std::int32_t perm[6] = {";
      for (std::size_t i = 0; i < 6; ++i)
         out << (i < fAttrPerm.size() ? fAttrPerm[i] : (int64_t)i) << (i < 5 ? ", " : "");
      out << "};\n";
      out << SP << "   " << "detail::Check(sofie_hip_transpose_f32(fCtx, reinterpret_cast<float *>(tensor_" << fNOutput << "), reinterpret_cast<const float *>(tensor_"
          << fNData << "), " << fShapeX.size() << ", shape, perm), \"" << opName << " Transpose\");\n";
      out << SP << "}\n";
      return out.str();
   }

private:
   std::vector<int64_t> fAttrPerm;
   std::string fNData, fNOutput;
   std::vector<std::size_t> fShapeX;
   bool fDynamic = false;
};

class ROperator_Concat final : public ROperator {
public:
   ROperator_Concat(std::vector<std::string> inputs, int axis, int newAxis, std::string output) : fAxis(axis), fNewAxis(newAxis), fNY(UTILITY::Clean_name(output))
   {
      for (auto &n : inputs)
         fInputs.push_back(UTILITY::Clean_name(n));
      fInputTensorNames = fInputs;
      fOutputTensorNames = {fNY};
   }
   void Initialize(RModel &model) override
   {
      if (fNewAxis)
         throw std::runtime_error("SOFIE Concat Op: ConcatFromSequence with new_axis is not supported");
      if (fInputs.empty())
         throw std::runtime_error("SOFIE Concat Op: no input");
      for (auto &n : fInputs) {
         if (!model.CheckIfTensorAlreadyExist(n))
            throw std::runtime_error("SOFIE Concat Op Input Tensor " + n + " is not found in model");
         if (GetTypeSize(model.GetTensorType(n)) != 4 || model.GetTensorType(n) != model.GetTensorType(fInputs[0]) || model.GetTensorLayout(n) != kLayoutNCHW)
            throw std::runtime_error("SOFIE Concat Op: input tensor " + n + " must hold 4-byte elements of the first input's type");
      }
      const auto first = model.GetTensorShape(fInputs[0]);
      const int rank = static_cast<int>(first.size());
      const int axis = fAxis < 0 ? fAxis + rank : fAxis;
      if (axis < 0 || axis >= rank)
         throw std::runtime_error("SOFIE Concat Op - invalid axis value ");
      fDynamic = model.IsDynamicTensor(fInputs[0]);
      if (fDynamic && axis == 0)
         throw std::runtime_error("SOFIE Concat Op: the axis is the run-time batch dimension");
      fShapeY = first;
      fShapeY[axis] = 0;
      fAxisLengths.clear();
      for (auto &n : fInputs) {
         const auto s = model.GetTensorShape(n);
         if ((int)s.size() != rank || model.IsDynamicTensor(n) != fDynamic)
            throw std::runtime_error("SOFIE Concat Op - input tensors have different shapes or are not all batched: " + n);
         for (int i = 0; i < rank; ++i)
            if (i != axis && s[i] != first[i])
               throw std::runtime_error("SOFIE Concat Op - input tensors have wrong shapes " + ConvertShapeToString(s) + " and " + ConvertShapeToString(first));
         fAxisLengths.push_back(s[axis]);
         fShapeY[axis] += s[axis];
      }
      fOuter = fInner = 1;
      for (int i = 0; i < axis; ++i)
         fOuter *= first[i];
      for (int i = axis + 1; i < rank; ++i)
         fInner *= first[i];
      fType = model.GetTensorType(fInputs[0]);
      model.AddIntermediateTensor(fNY, fType, fShapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//----  Concat " << opName << " --> " << ConvertShapeToString(fShapeY) << "\n";
      std::size_t total = 0, offset = 0;
      for (auto l : fAxisLengths)
         total += l;
      for (std::size_t i = 0; i < fInputs.size(); ++i) {
         if (fAxisLengths[i] == 0)
            continue;
         out << SP << "detail::Check(sofie_hip_copy_rows(fCtx, reinterpret_cast<char *>(tensor_" << fNY << ") + " << offset * fInner * 4 << ", " << total * fInner * 4
             << ", tensor_" << fInputs[i] << ", " << fAxisLengths[i] * fInner * 4 << ", " << BatchScaled(fDynamic, fOuter) << ", " << fAxisLengths[i] * fInner * 4
             << "), \"" << opName << " Concat\");\n";
         offset += fAxisLengths[i];
      }
      return out.str();
   }

private:
   int fAxis = 0, fNewAxis = 0;
   std::vector<std::string> fInputs;
   std::string fNY;
   std::vector<std::size_t> fShapeY, fAxisLengths;
   std::size_t fOuter = 1, fInner = 1;
   ETensorType fType = ETensorType::FLOAT;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
