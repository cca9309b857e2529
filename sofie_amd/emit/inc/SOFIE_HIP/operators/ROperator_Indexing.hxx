// Slice, Split, Expand, Tile and Gather with constant parameters (core/inc/SOFIE/operators/ROperator_Slice.hxx :54-80 constructors,
// ROperator_Split.hxx:31-90, ROperator_Expand.hxx:33-37, ROperator_Tile.hxx:29-33, ROperator_Gather.hxx:41-45; parsers/src/ParseSlice.cxx,
// ParseSplit.cxx, ParseExpand.cxx, ParseTile.cxx, ParseGather.cxx).  Starts, ends, steps, split sizes, target shapes, repeats and indices must
// be int64 initializers or attributes: each operator then is one strided read of its input (Gather: one pitched copy per index).
// A run-time batch has to stay the untouched leading dimension.
#ifndef SOFIE_HIP_ROPERATOR_INDEXING
#define SOFIE_HIP_ROPERATOR_INDEXING

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

namespace detail_indexing {

inline std::vector<int64_t> Int64Initializer(RModel &model, const std::string &op, const std::string &name)
{
   if (!model.IsInitializedTensor(name) || model.GetTensorType(name) != ETensorType::INT64)
      throw std::runtime_error("SOFIE " + op + " Op: " + name + " must be an int64 initializer (values computed at run time are not supported)");
   const int64_t *p = static_cast<const int64_t *>(model.GetInitializedTensorData(name).get());
   return std::vector<int64_t>(p, p + ConvertShapeToLength(model.GetTensorShape(name)));
}

inline std::vector<std::size_t> DenseStrides(const std::vector<std::size_t> &shape)
{
   std::vector<std::size_t> s(shape.size(), 1);
   for (std::size_t i = shape.size(); i-- > 1;)
      s[i - 1] = s[i] * shape[i];
   return s;
}

// the call that reads `in` (inLength elements per batch entry) through outShape / strides / offset into `out`
inline std::string EmitStridedGather(const std::string &opName, const std::string &what, const std::string &out, const std::string &in, bool dynamic,
                                     const std::vector<std::size_t> &outShape, const std::vector<int64_t> &strides, int64_t offset, std::size_t inLength)
{
   const std::string SP = "      "; // the operators' indentation inside doInfer
   std::stringstream o;
   o << SP << "{\n";
   o << SP << "   const std::int64_t shape[6] = {";
   for (std::size_t i = 0; i < 6; ++i)
      o << (i < outShape.size() ? BatchScaled(dynamic && i == 0, outShape[i]) : std::string("1")) << (i < 5 ? ", " : "");
   o << "};\n";
   o << SP << "   const std::int64_t strides[6] = {";
   for (std::size_t i = 0; i < 6; ++i)
      o << (i < strides.size() ? strides[i] : (int64_t)0) << (i < 5 ? ", " : "");
   o << "};\n";
   o << SP << "   detail::Check(sofie_hip_strided_gather_f32(fCtx, reinterpret_cast<float *>(tensor_" << out << "), reinterpret_cast<const float *>(tensor_" << in
     << "), " << outShape.size() << ", shape, strides, " << offset << ", " << BatchScaled(dynamic, inLength) << "), \"" << opName << " " << what << "\");\n";
   o << SP << "}\n";
   return o.str();
}

inline void CheckInput(RModel &model, const std::string &op, const std::string &name, std::size_t maxRank = 6)
{
   if (!model.CheckIfTensorAlreadyExist(name))
      throw std::runtime_error("SOFIE " + op + " Op Input Tensor " + name + " is not found in model");
   if (GetTypeSize(model.GetTensorType(name)) != 4 || model.GetTensorLayout(name) != kLayoutNCHW)
      throw std::runtime_error("SOFIE " + op + " Op: input tensor " + name + " must hold 4-byte elements in the ONNX layout");
   const std::size_t rank = model.GetTensorShape(name).size();
   if (rank < 1 || rank > maxRank)
      throw std::runtime_error("SOFIE " + op + " Op: rank " + std::to_string(rank) + " of " + name + " is not in [1, " + std::to_string(maxRank) + "]");
}

} // namespace detail_indexing

template <typename T, typename IType = int64_t>
class ROperator_Slice final : public ROperator {
public:
   // opset 10 and later: names = {starts, ends [, axes [, steps]]}
   ROperator_Slice(std::string nameData, std::vector<std::string> names, std::string nameOutput)
      : fNData(UTILITY::Clean_name(nameData)), fNOutput(UTILITY::Clean_name(nameOutput))
   {
      for (auto &n : names)
         fNames.push_back(UTILITY::Clean_name(n));
      fInputTensorNames = {fNData};
      fOutputTensorNames = {fNOutput};
   }
   // before opset 10: attributes
   ROperator_Slice(std::string nameData, std::vector<IType> starts, std::vector<IType> ends, std::vector<IType> axes, std::string nameOutput)
      : fNData(UTILITY::Clean_name(nameData)), fNOutput(UTILITY::Clean_name(nameOutput))
   {
      fAttr = {std::vector<int64_t>(starts.begin(), starts.end()), std::vector<int64_t>(ends.begin(), ends.end()), std::vector<int64_t>(axes.begin(), axes.end())};
      fInputTensorNames = {fNData};
      fOutputTensorNames = {fNOutput};
   }
   void Initialize(RModel &model) override
   {
      using namespace detail_indexing;
      CheckInput(model, "Slice", fNData);
      fShapeX = model.GetTensorShape(fNData);
      const int64_t rank = static_cast<int64_t>(fShapeX.size());
      std::vector<std::vector<int64_t>> p = fAttr;
      for (auto &n : fNames)
         p.push_back(n.empty() ? std::vector<int64_t>{} : Int64Initializer(model, "Slice", n));
      p.resize(4);
      if (p[0].size() != p[1].size())
         throw std::runtime_error("SOFIE Slice Op: starts and ends of " + fNData + " differ in length");
      if (p[2].empty()) // axes default to 0, 1, ...
         for (std::size_t i = 0; i < p[0].size(); ++i)
            p[2].push_back(static_cast<int64_t>(i));
      if (p[3].empty())
         p[3].assign(p[0].size(), 1);
      if (p[2].size() != p[0].size() || p[3].size() != p[0].size())
         throw std::runtime_error("SOFIE Slice Op: axes or steps of " + fNData + " do not match starts");
      fDynamic = model.IsDynamicTensor(fNData);
      const std::vector<std::size_t> dense = DenseStrides(fShapeX);
      fShapeY = fShapeX;
      fStrides.assign(dense.begin(), dense.end());
      fOffset = 0;
      for (std::size_t i = 0; i < p[0].size(); ++i) {
         int64_t axis = p[2][i] < 0 ? p[2][i] + rank : p[2][i];
         if (axis < 0 || axis >= rank)
            throw std::runtime_error("SOFIE Slice Op: axis " + std::to_string(p[2][i]) + " is out of range for " + fNData);
         if (fDynamic && axis == 0)
            throw std::runtime_error("SOFIE Slice Op: the run-time batch of " + fNData + " cannot be sliced");
         const int64_t d = static_cast<int64_t>(fShapeX[axis]), step = p[3][i];
         if (step == 0)
            throw std::runtime_error("SOFIE Slice Op: step 0 on axis " + std::to_string(axis) + " of " + fNData);
         // the ONNX rule: negative values count from the end, then starts clamp to [0, d] (to [0, d - 1] walking backwards) and ends to [0, d] ([-1, d - 1])
         int64_t start = p[0][i] < 0 ? p[0][i] + d : p[0][i], end = p[1][i] < 0 ? p[1][i] + d : p[1][i];
         if (step > 0) {
            start = std::min(std::max<int64_t>(start, 0), d);
            end = std::min(std::max<int64_t>(end, 0), d);
         } else {
            start = std::min(std::max<int64_t>(start, 0), d - 1);
            end = std::min(std::max<int64_t>(end, -1), d - 1);
         }
         const int64_t count = step > 0 ? (end - start + step - 1) / step : (start - end - step - 1) / (-step);
         fShapeY[axis] = static_cast<std::size_t>(std::max<int64_t>(count, 0));
         fOffset += start * static_cast<int64_t>(dense[axis]);
         fStrides[axis] = step * static_cast<int64_t>(dense[axis]);
      }
      if (ConvertShapeToLength(fShapeY) == 0)
         throw std::runtime_error("SOFIE Slice Op: the slice of " + fNData + " is empty");
      model.AddIntermediateTensor(fNOutput, model.GetTensorType(fNData), fShapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- Slice " << opName << " " << ConvertShapeToString(fShapeX) << " -> " << ConvertShapeToString(fShapeY) << "\n";
      out << detail_indexing::EmitStridedGather(opName, "Slice", fNOutput, fNData, fDynamic, fShapeY, fStrides, fOffset, ConvertShapeToLength(fShapeX));
      return out.str();
   }

private:
   std::string fNData, fNOutput;
   std::vector<std::string> fNames;
   std::vector<std::vector<int64_t>> fAttr;
   std::vector<std::size_t> fShapeX, fShapeY;
   std::vector<int64_t> fStrides;
   int64_t fOffset = 0;
   bool fDynamic = false;
};

class ROperator_Split final : public ROperator {
public:
   ROperator_Split(const std::string &nameX, const std::string &nameS, int axis, const std::vector<std::string> &namesY)
      : fAxis(axis), fNX(UTILITY::Clean_name(nameX)), fNSplit(UTILITY::Clean_name(nameS))
   {
      for (auto &n : namesY)
         fNYs.push_back(UTILITY::Clean_name(n));
      fInputTensorNames = {fNX};
      fOutputTensorNames = fNYs;
   }
   void Initialize(RModel &model) override
   {
      using namespace detail_indexing;
      CheckInput(model, "Split", fNX);
      fShapeX = model.GetTensorShape(fNX);
      const int rank = static_cast<int>(fShapeX.size());
      if (fAxis < 0)
         fAxis += rank;
      if (fAxis < 0 || fAxis >= rank)
         throw std::runtime_error("SOFIE Split - invalid axis " + std::to_string(fAxis));
      fDynamic = model.IsDynamicTensor(fNX);
      if (fDynamic && fAxis == 0)
         throw std::runtime_error("SOFIE Split - cannot compute an equal split of a dynamic (runtime-sized) axis 0 - provide explicit split sizes instead");
      const std::size_t nsplit = fNYs.size();
      const int64_t axisDim = static_cast<int64_t>(fShapeX[fAxis]);
      if (nsplit == 0)
         throw std::runtime_error("SOFIE Split - no outputs");
      if (fNSplit.empty()) { // equal parts; what does not divide goes, shorter, into the last one (ROperator_Split.hxx:58-72)
         if (axisDim % (int64_t)nsplit == 0) {
            fSplit.assign(nsplit, axisDim / (int64_t)nsplit);
         } else {
            const int64_t v = (axisDim + (int64_t)nsplit - 1) / (int64_t)nsplit;
            fSplit.assign(nsplit - 1, v);
            fSplit.push_back(axisDim % v);
         }
      } else {
         fSplit = Int64Initializer(model, "Split", fNSplit);
         if (fSplit.size() != nsplit)
            throw std::runtime_error("SOFIE Split - split input tensor has invalid shape");
      }
      int64_t total = 0;
      for (int64_t s : fSplit) {
         if (s <= 0)
            throw std::runtime_error("SOFIE Split - split sizes must be positive");
         total += s;
      }
      if (total != axisDim)
         throw std::runtime_error("SOFIE Split - Sum of split sizes must match the input dimension along the axis");
      for (std::size_t i = 0; i < nsplit; ++i) {
         std::vector<std::size_t> shapeY = fShapeX;
         shapeY[fAxis] = static_cast<std::size_t>(fSplit[i]);
         model.AddIntermediateTensor(fNYs[i], model.GetTensorType(fNX), shapeY, fDynamic);
      }
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      using namespace detail_indexing;
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- Split " << opName << " " << ConvertShapeToString(fShapeX) << " along axis " << fAxis << "\n";
      const std::vector<std::size_t> dense = DenseStrides(fShapeX);
      const std::vector<int64_t> strides(dense.begin(), dense.end());
      int64_t start = 0;
      for (std::size_t i = 0; i < fNYs.size(); ++i) {
         std::vector<std::size_t> shapeY = fShapeX;
         shapeY[fAxis] = static_cast<std::size_t>(fSplit[i]);
         out << EmitStridedGather(opName, "Split", fNYs[i], fNX, fDynamic, shapeY, strides, start * strides[fAxis], ConvertShapeToLength(fShapeX));
         start += fSplit[i];
      }
      return out.str();
   }

private:
   int fAxis;
   std::string fNX, fNSplit;
   std::vector<std::string> fNYs;
   std::vector<std::size_t> fShapeX;
   std::vector<int64_t> fSplit;
   bool fDynamic = false;
};

template <typename T>
class ROperator_Expand final : public ROperator {
public:
   ROperator_Expand(std::string nameX, std::string nameShape, std::string nameY)
      : fNX(UTILITY::Clean_name(nameX)), fNShape(UTILITY::Clean_name(nameShape)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   void Initialize(RModel &model) override
   {
      using namespace detail_indexing;
      CheckInput(model, "Expand", fNX);
      fShapeX = model.GetTensorShape(fNX);
      const std::vector<int64_t> target = Int64Initializer(model, "Expand", fNShape);
      fDynamic = model.IsDynamicTensor(fNX);
      // two-way broadcast of the input's shape and the target, aligned at the trailing axes
      const std::size_t rank = std::max(fShapeX.size(), target.size());
      if (rank > 6)
         throw std::runtime_error("SOFIE Expand Op: rank " + std::to_string(rank) + " of " + fNY + " is above 6");
      if (fDynamic && target.size() > fShapeX.size())
         throw std::runtime_error("SOFIE Expand Op: the run-time batch of " + fNX + " must stay the leading dimension");
      const std::vector<std::size_t> dense = DenseStrides(fShapeX);
      fShapeY.assign(rank, 1);
      fStrides.assign(rank, 0);
      for (std::size_t k = 0; k < rank; ++k) { // k counts from the last axis
         const std::size_t dx = k < fShapeX.size() ? fShapeX[fShapeX.size() - 1 - k] : 1;
         const int64_t dt = k < target.size() ? target[target.size() - 1 - k] : 1;
         if (dt < 0 || (dx != 1 && dt != 1 && static_cast<int64_t>(dx) != dt))
            throw std::runtime_error("SOFIE Expand Op: " + fNX + " of shape " + ConvertShapeToString(fShapeX) + " cannot be broadcast to the requested shape");
         fShapeY[rank - 1 - k] = dx != 1 ? dx : static_cast<std::size_t>(dt);
         fStrides[rank - 1 - k] = (dx != 1 && k < fShapeX.size()) ? static_cast<int64_t>(dense[fShapeX.size() - 1 - k]) : 0;
      }
      if (fDynamic) { // the batch axis: one entry per batch entry on both sides
         if (fShapeY[0] != 1)
            throw std::runtime_error("SOFIE Expand Op: the run-time batch of " + fNX + " cannot be expanded");
         fStrides[0] = static_cast<int64_t>(ConvertShapeToLength(fShapeX));
      }
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNX), fShapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- Expand " << opName << " " << ConvertShapeToString(fShapeX) << " -> " << ConvertShapeToString(fShapeY) << "\n";
      out << detail_indexing::EmitStridedGather(opName, "Expand", fNY, fNX, fDynamic, fShapeY, fStrides, 0, ConvertShapeToLength(fShapeX));
      return out.str();
   }

private:
   std::string fNX, fNShape, fNY;
   std::vector<std::size_t> fShapeX, fShapeY;
   std::vector<int64_t> fStrides;
   bool fDynamic = false;
};

template <typename T>
class ROperator_Tile final : public ROperator {
public:
   ROperator_Tile(std::string nameRepeat, std::string nameInput, std::string nameY)
      : fNRepeats(UTILITY::Clean_name(nameRepeat)), fNInput(UTILITY::Clean_name(nameInput)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNInput};
      fOutputTensorNames = {fNY};
   }
   void Initialize(RModel &model) override
   {
      using namespace detail_indexing;
      CheckInput(model, "Tile", fNInput);
      fShapeX = model.GetTensorShape(fNInput);
      const std::vector<int64_t> repeats = Int64Initializer(model, "Tile", fNRepeats);
      if (repeats.size() != fShapeX.size())
         throw std::runtime_error("SOFIE Tile Op: " + fNRepeats + " must hold one repeat per axis of " + fNInput);
      fDynamic = model.IsDynamicTensor(fNInput);
      if (fDynamic && repeats[0] != 1)
         throw std::runtime_error("SOFIE Tile Op: the run-time batch of " + fNInput + " cannot be repeated");
      // every axis becomes [repeat, length] with strides [0, stride]; axes that are not repeated, or hold one element, stay single
      const std::vector<std::size_t> dense = DenseStrides(fShapeX);
      fShapeY = fShapeX;
      for (std::size_t i = 0; i < fShapeX.size(); ++i) {
         if (repeats[i] <= 0)
            throw std::runtime_error("SOFIE Tile Op: repeats must be positive");
         fShapeY[i] = fShapeX[i] * static_cast<std::size_t>(repeats[i]);
         if (repeats[i] > 1) {
            fViewShape.push_back(static_cast<std::size_t>(repeats[i]));
            fViewStrides.push_back(0);
         }
         if (fShapeX[i] > 1 || repeats[i] == 1) {
            fViewShape.push_back(fShapeX[i]);
            fViewStrides.push_back(static_cast<int64_t>(dense[i]));
         }
      }
      // neighbours that walk the input in one stride (two kept axes of a dense input, two repeats) fold into one view axis
      for (std::size_t i = fDynamic ? 1 : 0; i + 1 < fViewShape.size();) {
         if (fViewStrides[i] == static_cast<int64_t>(fViewShape[i + 1]) * fViewStrides[i + 1]) {
            fViewShape[i] *= fViewShape[i + 1];
            fViewStrides[i] = fViewStrides[i + 1];
            fViewShape.erase(fViewShape.begin() + i + 1);
            fViewStrides.erase(fViewStrides.begin() + i + 1);
         } else {
            ++i;
         }
      }
      if (fViewShape.size() > 6)
         throw std::runtime_error("SOFIE Tile Op: " + fNInput + " repeats too many axes for one pass (at most 6 between repeated and kept axes)");
      if (fDynamic) {
         // the leading view axis is the batch (repeat 1): one input entry per output entry
         fViewStrides[0] = static_cast<int64_t>(ConvertShapeToLength(fShapeX));
      }
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNInput), fShapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- Tile " << opName << " " << ConvertShapeToString(fShapeX) << " -> " << ConvertShapeToString(fShapeY) << "\n";
      out << detail_indexing::EmitStridedGather(opName, "Tile", fNY, fNInput, fDynamic, fViewShape, fViewStrides, 0, ConvertShapeToLength(fShapeX));
      return out.str();
   }

private:
   std::string fNRepeats, fNInput, fNY;
   std::vector<std::size_t> fShapeX, fShapeY, fViewShape;
   std::vector<int64_t> fViewStrides;
   bool fDynamic = false;
};

class ROperator_Gather final : public ROperator {
public:
   ROperator_Gather(int64_t attrAxis, std::string nameX, std::string nameIndices, std::string nameY)
      : fAttrAxis(attrAxis), fNX(UTILITY::Clean_name(nameX)), fNIndices(UTILITY::Clean_name(nameIndices)), fNY(UTILITY::Clean_name(nameY))
   {
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
   }
   void Initialize(RModel &model) override
   {
      using namespace detail_indexing;
      CheckInput(model, "Gather", fNX, 8);
      fShapeX = model.GetTensorShape(fNX);
      const int64_t rank = static_cast<int64_t>(fShapeX.size());
      if (fAttrAxis < -rank || fAttrAxis >= rank)
         throw std::runtime_error("SOFIE Gather Op: axis " + std::to_string(fAttrAxis) + " is out of range for " + fNX);
      fAxis = static_cast<std::size_t>(fAttrAxis < 0 ? fAttrAxis + rank : fAttrAxis);
      fDynamic = model.IsDynamicTensor(fNX);
      if (fDynamic && fAxis == 0)
         throw std::runtime_error("SOFIE Gather Op: the run-time batch of " + fNX + " cannot be gathered from");
      fIndices = Int64Initializer(model, "Gather", fNIndices);
      const int64_t d = static_cast<int64_t>(fShapeX[fAxis]);
      for (int64_t &i : fIndices) { // negative indices count from the end (ROperator_Gather.hxx)
         if (i < -d || i >= d)
            throw std::runtime_error("SOFIE Gather Op: index " + std::to_string(i) + " is out of range for axis " + std::to_string(fAxis) + " of " + fNX);
         if (i < 0)
            i += d;
      }
      if (fIndices.empty() || fIndices.size() > 256)
         throw std::runtime_error("SOFIE Gather Op: " + fNIndices + " must hold between 1 and 256 constant indices");
      // output shape: the input's axes before the axis, the shape of the indices, the input's axes after it
      const std::vector<std::size_t> shapeI = model.GetTensorShape(fNIndices);
      fShapeY.assign(fShapeX.begin(), fShapeX.begin() + fAxis);
      fShapeY.insert(fShapeY.end(), shapeI.begin(), shapeI.end());
      fShapeY.insert(fShapeY.end(), fShapeX.begin() + fAxis + 1, fShapeX.end());
      fOuter = fInner = 1;
      for (std::size_t i = 0; i < fShapeX.size(); ++i)
         (i < fAxis ? fOuter : i > fAxis ? fInner : fLength) *= fShapeX[i];
      if (fShapeY.empty())
         fShapeY.push_back(1);
      model.AddIntermediateTensor(fNY, model.GetTensorType(fNX), fShapeY, fDynamic);
   }
   std::string Generate_GPU_HIP(std::string opName) override
   {
      opName = "op_" + opName;
      std::stringstream out;
      out << "\n" << SP << "//---- Gather " << opName << " " << ConvertShapeToString(fShapeX) << ", axis " << fAxis << ", " << fIndices.size() << " constant indices\n";
      const std::size_t K = fIndices.size(), rowBytes = fInner * 4;
      // runs of consecutive indices move as one piece
      for (std::size_t k = 0; k < K;) {
         std::size_t run = 1;
         while (k + run < K && fIndices[k + run] == fIndices[k] + (int64_t)run)
            ++run;
         out << SP << "detail::Check(sofie_hip_copy_rows(fCtx, reinterpret_cast<char *>(tensor_" << fNY << ") + " << k * rowBytes << ", " << K * rowBytes
             << ", reinterpret_cast<const char *>(tensor_" << fNX << ") + " << static_cast<std::size_t>(fIndices[k]) * rowBytes << ", " << fLength * rowBytes << ", "
             << BatchScaled(fDynamic, fOuter) << ", " << run * rowBytes << "), \"" << opName << " Gather\");\n";
         k += run;
      }
      return out.str();
   }

private:
   int64_t fAttrAxis;
   std::size_t fAxis = 0, fOuter = 1, fLength = 1, fInner = 1;
   std::string fNX, fNIndices, fNY;
   std::vector<std::size_t> fShapeX, fShapeY;
   std::vector<int64_t> fIndices;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
