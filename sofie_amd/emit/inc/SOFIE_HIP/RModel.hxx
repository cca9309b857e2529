// Model IR and Session generator of the gfx950 backend.  The model-building surface is the reference's
// (core/inc/SOFIE/RModel.hxx:105-215): AddInputTensorInfo, AddInitializedTensor, AddOperator,
// AddOutputTensorNameList, then GenerateGPU_HIP + OutputGenerated in place of Generate /
// GenerateGPU_ALPAKA.  The emitted header keeps `SOFIE_<model>::Session(std::string filename)` and
// `std::vector<float> infer(float const *...)` (core/src/RModel.cxx:1303-1334, 1529-1613).
#ifndef SOFIE_HIP_RMODEL
#define SOFIE_HIP_RMODEL

#include "SOFIE_HIP/MemoryPlanner.hxx"
#include "SOFIE_HIP/ROperator.hxx"

#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <set>
#include <utility>
#include <vector>

namespace SOFIE_HIP {

constexpr std::size_t kPoolAlignBytes = 256; // as the reference's GPU pool (core/src/RModel_ALPAKA.cxx:25)

class RModel {
public:
   RModel() = default;
   explicit RModel(std::string name);
   RModel(const RModel &) = delete;
   RModel &operator=(const RModel &) = delete;

   // ---- model building (the reference's names and meaning) ----
   void AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<std::size_t> shape);
   // an input whose LEADING dimension may be a named parameter (the batch): the Session then takes its maximum in
   // the constructor and its value in every infer call (core/src/RModel.cxx:1375-1395, 1537-1547); a positive
   // batchSize given to GenerateGPU_HIP fixes it at generation time instead
   void AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<Dim> shape);
   void AddInputTensorName(std::string name);
   void AddInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, std::shared_ptr<void> data);
   // copies `data` (length = product of shape)
   void AddInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, const void *data);
   void AddConstantTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, const void *data);
   // `batched`: the leading dimension is the run-time batch (given as 1 in `shape`)
   void AddIntermediateTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, bool batched = false);
   void AddOperator(std::unique_ptr<ROperator> op, int order_execution = -1);
   void AddOutputTensorNameList(std::vector<std::string> output_tensor_names);

   // ---- queries used by the operators ----
   bool CheckIfTensorAlreadyExist(const std::string &tensor_name) const;
   bool IsInitializedTensor(const std::string &name) const;
   bool IsInputTensor(const std::string &name) const;
   // an initialized tensor computed at generation time (embedded in the header, not in the weight file)
   bool IsConstantTensor(const std::string &name) const
   {
      auto f = fInitializedTensors.find(UTILITY::Clean_name(name));
      return f != fInitializedTensors.end() && f->second.constant;
   }
   const std::vector<std::size_t> &GetTensorShape(const std::string &name) const;
   ETensorType GetTensorType(const std::string &name) const;
   std::shared_ptr<void> GetInitializedTensorData(const std::string &name) const;
   void UpdateInitializedTensor(const std::string &name, ETensorType type, std::vector<std::size_t> shape, std::shared_ptr<void> data);
   // a float scalar initializer (scales of the quantised operators); throws if it is not one
   float GetScalarInitializer(const std::string &name) const;
   // storage order of a 4-D activation: kLayoutNCHW (what ONNX defines, the default) or kLayoutNHWC (kept
   // between quantised convolutions); set by the producing operator's Initialize
   void SetTensorLayout(const std::string &name, int layout) { fTensorLayout[UTILITY::Clean_name(name)] = layout; }
   int GetTensorLayout(const std::string &name) const
   {
      auto f = fTensorLayout.find(UTILITY::Clean_name(name));
      return f == fTensorLayout.end() ? kLayoutNCHW : f->second;
   }
   bool IsOutputTensor(const std::string &name) const;
   // true if the tensor's leading dimension is the run-time batch; its stored shape then has 1 there
   bool IsDynamicTensor(const std::string &name) const { return fBatched.count(UTILITY::Clean_name(name)) != 0; }
   // Options::kStridedInput: a graph input is read through strides handed to the Session's constructor
   // (core/src/RModel.cxx:376-385 of the reference)
   bool IsStridedInputTensor(const std::string &name) const
   {
      return fStridedInput && std::find(fInputTensorNames.begin(), fInputTensorNames.end(), UTILITY::Clean_name(name)) != fInputTensorNames.end();
   }
   bool HasDynamicBatch() const { return !fBatchParam.empty(); }
   const std::string &GetBatchParamName() const { return fBatchParam; }
   // kinds of the operators that read `name` (after fusion)
   std::vector<OperatorKind> ConsumerKinds(const std::string &name) const;
   const std::string &GetName() const { return fName; }
   const std::vector<std::unique_ptr<ROperator>> &Operators() const { return fOperators; }

   // ---- generation ----
   void GenerateGPU_HIP(std::underlying_type_t<Options> options, int batchSize = -1, bool verbose = false);
   void GenerateGPU_HIP(Options options = Options::kDefault, int batchSize = -1, bool verbose = false)
   {
      GenerateGPU_HIP(static_cast<std::underlying_type_t<Options>>(options), batchSize, verbose);
   }
   // writes <filename> (default <model>_GPU_HIP.hxx) and the weight file next to it (<stem>.dat)
   void OutputGenerated(std::string filename = "");
   const std::string &GetGeneratedCode() const { return fGC; }

   // ---- memory plan of the last generation (bytes), for tests and tooling ----
   struct PlannedTensor {
      std::string name;
      std::size_t offset, bytes;
      int begin, end; // lifetime in operator indices, [begin, end); statics have begin = -1
      bool pooled;
      bool perBatch = false; // offset and bytes are per batch entry, counted from the end of the static region
      bool view = false;     // placed on the tensor it is a view of (an operator that hands its input's bytes on unchanged)
   };
   const std::vector<PlannedTensor> &GetMemoryPlan() const { return fPlan; }
   std::size_t GetArenaBytes() const { return fArenaBytes; }
   std::size_t GetIntermediateMemoryPoolSize() const { return fPoolBytes; }
   // with a run-time batch the arena is GetStaticBytes() + capacity * GetBytesPerBatchEntry()
   std::size_t GetStaticBytes() const { return fStaticBytes; }
   std::size_t GetBytesPerBatchEntry() const { return fBatchEntryBytes; }

private:
   void Initialize(int batchSize);
   void FuseGemmActivations();
   void TryFuseResidual(std::size_t i);
   void TryFusePlaneSums(std::size_t i);
   void PlanMemory();
   void PlanMemoryPass(const std::set<std::size_t> &wholeChain);
   // Runs of consecutive Gemm operators of which each reads what the one before wrote: {first operator, count >= 2}.
   // Such a run goes to the runtime as ONE call that may execute every layer in a single launch, so the memory plan
   // treats it as one operator.
   std::vector<std::pair<std::size_t, std::size_t>> GemmChains() const;
   void GenerateSessionCode(std::underlying_type_t<Options> options);
   void WriteWeightFile(const std::string &filename) const;
   void WriteSafetensorsFile(const std::string &filename) const;

   std::string fName = "Model";
   std::vector<std::string> fInputTensorNames;
   std::vector<std::string> fOutputTensorNames;
   std::unordered_map<std::string, TensorInfo> fInputTensorInfos;
   std::map<std::string, InitializedTensor> fInitializedTensors; // ordered: header and weight file agree by construction
   std::unordered_map<std::string, TensorInfo> fIntermediateTensorInfos;
   std::vector<std::unique_ptr<ROperator>> fOperators;
   std::vector<PlannedTensor> fPlan;
   std::unordered_map<std::string, std::size_t> fOffsets;
   std::unordered_map<std::string, int> fTensorLayout;
   std::size_t fArenaBytes = 0, fPoolBytes = 0, fStaticBytes = 0, fBatchEntryBytes = 0;
   std::size_t fPoolBase = 0, fPoolFreeBytes = 0, fPoolLargestFreeBlock = 0;
   std::unordered_map<std::string, std::vector<Dim>> fInputDimShapes;
   std::unordered_map<std::string, bool> fBatched;
   std::string fBatchParam;
   std::size_t fBatchDefault = 1;
   bool fInitialized = false;
   bool fSafetensors = false;
   bool fStridedInput = false;
   std::string fGC;
   std::string fWeightFileName;

   friend class FusionPlanner;
};

} // namespace SOFIE_HIP
#endif
