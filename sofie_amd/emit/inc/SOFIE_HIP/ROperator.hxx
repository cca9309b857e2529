// Operator interface of the gfx950 emitter: the reference's ROperator contract (Initialize registers the
// outputs with the model, a Generate method returns C++ text that refers to tensors by name;
// core/inc/SOFIE/operators/ROperator.hxx:111-147) with the GPU methods this backend needs in place of the
// alpaka ones (core/inc/SOFIE/operators/ROperator_ALPAKA.hxx:23-56).
#ifndef SOFIE_HIP_ROPERATOR
#define SOFIE_HIP_ROPERATOR

#include "SOFIE_HIP/SOFIE_common.hxx"

namespace SOFIE_HIP {

class RModel;

enum class OperatorKind { GEMM, CONV, UNARY, BINARY, POOL, QUANTIZE, DEQUANTIZE, QGEMM, QCONV, QPOOL, OTHER };
constexpr int kLayoutNCHW = 0, kLayoutNHWC = 1;

class ROperator {
public:
   virtual ~ROperator() = default;
   // shape inference + registration of the output tensors (model.AddIntermediateTensor)
   virtual void Initialize(RModel &model) = 0;
   // C++ statements of Session::infer for this operator: calls into the C-ABI of include/sofie_hip.h.
   // A tensor X is referred to as `tensor_X` (a device pointer inside the Session's arena).
   virtual std::string Generate_GPU_HIP(std::string opName) = 0;
   // statements run once in the Session constructor after the weights are uploaded (weight re-layouts)
   virtual std::string GenerateInitCode_GPU_HIP() { return ""; }
   // bytes of persistent device memory the operator owns besides its tensors (packed weights): name -> bytes
   virtual std::vector<std::pair<std::string, std::size_t>> GetPersistentBuffers() { return {}; }
   // bytes of scratch the operator needs while it runs (planned like an intermediate tensor that lives for this operator)
   virtual std::size_t GetWorkspaceBytes() { return 0; }
   // in a model with a run-time batch: true if GetWorkspaceBytes() is the need of ONE batch entry
   virtual bool WorkspacePerBatchEntry() const { return false; }
   // An operator whose output holds the bytes of its input unchanged (Reshape, Flatten, Squeeze, Unsqueeze) can give its
   // output as a VIEW: the memory plan then places the output on the input and the operator generates no copy.  The plan
   // asks CanBeView() and tells the operator its decision with SetView().
   virtual bool CanBeView() const { return false; }
   virtual void SetView(bool) {}
   // Options::kStridedInput: true for an operator that reads a graph input through the strides given to the Session
   // (the reference's default is false too, core/inc/SOFIE/operators/ROperator.hxx:121)
   virtual bool SupportsStridedInput() const { return false; }
   // true for an operator that reads a tensor with a run-time batch and folds the batch away (a reduction over it): its outputs carry none
   virtual bool ConsumesBatch() const { return false; }
   virtual OperatorKind GetKind() const { return fKind; }
   const std::vector<std::string> &GetInputTensorNames() const { return fInputTensorNames; }
   const std::vector<std::string> &GetOutputTensorNames() const { return fOutputTensorNames; }
   // set by the generator: the operator's position and the name of its workspace tensor
   void SetOpOrder(std::size_t i) { fOpOrder = i; }
   std::size_t GetOpOrder() const { return fOpOrder; }

protected:
   OperatorKind fKind = OperatorKind::OTHER;
   std::size_t fOpOrder = 0;
   std::vector<std::string> fInputTensorNames;
   std::vector<std::string> fOutputTensorNames;
   const std::string SP = "      ";
};

} // namespace SOFIE_HIP
#endif
