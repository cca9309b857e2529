// Model IR, fusion, memory plan and Session text of the gfx950 backend.
#include "SOFIE_HIP/RModel.hxx"
#include "SOFIE_HIP/operators/OperatorList.hxx"

#include <cmath>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <limits>
#include <set>
#include <sstream>

namespace SOFIE_HIP {

static std::size_t AlignUp(std::size_t v) { return (v + kPoolAlignBytes - 1) / kPoolAlignBytes * kPoolAlignBytes; }

RModel::RModel(std::string name)
{
   // the model name is the file name without directory and extension, as the reference derives it
   auto slash = name.find_last_of("/\\");
   if (slash != std::string::npos)
      name = name.substr(slash + 1);
   auto dot = name.find_last_of('.');
   if (dot != std::string::npos)
      name = name.substr(0, dot);
   fName = UTILITY::Clean_name(name);
}

void RModel::AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<std::size_t> shape)
{
   input_name = UTILITY::Clean_name(input_name);
   if (CheckIfTensorAlreadyExist(input_name))
      throw std::runtime_error("SOFIE: input tensor with name " + input_name + " already exists \n");
   CheckedShapeLength(shape, input_name);
   fInputTensorInfos[input_name] = TensorInfo{type, shape};
}

void RModel::AddInputTensorInfo(std::string input_name, ETensorType type, std::vector<Dim> shape)
{
   std::vector<std::size_t> fixed;
   bool anyParam = false;
   for (std::size_t i = 0; i < shape.size(); ++i) {
      if (shape[i].isParam) {
         if (i != 0)
            throw std::runtime_error("SOFIE: input tensor " + input_name + " has the parameter " + shape[i].param +
                                     " in dimension " + std::to_string(i) + "; only the leading (batch) dimension may be a parameter");
         anyParam = true;
      }
      fixed.push_back(shape[i].isParam ? 1 : shape[i].dim);
   }
   AddInputTensorInfo(input_name, type, fixed);
   if (anyParam)
      fInputDimShapes[UTILITY::Clean_name(input_name)] = std::move(shape);
}

void RModel::AddInputTensorName(std::string name) { fInputTensorNames.push_back(UTILITY::Clean_name(name)); }

void RModel::AddInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, std::shared_ptr<void> data)
{
   tensor_name = UTILITY::Clean_name(tensor_name);
   if (CheckIfTensorAlreadyExist(tensor_name))
      throw std::runtime_error("SOFIE: initialized tensor with name " + tensor_name + " already exists \n");
   if (GetTypeSize(type) == 0)
      throw std::runtime_error("SOFIE: initialized tensor " + tensor_name + " has a type this backend cannot store");
   fInitializedTensors[tensor_name] = InitializedTensor{type, shape, data, false};
}

void RModel::AddInitializedTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, const void *data)
{
   const std::size_t bytes = ConvertShapeToLength(shape) * GetTypeSize(type);
   std::shared_ptr<void> copy(malloc(bytes ? bytes : 1), free);
   if (bytes)
      std::memcpy(copy.get(), data, bytes);
   AddInitializedTensor(tensor_name, type, shape, copy);
}

void RModel::AddConstantTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, const void *data)
{
   AddInitializedTensor(tensor_name, type, shape, data);
   fInitializedTensors[UTILITY::Clean_name(tensor_name)].constant = true;
}

void RModel::AddIntermediateTensor(std::string tensor_name, ETensorType type, std::vector<std::size_t> shape, bool batched)
{
   tensor_name = UTILITY::Clean_name(tensor_name);
   if (CheckIfTensorAlreadyExist(tensor_name))
      throw std::runtime_error("SOFIE: intermediate tensor with name " + tensor_name + " already exists \n");
   CheckedShapeLength(shape, tensor_name);
   if (batched && (shape.empty() || shape[0] != 1))
      throw std::runtime_error("SOFIE: tensor " + tensor_name + " does not carry the run-time batch as its leading dimension");
   fIntermediateTensorInfos[tensor_name] = TensorInfo{type, shape};
   if (batched)
      fBatched[tensor_name] = true;
}

void RModel::AddOperator(std::unique_ptr<ROperator> op, int order_execution)
{
   if (order_execution >= 0 && (std::size_t)order_execution <= fOperators.size())
      fOperators.insert(fOperators.begin() + order_execution, std::move(op));
   else
      fOperators.push_back(std::move(op));
}

void RModel::AddOutputTensorNameList(std::vector<std::string> names)
{
   fOutputTensorNames.clear();
   for (auto &n : names)
      fOutputTensorNames.push_back(UTILITY::Clean_name(n));
}

bool RModel::CheckIfTensorAlreadyExist(const std::string &n) const
{
   return fInputTensorInfos.count(n) || fInitializedTensors.count(n) || fIntermediateTensorInfos.count(n);
}
bool RModel::IsInitializedTensor(const std::string &n) const { return fInitializedTensors.count(UTILITY::Clean_name(n)) != 0; }
bool RModel::IsInputTensor(const std::string &n) const { return fInputTensorInfos.count(UTILITY::Clean_name(n)) != 0; }

const std::vector<std::size_t> &RModel::GetTensorShape(const std::string &name) const
{
   auto a = fInputTensorInfos.find(name);
   if (a != fInputTensorInfos.end())
      return a->second.shape;
   auto b = fInitializedTensors.find(name);
   if (b != fInitializedTensors.end())
      return b->second.shape;
   auto c = fIntermediateTensorInfos.find(name);
   if (c != fIntermediateTensorInfos.end())
      return c->second.shape;
   throw std::runtime_error("SOFIE tensor [" + name + "] for which the shape is requested is not found");
}

ETensorType RModel::GetTensorType(const std::string &name) const
{
   auto a = fInputTensorInfos.find(name);
   if (a != fInputTensorInfos.end())
      return a->second.type;
   auto b = fInitializedTensors.find(name);
   if (b != fInitializedTensors.end())
      return b->second.type;
   auto c = fIntermediateTensorInfos.find(name);
   if (c != fIntermediateTensorInfos.end())
      return c->second.type;
   throw std::runtime_error("SOFIE tensor [" + name + "] for which the type is requested is not found");
}

std::shared_ptr<void> RModel::GetInitializedTensorData(const std::string &name) const
{
   auto f = fInitializedTensors.find(name);
   if (f == fInitializedTensors.end())
      throw std::runtime_error("SOFIE tensor [" + name + "] for which the data is requested is not found");
   return f->second.data;
}

void RModel::UpdateInitializedTensor(const std::string &name, ETensorType type, std::vector<std::size_t> shape, std::shared_ptr<void> data)
{
   auto f = fInitializedTensors.find(name);
   if (f == fInitializedTensors.end())
      throw std::runtime_error("SOFIE tensor [" + name + "] for which update is requested is not found");
   f->second = InitializedTensor{type, shape, data, f->second.constant};
}

float RModel::GetScalarInitializer(const std::string &name) const
{
   auto f = fInitializedTensors.find(UTILITY::Clean_name(name));
   if (f == fInitializedTensors.end() || f->second.type != ETensorType::FLOAT || ConvertShapeToLength(f->second.shape) != 1)
      throw std::runtime_error("SOFIE: " + name + " must be a float scalar initializer (per-tensor scale)");
   return *static_cast<const float *>(f->second.data.get());
}

// ---------------------------------------------------------------------------------------------------------
// Fusion.  (1) the reference's FuseGemmActivations (core/src/RModel_Fusion_ALPAKA.cxx:367-416): an
// activation that is the only consumer of a Gemm / Conv output, which is not a graph output, moves into
// that operator's store.  Unlike the reference's cuBLASLt epilogue it does not need a bias to be present.
// (2) the quantised chain MatMulInteger -> Relu -> DequantizeLinear -> QuantizeLinear folds, link by link
// under the same single-consumer rule, into the store of the int8 product.
// ---------------------------------------------------------------------------------------------------------
void RModel::FuseGemmActivations()
{
   auto consumers = [&](const std::string &t) {
      std::vector<std::size_t> c;
      for (std::size_t i = 0; i < fOperators.size(); ++i)
         for (auto &in : fOperators[i]->GetInputTensorNames())
            if (in == t)
               c.push_back(i);
      return c;
   };
   auto isOutput = [&](const std::string &t) { return std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), t) != fOutputTensorNames.end(); };
   bool changed = true;
   while (changed) {
      changed = false;
      for (std::size_t i = 0; i < fOperators.size() && !changed; ++i) {
         ROperator *op = fOperators[i].get();
         if (op->GetOutputTensorNames().size() != 1)
            continue;
         const std::string y = op->GetOutputTensorNames()[0];
         if (isOutput(y))
            continue;
         auto cons = consumers(y);
         if (cons.size() != 1)
            continue;
         ROperator *next = fOperators[cons[0]].get();
         auto *act = dynamic_cast<ROperator_Activation *>(next);
         const bool plainRelu = act && act->Activation() == EActivationType::RELU && act->Chain().size() == 1;
         // A one-to-one float operator behind a Gemm, a Conv or another one-to-one operator joins its producer: as the
         // producer's own activation when that slot is free and nothing is queued behind it, else as the next link of the
         // chain the kernel applies in its store (at most kMaxPostOps links).
         auto absorb = [&](auto *producer) {
            if (!act)
               return false;
            if (!producer->HasActivation() && producer->PostOpCount() == 0 && IsProducerActivation(act->Activation())) {
               producer->FuseActivation(act->Activation(), act->Alpha(), act->OutputName());
               return true;
            }
            auto links = act->Chain();
            if (producer->PostOpCount() + links.size() > kMaxPostOps)
               return false;
            for (auto &l : links)
               producer->AddPostOp(l, act->OutputName());
            return true;
         };
         if (auto *g = dynamic_cast<ROperator_Gemm<float> *>(op)) {
            changed = absorb(g);
         } else if (auto *c = dynamic_cast<ROperator_Conv<float> *>(op)) {
            changed = absorb(c);
         } else if (auto *u = dynamic_cast<ROperator_Activation *>(op)) {
            if (act && u->Chain().size() + act->Chain().size() <= kMaxPostOps) {
               for (auto &l : act->Chain())
                  u->AddPostOp(l, act->OutputName());
               changed = true;
            }
         } else if (auto *bn = dynamic_cast<ROperator_BatchNormalization<float> *>(op)) {
            if (plainRelu && !bn->HasActivation()) {
               bn->FuseRelu(act->OutputName());
               changed = true;
            }
         } else if (auto *qc = dynamic_cast<ROperator_QConv *>(op)) {
            if (plainRelu && !qc->HasRelu()) {
               qc->FuseRelu(act->OutputName());
               changed = true;
            }
         } else if (auto *dqp = dynamic_cast<ROperator_DequantizeLinear *>(op)) {
            // DequantizeLinear whose only reader is a GlobalAveragePool: one kernel on the int8 map
            if (dynamic_cast<ROperator_Pool<float> *>(next)) {
               fOperators[i] = std::make_unique<ROperator_QGlobalAveragePool>(dqp->GetInputTensorNames()[0], dqp->ScaleName(),
                                                                              next->GetOutputTensorNames()[0]);
               changed = true;
            }
         } else if (auto *q = dynamic_cast<ROperator_QGemm *>(op)) {
            if (q->OutputKind() == ROperator_QGemm::Out::I8_REQUANT && plainRelu && !q->ReluOnOutput()) {
               q->SetReluOnOutput(); // Relu on the requantised int8 value: max(sat8(x), 0)
               q->SetOutputName(act->OutputName());
               changed = true;
            } else if (q->OutputKind() == ROperator_QGemm::Out::I32 && plainRelu && !q->ReluOnAccumulator()) {
               q->SetReluOnAccumulator();
               q->SetOutputName(act->OutputName());
               changed = true;
            } else if (auto *dq = dynamic_cast<ROperator_DequantizeLinear *>(next)) {
               if (q->OutputKind() == ROperator_QGemm::Out::I32) {
                  q->SetDequantize(GetScalarInitializer(dq->ScaleName()));
                  q->SetOutputName(dq->OutputName());
                  changed = true;
               }
            } else if (auto *ql = dynamic_cast<ROperator_QuantizeLinear *>(next)) {
               if (q->OutputKind() == ROperator_QGemm::Out::F32) {
                  q->SetDequantizeQuantize(q->DequantScale(), GetScalarInitializer(ql->ScaleName()));
                  q->SetOutputName(ql->OutputName());
                  changed = true;
               }
            }
         }
         if (changed)
            fOperators.erase(fOperators.begin() + cons[0]);
      }
   }
}

// Gemm or Conv whose only reader is an Add with a tensor of the same shape that already exists (a graph input, a weight, or
// the output of an earlier operator): the Add joins the kernel's store, before the activation, and an activation behind the Add
// can then join as well.  Runs just before operator i is initialised, when the shapes of everything before it are known.
void RModel::TryFuseResidual(std::size_t i)
{
   ROperator *op = fOperators[i].get();
   auto *g = dynamic_cast<ROperator_Gemm<float> *>(op);
   auto *c = dynamic_cast<ROperator_Conv<float> *>(op);
   if ((!g && !c) || op->GetOutputTensorNames().size() != 1)
      return;
   if (g ? (g->HasActivation() || g->PostOpCount() || g->HasResidual()) : (c->HasActivation() || c->PostOpCount() || c->HasResidual()))
      return;
   const std::string y = op->GetOutputTensorNames()[0];
   if (IsOutputTensor(y))
      return;
   if (g && IsInitializedTensor(op->GetInputTensorNames()[0]) && IsInitializedTensor(op->GetInputTensorNames()[1]))
      return; // a product of weights: left whole, so that it can be folded into a constant
   std::size_t reader = fOperators.size(), readers = 0;
   for (std::size_t j = 0; j < fOperators.size(); ++j)
      for (auto &in : fOperators[j]->GetInputTensorNames())
         if (in == y) {
            reader = j;
            ++readers;
         }
   if (readers != 1 || reader <= i)
      return;
   auto *add = dynamic_cast<ROperator_BasicBinary<float, Add> *>(fOperators[reader].get());
   if (!add)
      return;
   const auto &in = add->GetInputTensorNames();
   const std::string other = in[0] == y ? in[1] : in[0];
   if (other == y || !CheckIfTensorAlreadyExist(other) || GetTensorType(other) != ETensorType::FLOAT)
      return;
   std::vector<std::size_t> shapeY;
   bool batched = false;
   try {
      if (g) {
         g->ResolveShapes(*this);
         shapeY = g->OutputShape();
         batched = g->IsBatched();
      } else {
         c->ResolveShapes(*this);
         shapeY = c->OutputShape();
         batched = c->IsBatched();
      }
   } catch (const std::exception &) {
      return; // the operator's own Initialize reports the problem
   }
   if (GetTensorShape(other) != shapeY || IsDynamicTensor(other) != batched)
      return; // a broadcasting Add stays an operator of its own
   const std::string sum = add->GetOutputTensorNames()[0];
   if (g)
      g->SetResidual(other, sum);
   else
      c->SetResidual(other, sum);
   fOperators.erase(fOperators.begin() + reader);
   FuseGemmActivations(); // what followed the Add may now join the same store
}

// A quantised convolution whose only reader is the fused DequantizeLinear + GlobalAveragePool, and whose shape the runtime can
// sum plane by plane in the kernel's store: the pooling joins the convolution and the feature map is never stored.  Runs just
// before operator i is initialised, like TryFuseResidual.
void RModel::TryFusePlaneSums(std::size_t i)
{
   auto *qc = dynamic_cast<ROperator_QConv *>(fOperators[i].get());
   if (!qc || qc->SumsPlanes())
      return;
   const std::string y = qc->OutputName();
   if (IsOutputTensor(y))
      return;
   std::size_t reader = fOperators.size(), readers = 0;
   for (std::size_t j = 0; j < fOperators.size(); ++j)
      for (auto &in : fOperators[j]->GetInputTensorNames())
         if (in == y) {
            reader = j;
            ++readers;
         }
   if (readers != 1 || reader <= i)
      return;
   auto *pool = dynamic_cast<ROperator_QGlobalAveragePool *>(fOperators[reader].get());
   if (!pool || !qc->CanSumPlanes(*this))
      return;
   qc->SumPlanes(GetScalarInitializer(pool->ScaleName()), pool->OutputName());
   fOperators.erase(fOperators.begin() + reader);
}

bool RModel::IsOutputTensor(const std::string &name) const
{
   return std::find(fOutputTensorNames.begin(), fOutputTensorNames.end(), UTILITY::Clean_name(name)) != fOutputTensorNames.end();
}

std::vector<OperatorKind> RModel::ConsumerKinds(const std::string &name) const
{
   std::vector<OperatorKind> kinds;
   const std::string n = UTILITY::Clean_name(name);
   for (auto &op : fOperators)
      for (auto &in : op->GetInputTensorNames())
         if (in == n)
            kinds.push_back(op->GetKind());
   return kinds;
}

void RModel::Initialize(int batchSize)
{
   if (fInitialized)
      return;
   // the batch parameter: fixed now if a batch size is given, else left to the Session
   for (auto &kv : fInputDimShapes) {
      const Dim &d = kv.second[0];
      if (batchSize > 0) {
         fInputTensorInfos[kv.first].shape[0] = static_cast<std::size_t>(batchSize);
         continue;
      }
      if (!fBatchParam.empty() && fBatchParam != d.param)
         throw std::runtime_error("SOFIE: inputs use two shape parameters, " + fBatchParam + " and " + d.param +
                                  "; this backend takes one (the batch)");
      fBatchParam = d.param;
      fBatchDefault = std::max<std::size_t>(fBatchDefault, d.dim ? d.dim : 1);
      fBatched[kv.first] = true;
   }
   for (auto &n : fInputTensorNames)
      if (!fInputTensorInfos.count(n))
         throw std::runtime_error("SOFIE: input tensor " + n + " has no tensor info");
   if (fInputTensorNames.empty())
      for (auto &kv : fInputTensorInfos)
         fInputTensorNames.push_back(kv.first);
   FuseGemmActivations();
   for (std::size_t i = 0; i < fOperators.size(); ++i) {
      TryFuseResidual(i);
      TryFusePlaneSums(i);
      fOperators[i]->SetOpOrder(i);
      fOperators[i]->Initialize(*this);
      // an operator that reads a batched tensor has to say what it makes of the batch
      bool batchedIn = false, batchedOut = false;
      for (auto &in : fOperators[i]->GetInputTensorNames())
         batchedIn = batchedIn || IsDynamicTensor(in);
      for (auto &y : fOperators[i]->GetOutputTensorNames())
         batchedOut = batchedOut || IsDynamicTensor(y);
      // every operator that reads a strided graph input must be able to read it through its strides
      // (core/src/RModel.cxx:764-772 of the reference)
      if (fStridedInput)
         for (auto &in : fOperators[i]->GetInputTensorNames())
            if (IsStridedInputTensor(in) && !fOperators[i]->SupportsStridedInput())
               throw std::runtime_error("sofie: Options::kStridedInput - operator " + std::to_string(i) + " (output " +
                                        fOperators[i]->GetOutputTensorNames().at(0) + ") reads the input tensor " + in +
                                        " but does not support strided input access");
      if (batchedIn && !batchedOut && !fOperators[i]->ConsumesBatch())
         throw std::runtime_error("SOFIE: operator " + std::to_string(i) + " (output " + fOperators[i]->GetOutputTensorNames().at(0) +
                                  ") does not support a run-time batch; generate with a fixed batch size");
   }
   for (auto &o : fOutputTensorNames)
      if (!CheckIfTensorAlreadyExist(o))
         throw std::runtime_error("SOFIE: output tensor " + o + " is not produced by any operator");
   fInitialized = true;
}

// ---------------------------------------------------------------------------------------------------------
// Memory plan: ONE arena.  Static regions first (weights, operator-owned buffers such as re-laid-out
// weights, graph inputs, graph outputs), each 256-byte aligned; then the pool of intermediates and operator
// workspaces, placed by OrganizeMemory from their lifetimes [producer, last consumer + 1), as the reference's
// GPU generator does (core/src/RModel_ALPAKA.cxx:360-540).
// ---------------------------------------------------------------------------------------------------------
std::vector<std::pair<std::size_t, std::size_t>> RModel::GemmChains() const
{
   std::vector<std::pair<std::size_t, std::size_t>> chains;
   for (std::size_t i = 0; i < fOperators.size(); ++i) {
      std::size_t n = 0;
      const ROperator_Gemm<float> *prev = nullptr;
      for (std::size_t j = i; j < fOperators.size() && n < kMaxGemmChain; ++j) {
         auto *g = dynamic_cast<const ROperator_Gemm<float> *>(fOperators[j].get());
         if (!g || !g->IsChainLink() || (prev && g->NameA() != prev->NameY()))
            break;
         prev = g;
         ++n;
      }
      if (n >= 2) {
         chains.emplace_back(i, n);
         i += n - 1;
      }
   }
   return chains;
}

void RModel::PlanMemory()
{
   std::set<std::size_t> wholeChain; // first operators of the chains whose tensors must not share memory at all
   for (;;) {
      PlanMemoryPass(wholeChain);
      bool again = false;
      for (auto &ch : GemmChains()) {
         if (wholeChain.count(ch.first))
            continue;
         // what the layers of this chain read and write, with its shape
         std::vector<std::pair<std::string, std::vector<std::size_t>>> tensors;
         for (std::size_t i = ch.first; i < ch.first + ch.second; ++i) {
            for (auto &n : fOperators[i]->GetInputTensorNames())
               tensors.emplace_back("tensor_" + std::string(n), GetTensorShape(std::string(n)));
            for (auto &n : fOperators[i]->GetOutputTensorNames())
               tensors.emplace_back("tensor_" + std::string(n), GetTensorShape(std::string(n)));
         }
         bool clash = false;
         for (std::size_t x = 0; x < tensors.size() && !clash; ++x)
            for (std::size_t y = x + 1; y < tensors.size() && !clash; ++y) {
               if (tensors[x].first == tensors[y].first || !fOffsets.count(tensors[x].first) || !fOffsets.count(tensors[y].first))
                  continue;
               const PlannedTensor *px = nullptr, *py = nullptr;
               for (auto &e : fPlan) {
                  if (e.name == tensors[x].first)
                     px = &e;
                  if (e.name == tensors[y].first)
                     py = &e;
               }
               if (!px || !py || px->perBatch != py->perBatch) // the per-entry region of a run-time batch lies apart from the static one
                  continue;
               const bool overlap = px->offset < py->offset + py->bytes && py->offset < px->offset + px->bytes;
               if (overlap && !(px->offset == py->offset && tensors[x].second == tensors[y].second))
                  clash = true;
            }
         if (clash) {
            wholeChain.insert(ch.first);
            again = true;
         }
      }
      if (!again)
         break;
   }
}

void RModel::PlanMemoryPass(const std::set<std::size_t> &wholeChain)
{
   fPlan.clear();
   fOffsets.clear();
   const bool dyn = HasDynamicBatch();
   // With a run-time batch the arena has two parts.  The static part holds what does not depend on the batch.  Everything
   // that carries the batch is planned for ONE batch entry, in units of 16 bytes; the Session multiplies those offsets by
   // its capacity (the maximum batch rounded up to a multiple of 16), so regions that are disjoint per entry stay disjoint
   // and every region starts on a 256-byte boundary.
   const std::size_t entryAlign = 16;
   auto alignEntry = [&](std::size_t b) { return (b + entryAlign - 1) / entryAlign * entryAlign; };
   std::size_t off = 0, entryOff = 0;
   auto addStatic = [&](const std::string &name, std::size_t bytes) {
      fPlan.push_back({name, off, bytes, -1, (int)fOperators.size() + 1, false, false});
      fOffsets[name] = off;
      off += AlignUp(bytes ? bytes : 1);
   };
   auto addPerEntry = [&](const std::string &name, std::size_t bytes) {
      fPlan.push_back({name, entryOff, bytes, -1, (int)fOperators.size() + 1, false, true});
      fOffsets[name] = entryOff;
      entryOff += alignEntry(bytes ? bytes : 1);
   };
   auto tensorBytes = [&](const TensorInfo &ti) { return ConvertShapeToLength(ti.shape) * GetTypeSize(ti.type); };
   for (auto &kv : fInitializedTensors)
      addStatic("tensor_" + kv.first, ConvertShapeToLength(kv.second.shape) * GetTypeSize(kv.second.type));
   for (auto &op : fOperators)
      for (auto &pb : op->GetPersistentBuffers())
         addStatic(pb.first, pb.second);
   auto addGraphTensor = [&](const std::string &n, const TensorInfo &ti) {
      if (IsDynamicTensor(n))
         addPerEntry("tensor_" + n, tensorBytes(ti));
      else
         addStatic("tensor_" + n, tensorBytes(ti));
   };
   for (auto &n : fInputTensorNames)
      addGraphTensor(n, fInputTensorInfos[n]);
   for (auto &n : fOutputTensorNames)
      if (fIntermediateTensorInfos.count(n))
         addGraphTensor(n, fIntermediateTensorInfos[n]);

   // A Gemm chain may run all its layers in one launch, every workgroup taking its rows through all the layers on its own.
   // Tensors of the chain may then share memory only row for row (equal shapes at the same offset: the ping-pong of equal
   // layers).  The plan is made from per-operator lifetimes first; a chain in which two tensors of different shape came to
   // share bytes is planned again with everything it touches live from its first operator to its last (`wholeChain`).
   std::vector<int> opFirst(fOperators.size()), opLast(fOperators.size());
   for (std::size_t i = 0; i < fOperators.size(); ++i)
      opFirst[i] = opLast[i] = (int)i;
   for (auto &ch : GemmChains())
      if (wholeChain.count(ch.first))
         for (std::size_t i = ch.first; i < ch.first + ch.second; ++i) {
            opFirst[i] = (int)ch.first;
            opLast[i] = (int)(ch.first + ch.second - 1);
         }
   // Views: the output of an operator that only hands its input's bytes on is placed ON its input when both live in the pool
   // (not a graph input or output, which have regions of their own).  The tensor at the root of a chain of views then lives
   // until the last reader of any of them.
   std::map<std::string, std::string> viewRoot; // view -> the pool tensor whose bytes it is
   std::vector<std::pair<std::string, std::size_t>> views; // (view, its operator) in operator order
   for (std::size_t i = 0; i < fOperators.size(); ++i) {
      auto &op = fOperators[i];
      if (!op->CanBeView())
         continue;
      op->SetView(false);
      if (op->GetInputTensorNames().empty() || op->GetOutputTensorNames().size() != 1)
         continue;
      const std::string x(op->GetInputTensorNames()[0]), y(op->GetOutputTensorNames()[0]);
      auto pooledTensor = [&](const std::string &t) {
         return fIntermediateTensorInfos.count(t) && !fOffsets.count("tensor_" + t) && (!dyn || IsDynamicTensor(t));
      };
      if (!pooledTensor(x) || !pooledTensor(y) || opFirst[i] != (int)i || opLast[i] != (int)i)
         continue;
      viewRoot[y] = viewRoot.count(x) ? viewRoot[x] : x;
      views.emplace_back(y, i);
      op->SetView(true);
   }
   std::vector<TensorLifeInfo> life;
   std::vector<std::string> names;
   for (std::size_t i = 0; i < fOperators.size(); ++i) {
      for (auto &y : fOperators[i]->GetOutputTensorNames()) {
         if (!fIntermediateTensorInfos.count(y) || fOffsets.count("tensor_" + y))
            continue; // graph outputs are placed above
         if (viewRoot.count(y))
            continue; // placed on its root below
         const auto &ti = fIntermediateTensorInfos[y];
         if (dyn && !IsDynamicTensor(y)) { // rare: an intermediate that does not depend on the batch keeps a region of its own
            addStatic("tensor_" + y, tensorBytes(ti));
            continue;
         }
         int last = opLast[i];
         for (std::size_t j = i + 1; j < fOperators.size(); ++j)
            for (auto &in : fOperators[j]->GetInputTensorNames()) {
               auto v = viewRoot.find(std::string(in));
               if (in == y || (v != viewRoot.end() && v->second == y))
                  last = std::max(last, opLast[j]);
            }
         life.push_back({opFirst[i], last + 1, dyn ? alignEntry(tensorBytes(ti)) : AlignUp(tensorBytes(ti))});
         names.push_back("tensor_" + y);
      }
      if (std::size_t ws = fOperators[i]->GetWorkspaceBytes()) {
         const std::string wname = "workspace_op_" + std::to_string(i);
         if (dyn && !fOperators[i]->WorkspacePerBatchEntry()) {
            addStatic(wname, ws);
            continue;
         }
         life.push_back({(int)i, (int)i + 1, dyn ? alignEntry(ws) : AlignUp(ws)});
         names.push_back(wname);
      }
   }
   const std::size_t poolBase = dyn ? entryOff : off;
   MemoryResult r = OrganizeMemory(life);
   for (std::size_t t = 0; t < life.size(); ++t) {
      fPlan.push_back({names[t], poolBase + r.offsets[t], life[t].size, life[t].begin, life[t].end, true, dyn});
      fOffsets[names[t]] = poolBase + r.offsets[t];
   }
   for (auto &v : views) {
      const std::string root = "tensor_" + viewRoot[v.first];
      for (std::size_t t = 0; t < life.size(); ++t)
         if (names[t] == root) {
            const auto &ti = fIntermediateTensorInfos[v.first];
            fPlan.push_back({"tensor_" + v.first, poolBase + r.offsets[t], dyn ? alignEntry(tensorBytes(ti)) : AlignUp(tensorBytes(ti)), (int)v.second,
                             life[t].end, true, dyn, true});
            fOffsets["tensor_" + v.first] = poolBase + r.offsets[t];
         }
   }
   fPoolBytes = r.total_bytes; // per batch entry when the batch is a run-time parameter
   fPoolBase = poolBase;
   fPoolFreeBytes = r.total_free_bytes;
   fPoolLargestFreeBlock = r.largest_free_block;
   fStaticBytes = off;
   fBatchEntryBytes = dyn ? entryOff + r.total_bytes : 0;
   fArenaBytes = dyn ? off + entryAlign * fBatchEntryBytes : poolBase + r.total_bytes; // dynamic: the smallest Session (capacity 16)
   if (fArenaBytes == 0)
      fArenaBytes = kPoolAlignBytes;
}

// ---------------------------------------------------------------------------------------------------------
// Session text
// ---------------------------------------------------------------------------------------------------------
static const char *kRuntimeHelpers = R"SOFIE(
namespace detail {
inline void Check(int status, const char *what)
{
   if (status != 0)
      throw std::runtime_error(std::string("SOFIE HIP runtime error in ") + what + ": " + sofie_hip_last_error());
}
// Reads one tensor of the text weight file: a header line `tensor_<name> <length>` and the values
// (the format of the reference's weight files, core/src/RModel.cxx:1929-1958).
template <class T>
inline void ReadTensorFromStream(std::istream &is, std::vector<T> &target, std::string const &expected_name, const std::size_t expected_length)
{
   std::string name;
   std::size_t length;
   is >> name >> length;
   if (name != expected_name) {
      std::string err_msg = "SOFIE failed to read the correct tensor name; expected name is " + expected_name + " , read " + name;
      throw std::runtime_error(err_msg);
   }
   if (length != expected_length) {
      std::string err_msg = "SOFIE failed to read the correct tensor size; expected size is " + std::to_string(expected_length) + " , read " + std::to_string(length);
      throw std::runtime_error(err_msg);
   }
   target.resize(length);
   for (std::size_t i = 0; i < length; ++i) {
      if (sizeof(T) == 1) {
         int v;
         is >> v;
         target[i] = static_cast<T>(v);
      } else {
         std::string tok;
         is >> tok;
         if (std::is_floating_point<T>::value)
            target[i] = static_cast<T>(std::strtod(tok.c_str(), nullptr));
         else
            target[i] = static_cast<T>(std::strtoll(tok.c_str(), nullptr, 10));
      }
   }
   if (is.fail())
      throw std::runtime_error("SOFIE failed to read the values for tensor " + expected_name);
}
} // namespace detail
)SOFIE";


// Weights in the safetensors container (the reference's Options::kSafetensorsWeightFile, core/src/RModel.cxx:1967-2010):
// 8 bytes little-endian header length, a JSON header {"tensor_<name>": {"dtype": "F32", "shape": [..], "data_offsets": [b, e]}, ...},
// then the raw little-endian tensor bytes.
static const char *kSafetensorsHelpers = R"SOFIE(
struct SafetensorsBlob {
   const char *data = nullptr;
   std::size_t size = 0;
   SafetensorsBlob() = default;
   SafetensorsBlob(const char *d, std::size_t n) : data(d), size(n) {}
   SafetensorsBlob(const std::string &s) : data(s.data()), size(s.size()) {}
};

namespace detail {
inline std::string LoadWeightsFromFile(const std::string &filename)
{
   std::ifstream f(filename, std::ios::binary);
   if (!f.is_open())
      throw std::runtime_error("tmva-sofie failed to open file " + filename + " for input weights");
   std::string bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
   if (f.bad())
      throw std::runtime_error("tmva-sofie failed to read file " + filename);
   return bytes;
}

// Reads the header of a safetensors payload once; Expect() checks a tensor against what the model needs,
// Data() returns where its bytes start.  Every inconsistency is a std::runtime_error naming the tensor.
class SafetensorsReader {
public:
   explicit SafetensorsReader(SafetensorsBlob blob)
   {
      if (!blob.data || blob.size < 8)
         throw std::runtime_error("SOFIE safetensors: the payload is shorter than its 8-byte header length");
      std::uint64_t n = 0;
      for (int i = 0; i < 8; ++i)
         n |= static_cast<std::uint64_t>(static_cast<unsigned char>(blob.data[i])) << (8 * i);
      if (n > blob.size - 8)
         throw std::runtime_error("SOFIE safetensors: the header length exceeds the payload");
      fText = blob.data + 8;
      fEnd = fText + n;
      fPayload = blob.data + 8 + n;
      fPayloadBytes = blob.size - 8 - n;
      const char *p = fText;
      Space(p);
      Take(p, '{');
      Space(p);
      if (p < fEnd && *p == '}')
         return;
      for (;;) {
         Space(p);
         const std::string name = String(p);
         Space(p);
         Take(p, ':');
         Space(p);
         if (name == "__metadata__") {
            SkipValue(p);
         } else {
            if (fEntries.count(name))
               throw std::runtime_error("SOFIE safetensors: tensor " + name + " appears twice");
            fEntries[name] = Entry(p, name);
         }
         Space(p);
         if (p < fEnd && *p == ',') {
            ++p;
            continue;
         }
         Take(p, '}');
         break;
      }
   }
   void Expect(const std::string &name, const char *dtype, std::size_t elemBytes, std::size_t count) const
   {
      auto f = fEntries.find(name);
      if (f == fEntries.end())
         throw std::runtime_error("SOFIE safetensors: tensor " + name + " is missing");
      const Info &e = f->second;
      if (e.dtype != dtype)
         throw std::runtime_error("SOFIE safetensors: tensor " + name + " has dtype " + e.dtype + ", the model needs " + dtype);
      std::uint64_t len = 1;
      for (auto d : e.shape)
         len *= d;
      if (len != count)
         throw std::runtime_error("SOFIE safetensors: tensor " + name + " has " + std::to_string(len) + " elements, the model needs " +
                                  std::to_string(count));
      if (e.end < e.begin || e.end > fPayloadBytes || e.end - e.begin != count * elemBytes)
         throw std::runtime_error("SOFIE safetensors: tensor " + name + " has data offsets that do not match its size");
   }
   const char *Data(const std::string &name) const { return fPayload + fEntries.at(name).begin; }

private:
   struct Info {
      std::string dtype;
      std::vector<std::uint64_t> shape;
      std::uint64_t begin = 0, end = 0;
   };
   [[noreturn]] void Bad(const std::string &what) const { throw std::runtime_error("SOFIE safetensors: malformed header: " + what); }
   void Space(const char *&p) const
   {
      while (p < fEnd && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r'))
         ++p;
   }
   void Take(const char *&p, char c) const
   {
      if (p >= fEnd || *p != c)
         Bad(std::string("expected '") + c + "'");
      ++p;
   }
   std::string String(const char *&p) const
   {
      Take(p, '"');
      std::string s;
      while (p < fEnd && *p != '"') {
         if (*p == '\\') {
            if (++p >= fEnd)
               Bad("unterminated string");
            if (*p == 'u') { // \uXXXX: tensor names of this backend are ASCII; keep the escape verbatim
               s += "\\u";
               ++p;
               continue;
            }
            s.push_back(*p == 'n' ? '\n' : *p == 't' ? '\t' : *p);
            ++p;
            continue;
         }
         s.push_back(*p++);
      }
      Take(p, '"');
      return s;
   }
   std::uint64_t Number(const char *&p) const
   {
      if (p >= fEnd || *p < '0' || *p > '9')
         Bad("expected a non-negative integer");
      std::uint64_t v = 0;
      while (p < fEnd && *p >= '0' && *p <= '9') {
         if (v > (~std::uint64_t(0) - 9) / 10)
            Bad("number too large");
         v = v * 10 + static_cast<std::uint64_t>(*p++ - '0');
      }
      return v;
   }
   std::vector<std::uint64_t> Numbers(const char *&p) const
   {
      std::vector<std::uint64_t> v;
      Take(p, '[');
      Space(p);
      if (p < fEnd && *p == ']') {
         ++p;
         return v;
      }
      for (;;) {
         Space(p);
         v.push_back(Number(p));
         Space(p);
         if (p < fEnd && *p == ',') {
            ++p;
            continue;
         }
         Take(p, ']');
         return v;
      }
   }
   void SkipValue(const char *&p) const
   {
      Space(p);
      if (p >= fEnd)
         Bad("unexpected end");
      if (*p == '"') {
         String(p);
      } else if (*p == '{' || *p == '[') {
         const char close = *p == '{' ? '}' : ']';
         ++p;
         Space(p);
         if (p < fEnd && *p == close) {
            ++p;
            return;
         }
         for (;;) {
            Space(p);
            if (close == '}') {
               String(p);
               Space(p);
               Take(p, ':');
            }
            SkipValue(p);
            Space(p);
            if (p < fEnd && *p == ',') {
               ++p;
               continue;
            }
            Take(p, close);
            return;
         }
      } else {
         while (p < fEnd && *p != ',' && *p != '}' && *p != ']')
            ++p;
      }
   }
   Info Entry(const char *&p, const std::string &name) const
   {
      Info e;
      bool haveType = false, haveShape = false, haveOffsets = false;
      Take(p, '{');
      for (;;) {
         Space(p);
         const std::string key = String(p);
         Space(p);
         Take(p, ':');
         Space(p);
         if (key == "dtype") {
            e.dtype = String(p);
            haveType = true;
         } else if (key == "shape") {
            e.shape = Numbers(p);
            haveShape = true;
         } else if (key == "data_offsets") {
            auto o = Numbers(p);
            if (o.size() != 2)
               Bad("data_offsets of " + name + " must have two entries");
            e.begin = o[0];
            e.end = o[1];
            haveOffsets = true;
         } else {
            SkipValue(p);
         }
         Space(p);
         if (p < fEnd && *p == ',') {
            ++p;
            continue;
         }
         Take(p, '}');
         break;
      }
      if (!haveType || !haveShape || !haveOffsets)
         Bad("tensor " + name + " lacks dtype, shape or data_offsets");
      return e;
   }
   const char *fText = nullptr, *fEnd = nullptr, *fPayload = nullptr;
   std::size_t fPayloadBytes = 0;
   std::map<std::string, Info> fEntries;
};
} // namespace detail
)SOFIE";

static std::string SafetensorsDType(ETensorType t)
{
   switch (t) {
   case ETensorType::FLOAT: return "F32";
   case ETensorType::DOUBLE: return "F64";
   case ETensorType::INT64: return "I64";
   case ETensorType::INT32: return "I32";
   case ETensorType::INT8: return "I8";
   case ETensorType::UINT8: return "U8";
   case ETensorType::BOOL: return "BOOL";
   case ETensorType::FLOAT8E4M3FN: return "F8_E4M3";
   default: throw std::runtime_error("sofie tensor with type " + ConvertTypeToString(t) + " cannot be written to a safetensors file");
   }
}

void RModel::GenerateSessionCode(std::underlying_type_t<Options> options)
{
   const bool externalStream = options & static_cast<std::underlying_type_t<Options>>(Options::kExternalStream);
   const bool noWeightFile = options & static_cast<std::underlying_type_t<Options>>(Options::kNoWeightFile);
   const bool customMemory = options & static_cast<std::underlying_type_t<Options>>(Options::kCustomMemory);
   const bool safetensors = !noWeightFile && (options & static_cast<std::underlying_type_t<Options>>(Options::kSafetensorsWeightFile));
   const bool strided = fStridedInput;
   fSafetensors = safetensors;
   std::stringstream gc;
   std::string guard = "SOFIE_" + fName;
   std::transform(guard.begin(), guard.end(), guard.begin(), [](unsigned char c) { return std::toupper(c); });
   gc << "//Code generated automatically by SOFIE (gfx950 HIP backend)\n";
   gc << "#ifndef " << guard << "_GPU_HIP\n#define " << guard << "_GPU_HIP\n\n";
   gc << "#include <algorithm>\n#include <array>\n#include <cstddef>\n#include <cstdint>\n#include <cstdlib>\n#include <fstream>\n#include <stdexcept>\n#include <string>\n#include <string_view>\n"
         "#include <tuple>\n#include <type_traits>\n#include <vector>\n#if __cplusplus >= 202002L\n#include <span>\n#endif\n#include \"sofie_hip.h\"\n";
   if (customMemory)
      gc << "#include <functional>\n";
   if (safetensors)
      gc << "#include <iterator>\n#include <map>\n";
   gc << "\n";
   gc << "namespace SOFIE_" << fName << " {\n" << kRuntimeHelpers << "\n";
   if (safetensors)
      gc << kSafetensorsHelpers << "\n";
   if (customMemory) {
      // the reference's contract for caller-owned device memory (core/src/utils/SOFIE_common_helpers.cxx:741-804):
      // alloc is called once for the whole block, assign (optional) maps an offset of the plan to an address, dealloc
      // gets the block back when the Session ends
      gc << "struct MemoryProvider {\n   std::function<void *(std::size_t)> alloc;\n   std::function<void *(std::size_t)> assign;\n"
            "   std::function<void(void *)> dealloc;\n};\n\n";
   }
   // views of device memory owned by the caller (the reference's ViewF1D / ViewConstF1D, README.md:283-297)
   gc << "template <class T>\nstruct DeviceView {\n   T *data = nullptr;\n   std::size_t size = 0; // elements\n};\n"
         "using ViewF1D = DeviceView<float>;\nusing ViewConstF1D = DeviceView<float const>;\n\n";
   gc << "struct Session {\n";
   gc << "   // one arena: weights, operator-owned buffers, inputs, outputs, then the pool of intermediates\n";
   const bool dyn = HasDynamicBatch();
   // name of the batch parameter in the emitted signatures (the reference uses the parameter's own name)
   std::string bp = fBatchParam;
   for (const char *reserved : {"filename", "stream", "device", "provider", "weights_blob", "base", "place", "f", "host", "init"})
      if (bp == reserved)
         bp += "_batch";
   const std::string arenaBytes = dyn ? "ArenaBytes(fMaxBatch)" : "kArenaBytes";
   const std::string arenaTotal = strided ? arenaBytes + " + sofie_strided_bytes" : arenaBytes;
   if (dyn) {
      gc << "   // the batch is a run-time parameter: what carries it is planned per batch entry and scaled by the capacity,\n";
      gc << "   // the constructor's maximum rounded up to a multiple of 16 (every region stays 256-byte aligned)\n";
      gc << "   static constexpr std::size_t kStaticBytes = " << fStaticBytes << ";\n";
      gc << "   static constexpr std::size_t kBytesPerBatchEntry = " << fBatchEntryBytes << ";\n";
      gc << "   static constexpr std::size_t kIntermediatePoolBytesPerBatchEntry = " << fPoolBytes << ";\n";
      gc << "   static std::size_t Capacity(std::size_t maxBatch) { return ((maxBatch ? maxBatch : 1) + 15) / 16 * 16; }\n";
      gc << "   static std::size_t ArenaBytes(std::size_t maxBatch) { return kStaticBytes + Capacity(maxBatch) * kBytesPerBatchEntry; }\n";
      gc << "   std::size_t fMaxBatch = 0, fCapacity = 0;\n";
   } else {
      gc << "   static constexpr std::size_t kArenaBytes = " << fArenaBytes << ";\n";
      gc << "   static constexpr std::size_t kIntermediatePoolBytes = " << fPoolBytes << ";\n";
   }
   gc << "   sofie_hip_ctx *fCtx = nullptr;\n";
   // Options::kStridedInput: the strides (in elements) of the graph inputs as the constructor received them, one member per
   // input (empty = contiguous), as in the reference's Sessions (core/src/RModel.cxx:1272-1300, 1517-1520)
   auto extentOf = [&](const std::string &n, const std::string &batch) {
      return strided ? "InputExtent_" + n + "(" + (IsDynamicTensor(n) ? batch : std::string()) + ")"
                     : (IsDynamicTensor(n) ? batch + " * " : std::string()) + std::to_string(ConvertShapeToLength(GetTensorShape(n)));
   };
   if (strided) {
      for (auto &n : fInputTensorNames)
         gc << "   std::vector<std::size_t> " << InputStrideMemberName(n) << ";\n";
      gc << "   // elements a graph input spans in memory: from its first to its last element through the strides, or its length\n";
      for (auto &n : fInputTensorNames) {
         const auto &shape = GetTensorShape(n);
         const bool dynIn = IsDynamicTensor(n);
         gc << "   std::size_t InputExtent_" << n << "(" << (dynIn ? "std::size_t sofie_rows" : "") << ") const\n   {\n";
         gc << "      const std::size_t shape[" << std::max<std::size_t>(shape.size(), 1) << "] = {";
         for (std::size_t d = 0; d < shape.size(); ++d)
            gc << (d ? ", " : "") << (d == 0 && dynIn ? std::string("sofie_rows") : std::to_string(shape[d]));
         if (shape.empty())
            gc << "1";
         gc << "};\n";
         gc << "      std::size_t length = 1, last = 0;\n";
         gc << "      for (std::size_t d = 0; d < " << shape.size() << "; ++d) {\n         length *= shape[d];\n";
         gc << "         if (!" << InputStrideMemberName(n) << ".empty() && shape[d])\n            last += (shape[d] - 1) * " << InputStrideMemberName(n) << "[d];\n      }\n";
         gc << "      return " << InputStrideMemberName(n) << ".empty() || length == 0 ? length : last + 1;\n   }\n";
      }
   }
   if (customMemory)
      gc << "   MemoryProvider fProvider;\n   void *fBlock = nullptr;\n";
   auto typeOf = [&](const std::string &planName) -> std::string {
      if (planName.rfind("tensor_", 0) == 0)
         return ConvertTypeToString(GetTensorType(planName.substr(7)));
      return "int8_t";
   };
   auto offsetText = [&](const PlannedTensor &p) {
      return p.perBatch ? "kStaticBytes + fCapacity * " + std::to_string(p.offset) : std::to_string(p.offset);
   };
   for (auto &p : fPlan)
      gc << "   " << typeOf(p.name) << " *" << p.name << " = nullptr; // " << (p.perBatch ? "per batch entry: offset " : "arena offset ") << p.offset
         << ", " << p.bytes << " bytes" << (p.pooled ? ", live [" + std::to_string(p.begin) + "," + std::to_string(p.end) + ")" : "") << (p.view ? ", a view" : "") << "\n";
   gc << "\n";
   // constructor
   // (Options::kStridedInput adds the strides of the inputs behind the shape parameter, as the reference does:
   // core/src/RModel.cxx:1546-1549)
   const std::string stridesDecl = strided ? ", std::vector<std::vector<std::size_t>> inputStrides = {}" : "";
   const std::string stridesArg = strided ? ", inputStrides" : "";
   if (safetensors) {
      // the file is read whole and handed to the constructor that takes the payload
      gc << "   Session(" << (customMemory ? "MemoryProvider provider, " : "") << "std::string filename = \"" << fName << "_GPU_HIP.safetensors\""
         << (dyn ? ", std::size_t " + bp + " = " + std::to_string(fBatchDefault) : std::string()) << stridesDecl << (externalStream ? ", void *stream = nullptr" : "") << ", int device = 0)\n";
      gc << "      : Session(" << (customMemory ? "std::move(provider), " : "") << "SafetensorsBlob(detail::LoadWeightsFromFile(filename))"
         << (dyn ? ", " + bp : std::string()) << stridesArg << (externalStream ? ", stream" : "") << ", device)\n   {\n   }\n";
      gc << "   Session(" << (customMemory ? "MemoryProvider provider, " : "") << "SafetensorsBlob weights_blob"
         << (dyn ? ", std::size_t " + bp + " = " + std::to_string(fBatchDefault) : std::string()) << stridesDecl << (externalStream ? ", void *stream = nullptr" : "") << ", int device = 0)\n";
   } else {
      gc << "   Session(" << (customMemory ? "MemoryProvider provider, " : "") << "std::string filename = \""
         << (noWeightFile ? "" : fName + "_GPU_HIP.dat") << "\"" << (dyn ? ", std::size_t " + bp + " = " + std::to_string(fBatchDefault) : std::string()) << stridesDecl
         << (externalStream ? ", void *stream = nullptr" : "") << ", int device = 0)\n";
   }
   if (customMemory)
      gc << "      : fProvider(std::move(provider))\n";
   gc << "   {\n";
   if (dyn)
      gc << "      fMaxBatch = " << bp << ";\n      fCapacity = Capacity(" << bp << ");\n";
   if (strided) {
      // the checks and messages of the reference (core/src/RModel.cxx:1272-1300)
      gc << "      if (!inputStrides.empty()) {\n";
      gc << "         if (inputStrides.size() != " << fInputTensorNames.size() << ")\n";
      gc << "            throw std::runtime_error(\"sofie: expected " << fInputTensorNames.size() << " input stride array(s), one per input tensor\");\n";
      for (std::size_t i = 0; i < fInputTensorNames.size(); ++i) {
         const auto &n = fInputTensorNames[i];
         const std::string member = InputStrideMemberName(n);
         gc << "         " << member << " = inputStrides[" << i << "];\n";
         gc << "         if (!" << member << ".empty() && " << member << ".size() != " << GetTensorShape(n).size() << ")\n";
         gc << "            throw std::runtime_error(\"sofie: the stride array of input tensor " << n << " must have " << GetTensorShape(n).size()
            << " element(s)\");\n";
      }
      gc << "      }\n";
      gc << "      // an input given with strides does not fit its planned region: it gets one behind the planned arena, sized by its extent\n";
      gc << "      std::size_t sofie_strided_bytes = 0;\n";
      for (auto &n : fInputTensorNames) {
         gc << "      const std::size_t sofie_strided_offset_" << n << " = sofie_strided_bytes;\n";
         gc << "      if (!" << InputStrideMemberName(n) << ".empty())\n         sofie_strided_bytes += (" << extentOf(n, "fMaxBatch") << " * sizeof("
            << ConvertTypeToString(fInputTensorInfos[n].type) << ") + 255) / 256 * 256;\n";
      }
   }
   if (safetensors) {
      // the payload is checked against the model before any device work
      gc << "      detail::SafetensorsReader sofie_weights_reader(weights_blob);\n";
      for (auto &kv : fInitializedTensors)
         if (!kv.second.constant)
            gc << "      sofie_weights_reader.Expect(\"tensor_" << kv.first << "\", \"" << SafetensorsDType(kv.second.type) << "\", "
               << GetTypeSize(kv.second.type) << ", " << ConvertShapeToLength(kv.second.shape) << ");\n";
   }
   if (customMemory)
      gc << "      if (!fProvider.alloc)\n         throw std::runtime_error(\"SOFIE HIP Session: the memory provider has no alloc function\");\n";
   gc << "      if (sofie_hip_abi_version() != SOFIE_HIP_ABI_VERSION)\n"
      << "         throw std::runtime_error(\"SOFIE HIP: this Session was generated for version \" + std::to_string(SOFIE_HIP_ABI_VERSION) +\n"
      << "                                  \" of the runtime library's interface, the library loaded has version \" + std::to_string(sofie_hip_abi_version()));\n";
   gc << "      detail::Check(sofie_hip_ctx_create(&fCtx, device, " << (externalStream ? "stream" : "nullptr") << "), \"Session\");\n";
   gc << "      try {\n";
   if (customMemory) {
      gc << "         fBlock = fProvider.alloc(" << arenaTotal << ");\n";
      gc << "         if (!fBlock)\n            throw std::runtime_error(\"SOFIE HIP Session: the memory provider returned no block\");\n";
      gc << "         detail::Check(sofie_hip_arena_adopt(fCtx, fBlock, " << arenaTotal << "), \"adoption of the caller's block\");\n";
      gc << "         auto place = [&](std::size_t offset) -> char * {\n"
            "            void *p = fProvider.assign ? fProvider.assign(offset) : static_cast<char *>(fBlock) + offset;\n"
            "            if (!p)\n               throw std::runtime_error(\"SOFIE HIP Session: the memory provider assigned no address\");\n"
            "            return static_cast<char *>(p);\n         };\n";
      for (auto &p : fPlan)
         gc << "         " << p.name << " = reinterpret_cast<" << typeOf(p.name) << " *>(place(" << offsetText(p) << "));\n";
      if (strided)
         for (auto &n : fInputTensorNames)
            gc << "         if (!" << InputStrideMemberName(n) << ".empty())\n            tensor_" << n << " = reinterpret_cast<" << ConvertTypeToString(fInputTensorInfos[n].type)
               << " *>(place(" << arenaBytes << " + sofie_strided_offset_" << n << "));\n";
   } else {
      gc << "         detail::Check(sofie_hip_arena_create(fCtx, " << arenaTotal << ", " << kPoolAlignBytes << "), \"arena allocation\");\n";
      gc << "         char *base = static_cast<char *>(sofie_hip_arena_ptr(fCtx, 0));\n";
      gc << "         if (!base)\n            throw std::runtime_error(\"SOFIE HIP runtime error: arena is null\");\n";
      for (auto &p : fPlan)
         gc << "         " << p.name << " = reinterpret_cast<" << typeOf(p.name) << " *>(base + " << offsetText(p) << ");\n";
      if (strided)
         for (auto &n : fInputTensorNames)
            gc << "         if (!" << InputStrideMemberName(n) << ".empty())\n            tensor_" << n << " = reinterpret_cast<" << ConvertTypeToString(fInputTensorInfos[n].type)
               << " *>(base + " << arenaBytes << " + sofie_strided_offset_" << n << ");\n";
   }
   bool anyWeights = false, anyConstants = false;
   for (auto &kv : fInitializedTensors)
      (kv.second.constant ? anyConstants : anyWeights) = true;
   if (anyWeights && safetensors) {
      gc << "         // upload the weights straight from the payload\n";
      for (auto &kv : fInitializedTensors) {
         if (kv.second.constant)
            continue;
         const std::size_t bytes = ConvertShapeToLength(kv.second.shape) * GetTypeSize(kv.second.type);
         if (bytes)
            gc << "         detail::Check(sofie_hip_upload(fCtx, tensor_" << kv.first << ", sofie_weights_reader.Data(\"tensor_" << kv.first << "\"), "
               << bytes << "), \"upload of tensor_" << kv.first << "\");\n";
      }
      gc << "         detail::Check(sofie_hip_sync(fCtx), \"upload of the weights\");\n";
   } else if (anyWeights && !noWeightFile) {
      gc << "         // read and upload the weights\n";
      gc << "         std::ifstream f;\n         f.open(filename);\n";
      gc << "         if (!f.is_open()) {\n            throw std::runtime_error(\"tmva-sofie failed to open file \" + filename + \" for input weights\");\n         }\n";
      for (auto &kv : fInitializedTensors) {
         if (kv.second.constant)
            continue;
         const std::size_t len = ConvertShapeToLength(kv.second.shape);
         gc << "         {\n            std::vector<" << ConvertTypeToString(kv.second.type) << "> host;\n";
         gc << "            detail::ReadTensorFromStream(f, host, \"tensor_" << kv.first << "\", " << len << ");\n";
         gc << "            detail::Check(sofie_hip_upload(fCtx, tensor_" << kv.first << ", host.data(), " << len * GetTypeSize(kv.second.type)
            << "), \"upload of tensor_" << kv.first << "\");\n";
         gc << "            detail::Check(sofie_hip_sync(fCtx), \"upload of tensor_" << kv.first << "\");\n         }\n";
      }
      gc << "         f.close();\n";
   }
   if (anyConstants || noWeightFile) {
      for (auto &kv : fInitializedTensors) {
         if (!kv.second.constant && !noWeightFile)
            continue;
         const std::size_t len = ConvertShapeToLength(kv.second.shape);
         gc << "         {\n            static const " << ConvertTypeToString(kv.second.type) << " host[" << (len ? len : 1) << "] = {";
         for (std::size_t i = 0; i < len; ++i) {
            if (kv.second.type == ETensorType::FLOAT)
               gc << FloatLiteral(static_cast<const float *>(kv.second.data.get())[i]);
            else if (kv.second.type == ETensorType::INT8)
               gc << (int)static_cast<const int8_t *>(kv.second.data.get())[i];
            else if (kv.second.type == ETensorType::INT32)
               gc << static_cast<const int32_t *>(kv.second.data.get())[i];
            else if (kv.second.type == ETensorType::INT64)
               gc << static_cast<const int64_t *>(kv.second.data.get())[i];
            else
               gc << (unsigned)static_cast<const uint8_t *>(kv.second.data.get())[i];
            gc << (i + 1 < len ? ", " : "");
         }
         gc << "};\n";
         gc << "            detail::Check(sofie_hip_upload(fCtx, tensor_" << kv.first << ", host, " << len * GetTypeSize(kv.second.type)
            << "), \"upload of tensor_" << kv.first << "\");\n";
         gc << "            detail::Check(sofie_hip_sync(fCtx), \"upload of tensor_" << kv.first << "\");\n         }\n";
      }
   }
   std::string init;
   for (auto &op : fOperators)
      init += op->GenerateInitCode_GPU_HIP();
   if (!init.empty())
      gc << "         // one-time operator set-up (weight re-layouts)\n" << init;
   gc << "         detail::Check(sofie_hip_sync(fCtx), \"Session\");\n";
   if (customMemory) {
      gc << "      } catch (...) {\n         sofie_hip_ctx_destroy(fCtx);\n         fCtx = nullptr;\n"
            "         if (fBlock && fProvider.dealloc)\n            fProvider.dealloc(fBlock);\n         throw;\n      }\n   }\n";
      gc << "   ~Session()\n   {\n      sofie_hip_ctx_destroy(fCtx); // waits for the stream; an adopted block is not freed by the runtime\n"
            "      if (fBlock && fProvider.dealloc)\n         fProvider.dealloc(fBlock);\n   }\n";
   } else {
      gc << "      } catch (...) {\n         sofie_hip_ctx_destroy(fCtx);\n         fCtx = nullptr;\n         throw;\n      }\n   }\n";
      gc << "   ~Session() { sofie_hip_ctx_destroy(fCtx); }\n";
   }
   gc << "   Session(const Session &) = delete;\n   Session &operator=(const Session &) = delete;\n\n";
   gc << "   std::size_t GetIntermediateMemoryPoolSize() const { return "
      << (dyn ? "fCapacity * kIntermediatePoolBytesPerBatchEntry" : "kIntermediatePoolBytes") << "; }\n";
   if (dyn)
      gc << "   std::size_t GetMaxBatch() const { return fMaxBatch; }\n";
   // statistics of the pool of intermediate tensors, as the reference's GPU sessions report them (core/src/RModel_ALPAKA.cxx:1262-1269)
   {
      const std::string scale = dyn ? "fCapacity * " : "";
      gc << "   std::size_t GetTotalFreeMemory() const { return " << scale << fPoolFreeBytes << "; }\n";
      gc << "   std::size_t GetLargestFreeBlock() const { return " << scale << fPoolLargestFreeBlock << "; }\n";
      gc << "   double GetFragmentation() const { return " << (fPoolFreeBytes == 0 ? std::string("0.0") : "1.0 - " + std::to_string(fPoolLargestFreeBlock) + ".0 / " + std::to_string(fPoolFreeBytes) + ".0")
         << "; }\n";
      // zero the intermediate tensors (the reference's resetState, core/src/RModel_ALPAKA.cxx:1543-1568) and the weights
      // (SetWeightsToZero, core/src/RModel.cxx:1632-1643)
      gc << "   void resetState()\n   {\n";
      const std::string base = dyn ? "static_cast<char *>(sofie_hip_arena_ptr(fCtx, 0)) + kStaticBytes + fCapacity * " + std::to_string(fPoolBase)
                                   : "static_cast<char *>(sofie_hip_arena_ptr(fCtx, 0)) + " + std::to_string(fPoolBase);
      if (fPoolBytes && !customMemory)
         gc << "      detail::Check(sofie_hip_fill_zero(fCtx, " << base << ", " << scale << fPoolBytes << "), \"resetState\");\n";
      else
         for (auto &p : fPlan)
            if (p.pooled)
               gc << "      detail::Check(sofie_hip_fill_zero(fCtx, " << p.name << ", " << (p.perBatch ? scale : "") << p.bytes << "), \"resetState\");\n";
      gc << "      detail::Check(sofie_hip_sync(fCtx), \"resetState\");\n   }\n";
      gc << "   void SetWeightsToZero()\n   {\n";
      for (auto &kv : fInitializedTensors)
         if (!kv.second.constant && kv.second.type == ETensorType::FLOAT && ConvertShapeToLength(kv.second.shape))
            gc << "      detail::Check(sofie_hip_fill_zero(fCtx, tensor_" << kv.first << ", " << ConvertShapeToLength(kv.second.shape) * 4
               << "), \"SetWeightsToZero\");\n";
      gc << "      detail::Check(sofie_hip_sync(fCtx), \"SetWeightsToZero\");\n   }\n";
   }
   // device-resident use: where to write the inputs and read the outputs around infer_nosync()
   for (auto &n : fInputTensorNames)
      gc << "   " << ConvertTypeToString(fInputTensorInfos[n].type) << " *device_input_" << n << "() const { return tensor_" << n << "; }\n";
   for (auto &n : fOutputTensorNames)
      gc << "   " << ConvertTypeToString(GetTensorType(n)) << " const *device_output_" << n << "() const { return tensor_" << n << "; }\n";
   gc << "   void *stream() const { return sofie_hip_stream(fCtx); }\n";
   gc << "   // the runtime context of the Session (its stream, arena and event timer), as the reference's GPU Session leaves its queue public\n";
   gc << "   sofie_hip_ctx *context() const { return fCtx; }\n";
   gc << "   // waits for everything enqueued on the session's stream (what follows a run of infer_nosync calls)\n";
   gc << "   void sync() { detail::Check(sofie_hip_sync(fCtx), \"sync\"); }\n\n";

   // doInfer: the operators.  The graph inputs and outputs are parameters named like the members they shadow, so that the
   // same statements run on the arena's regions (infer_nosync) or on memory of the caller (the overload that takes views).
   std::vector<std::string> boundOutputs; // graph outputs an operator writes (an output that is an input or a weight is not)
   for (auto &o : fOutputTensorNames)
      if (fIntermediateTensorInfos.count(o) && std::find(boundOutputs.begin(), boundOutputs.end(), o) == boundOutputs.end())
         boundOutputs.push_back(o);
   gc << "   // the operators of the model; the graph inputs and outputs are passed in (these parameters shadow the members)\n";
   gc << "   void doInfer(" << (dyn ? "std::int64_t sofie_batch" : "");
   {
      bool first = !dyn;
      for (auto &n : fInputTensorNames) {
         gc << (first ? "" : ", ") << ConvertTypeToString(fInputTensorInfos[n].type) << " const *tensor_" << n;
         first = false;
      }
      for (auto &o : boundOutputs) {
         gc << (first ? "" : ", ") << ConvertTypeToString(GetTensorType(o)) << " *tensor_" << o;
         first = false;
      }
   }
   gc << ")\n   {";
   if (dyn)
      gc << "\n      (void)sofie_batch;";
   const auto chains = GemmChains(); // the runs the memory plan was made for
   for (std::size_t i = 0; i < fOperators.size(); ++i) {
      // Consecutive products of which each reads what the one before wrote (the layers of an MLP) go to the runtime as one
      // call: at small batch it runs them in a single launch, otherwise layer by layer -- the results are the same.
      std::vector<ROperator_Gemm<float> *> chain;
      for (auto &ch : chains)
         if (ch.first == i)
            for (std::size_t j = i; j < i + ch.second; ++j)
               chain.push_back(static_cast<ROperator_Gemm<float> *>(fOperators[j].get()));
      if (chain.size() < 2) {
         gc << fOperators[i]->Generate_GPU_HIP(std::to_string(i));
         continue;
      }
      const std::string last = std::to_string(i + chain.size() - 1);
      const std::string SP = "      "; // the operators' indentation inside doInfer
      gc << "\n" << SP << "//--------- Gemm chain op_" << i << " .. op_" << last << "\n";
      gc << SP << "{\n";
      gc << SP << "   " << "sofie_gemm_f32_desc chain[" << chain.size() << "]{};\n";
      for (std::size_t l = 0; l < chain.size(); ++l) {
         gc << SP << "   " << "// op_" << (i + l) << " " << chain[l]->Title() << "\n";
         gc << chain[l]->DescriptorStatements("chain[" + std::to_string(l) + "]", "post_" + std::to_string(l));
      }
      gc << SP << "   " << "detail::Check(sofie_hip_gemm_chain_f32(fCtx, chain, " << chain.size() << "), \"op_" << i << " .. op_" << last << " Gemm chain\");\n";
      gc << SP << "}\n";
      i += chain.size() - 1;
   }
   gc << "   }\n\n";
   auto boundArgs = [&](const std::string &inPrefix, const std::string &outPrefix) {
      std::string a = dyn ? "static_cast<std::int64_t>(" + bp + ")" : "";
      for (auto &n : fInputTensorNames)
         a += std::string(a.empty() ? "" : ", ") + inPrefix + n;
      for (auto &o : boundOutputs)
         a += std::string(a.empty() ? "" : ", ") + outPrefix + o;
      return a;
   };
   const std::string batchCheck = !dyn ? std::string()
                                       : "      if (" + bp + " > fMaxBatch) {\n         throw std::runtime_error(\"sofie: dynamic input tensor shape parameter " +
                                            fBatchParam + " exceeds the initialized maximum allowed shape.\");\n      }\n";
   // infer_nosync: inputs and outputs resident in the arena
   gc << "   // enqueues one inference on the session's stream: inputs are read from the tensor_<input> regions of the arena,\n";
   gc << "   // results land in the tensor_<output> regions (overwritten by the next call)\n";
   if (dyn) {
      gc << "   // " << bp << ": the batch of this call, at most the constructor's maximum\n";
      gc << "   void infer_nosync(std::size_t " << bp << ")\n   {\n" << batchCheck;
      gc << "      if (" << bp << " == 0)\n         return;\n";
   } else
      gc << "   void infer_nosync()\n   {\n";
   gc << "      doInfer(" << boundArgs("tensor_", "tensor_") << ");\n   }\n\n";

   // infer on views of device memory: the third signature of the reference's GPU sessions
   // (infer(std::span<ViewConstF1D const> inputs, std::span<ViewF1D> outputs, params...))
   bool allFloat = true;
   for (auto &n : fInputTensorNames)
      allFloat = allFloat && fInputTensorInfos[n].type == ETensorType::FLOAT;
   for (auto &o : fOutputTensorNames)
      allFloat = allFloat && GetTensorType(o) == ETensorType::FLOAT;
   if (allFloat) {
      gc << "#if __cplusplus >= 202002L\n";
      gc << "   // Runs the model on device memory of the caller and waits.  inputs[i] / outputs[i] follow the order of the model's\n";
      gc << "   // inputs / outputs.  Views that start on a 256-byte boundary are read and written in place (no copy); any other\n";
      gc << "   // view goes through the session's own region with one device-to-device copy.\n";
      gc << "   void infer(std::span<ViewConstF1D const> inputs, std::span<ViewF1D> outputs" << (dyn ? ", std::size_t " + bp : "") << ")\n   {\n";
      gc << batchCheck;
      gc << "      if (inputs.size() != " << fInputTensorNames.size() << " || outputs.size() != " << fOutputTensorNames.size()
         << ")\n         throw std::runtime_error(\"SOFIE HIP Session: infer takes " << fInputTensorNames.size() << " input and "
         << fOutputTensorNames.size() << " output views\");\n";
      auto lenOf = [&](const std::string &n) {
         return (IsDynamicTensor(n) ? bp + " * " : std::string()) + std::to_string(ConvertShapeToLength(GetTensorShape(n)));
      };
      for (std::size_t i = 0; i < fInputTensorNames.size(); ++i)
         gc << "      if (inputs[" << i << "].size < " << extentOf(fInputTensorNames[i], bp) << " || !inputs[" << i << "].data)\n"
            << "         throw std::runtime_error(\"SOFIE HIP Session: the view of input " << fInputTensorNames[i] << " is too small\");\n";
      for (std::size_t i = 0; i < fOutputTensorNames.size(); ++i)
         gc << "      if (outputs[" << i << "].size < " << lenOf(fOutputTensorNames[i]) << " || !outputs[" << i << "].data)\n"
            << "         throw std::runtime_error(\"SOFIE HIP Session: the view of output " << fOutputTensorNames[i] << " is too small\");\n";
      if (dyn)
         gc << "      if (" << bp << " == 0)\n         return;\n";
      gc << "      auto inPlace = [](const void *p) { return (reinterpret_cast<std::uintptr_t>(p) & 255) == 0; };\n";
      for (std::size_t i = 0; i < fInputTensorNames.size(); ++i) {
         const auto &n = fInputTensorNames[i];
         gc << "      float const *in_" << n << " = inputs[" << i << "].data;\n";
         gc << "      if (!inPlace(in_" << n << ")) {\n         detail::Check(sofie_hip_copy(fCtx, tensor_" << n << ", in_" << n << ", (" << extentOf(n, bp)
            << ") * sizeof(float)), \"copy of input " << n << "\");\n         in_" << n << " = tensor_" << n << ";\n      }\n";
      }
      for (std::size_t i = 0; i < fOutputTensorNames.size(); ++i) {
         const auto &o = fOutputTensorNames[i];
         if (std::find(boundOutputs.begin(), boundOutputs.end(), o) == boundOutputs.end())
            continue;
         // the first view of an output is the one the operators write
         bool firstUse = std::find(fOutputTensorNames.begin(), fOutputTensorNames.begin() + i, o) == fOutputTensorNames.begin() + i;
         if (firstUse)
            gc << "      float *out_" << o << " = inPlace(outputs[" << i << "].data) ? outputs[" << i << "].data : tensor_" << o << ";\n";
      }
      gc << "      doInfer(" << boundArgs("in_", "out_") << ");\n";
      for (std::size_t i = 0; i < fOutputTensorNames.size(); ++i) {
         const auto &o = fOutputTensorNames[i];
         const bool bound = std::find(boundOutputs.begin(), boundOutputs.end(), o) != boundOutputs.end();
         const std::string src = bound ? "out_" + o : "tensor_" + o;
         gc << "      if (outputs[" << i << "].data != " << src << ")\n         detail::Check(sofie_hip_copy(fCtx, outputs[" << i << "].data, " << src
            << ", (" << lenOf(o) << ") * sizeof(float)), \"copy of output " << o << "\");\n";
      }
      gc << "      detail::Check(sofie_hip_sync(fCtx), \"infer\");\n   }\n";
      gc << "#endif\n\n";
   }

   // infer with host pointers: the CPU signature of the reference
   std::string args = dyn ? "std::size_t " + bp + (fInputTensorNames.empty() ? "" : ", ") : "";
   for (std::size_t i = 0; i < fInputTensorNames.size(); ++i) {
      const auto &ti = fInputTensorInfos[fInputTensorNames[i]];
      args += ConvertTypeToString(ti.type) + " const* host_" + fInputTensorNames[i] + (i + 1 < fInputTensorNames.size() ? ", " : "");
   }
   bool sameType = true;
   for (auto &o : fOutputTensorNames)
      sameType = sameType && GetTensorType(o) == GetTensorType(fOutputTensorNames[0]);
   std::string retType;
   const std::string t0 = ConvertTypeToString(GetTensorType(fOutputTensorNames.at(0)));
   if (fOutputTensorNames.size() == 1)
      retType = "std::vector<" + t0 + ">";
   else if (sameType)
      retType = "std::vector<std::vector<" + t0 + ">>";
   else {
      retType = "std::tuple<";
      for (std::size_t i = 0; i < fOutputTensorNames.size(); ++i)
         retType += "std::vector<" + ConvertTypeToString(GetTensorType(fOutputTensorNames[i])) + ">" + (i + 1 < fOutputTensorNames.size() ? ", " : "");
      retType += ">";
   }
   gc << "   " << retType << " infer(" << args << ")\n   {\n";
   if (dyn)
      gc << "      if (" << bp << " > fMaxBatch) {\n         throw std::runtime_error(\"sofie: dynamic input tensor shape parameter " << fBatchParam
         << " exceeds the initialized maximum allowed shape.\");\n      }\n";
   for (auto &n : fInputTensorNames) {
      const auto &ti = fInputTensorInfos[n];
      if (strided)
         gc << "      detail::Check(sofie_hip_upload(fCtx, tensor_" << n << ", host_" << n << ", " << extentOf(n, bp) << " * " << GetTypeSize(ti.type)
            << "), \"upload of input " << n << "\");\n";
      else
         gc << "      detail::Check(sofie_hip_upload(fCtx, tensor_" << n << ", host_" << n << ", " << (IsDynamicTensor(n) ? bp + " * " : "")
            << ConvertShapeToLength(ti.shape) * GetTypeSize(ti.type) << "), \"upload of input " << n << "\");\n";
   }
   gc << "      infer_nosync(" << (dyn ? bp : "") << ");\n";
   for (std::size_t i = 0; i < fOutputTensorNames.size(); ++i) {
      const auto &o = fOutputTensorNames[i];
      const std::size_t len = ConvertShapeToLength(GetTensorShape(o));
      const std::string scale = IsDynamicTensor(o) ? bp + " * " : "";
      gc << "      std::vector<" << ConvertTypeToString(GetTensorType(o)) << "> out_" << i << "(" << scale << len << ");\n";
      gc << "      detail::Check(sofie_hip_download(fCtx, out_" << i << ".data(), tensor_" << o << ", " << scale << len * GetTypeSize(GetTensorType(o))
         << "), \"download of output " << o << "\");\n";
   }
   gc << "      detail::Check(sofie_hip_sync(fCtx), \"infer\");\n";
   if (fOutputTensorNames.size() == 1)
      gc << "      return out_0;\n";
   else {
      gc << "      return " << (sameType ? retType : std::string("std::make_tuple")) << (sameType ? "{" : "(");
      for (std::size_t i = 0; i < fOutputTensorNames.size(); ++i)
         gc << "std::move(out_" << i << ")" << (i + 1 < fOutputTensorNames.size() ? ", " : "");
      gc << (sameType ? "};\n" : ");\n");
   }
   gc << "   }\n";
   gc << "}; // end of Session\n\n";
   // the shapes of the graph tensors in the reference's form (core/src/RModel.cxx:2036-2112,
   // core/src/utils/SOFIE_common_helpers.cxx:880-907): a run-time dimension carries its parameter's name
   gc << "struct SingleDim {\n   enum class Kind { Static, Symbolic };\n   Kind kind;\n   std::size_t dim;\n   std::string_view name;\n"
         "   constexpr SingleDim(std::size_t v) : kind(Kind::Static), dim(v), name() {}\n"
         "   constexpr SingleDim(const char *v) : kind(Kind::Symbolic), dim(0), name(v) {}\n};\n"
         "struct TensorDims {\n   const SingleDim *data;\n   std::size_t size;\n   constexpr std::size_t total_size() const\n   {\n"
         "      std::size_t result = 1;\n      for (std::size_t i = 0; i < size; ++i)\n         result *= data[i].dim;\n      return result;\n   }\n};\n"
         "template <class Arr>\nconstexpr TensorDims makeDims(Arr const &arr)\n{\n   return TensorDims{arr.data(), arr.size()};\n}\n\n";
   std::set<std::string> dimsEmitted;
   auto dimsArray = [&](const std::string &what, const std::vector<std::string> &names) {
      gc << "// " << what << " tensor dimensions\n";
      bool anyDynamic = false;
      for (auto &n : names) {
         const auto &s = GetTensorShape(n);
         anyDynamic = anyDynamic || IsDynamicTensor(n);
         if (!dimsEmitted.insert(n).second)
            continue; // a graph output that is also an input, or listed twice
         gc << "constexpr std::array<SingleDim, " << s.size() << "> dim_" << n << "{";
         for (std::size_t i = 0; i < s.size(); ++i) {
            if (i == 0 && IsDynamicTensor(n)) {
               gc << "SingleDim{\"" << fBatchParam << "\"}";
            } else
               gc << "SingleDim{" << s[i] << "}";
            gc << (i + 1 < s.size() ? ", " : "");
         }
         gc << "};\n";
      }
      gc << "constexpr std::array<TensorDims, " << names.size() << "> " << what << "TensorDims{";
      for (std::size_t i = 0; i < names.size(); ++i)
         gc << "makeDims(dim_" << names[i] << ")" << (i + 1 < names.size() ? ", " : "");
      gc << "};\n";
      gc << "constexpr bool hasDynamic" << (what == "input" ? "Input" : "Output") << "Tensors{" << (anyDynamic ? "true" : "false") << "};\n\n";
   };
   dimsArray("input", fInputTensorNames);
   dimsArray("output", fOutputTensorNames);
   gc << "} //SOFIE_" << fName << "\n\n#endif  // " << guard << "_GPU_HIP\n";
   fGC = gc.str();
}

void RModel::GenerateGPU_HIP(std::underlying_type_t<Options> options, int batchSize, bool verbose)
{
   if (fOutputTensorNames.empty())
      throw std::runtime_error("SOFIE: the model has no output tensor");
   fStridedInput = options & static_cast<std::underlying_type_t<Options>>(Options::kStridedInput);
   Initialize(batchSize);
   PlanMemory();
   GenerateSessionCode(options);
   if (verbose)
      std::cout << "SOFIE HIP: " << fOperators.size() << " operators, arena " << fArenaBytes << " bytes, pool " << fPoolBytes << " bytes\n";
}

void RModel::WriteWeightFile(const std::string &filename) const
{
   std::ofstream f(filename);
   if (!f.is_open())
      throw std::runtime_error("tmva-sofie failed to open file " + filename + " for tensor weight data");
   for (auto &kv : fInitializedTensors) {
      if (kv.second.constant)
         continue;
      const std::size_t len = ConvertShapeToLength(kv.second.shape);
      f << "tensor_" << kv.first << " " << len << "\n";
      for (std::size_t i = 0; i < len; ++i) {
         switch (kv.second.type) {
         case ETensorType::FLOAT: {
            float v = static_cast<const float *>(kv.second.data.get())[i];
            if (v != 0. && std::abs(v) < std::numeric_limits<float>::min())
               v = 0; // sub-normal values are rounded to zero, as the reference's writer does
            if (std::isinf(v))
               f << (v > 0 ? "inf" : "-inf");
            else if (std::isnan(v))
               f << "nan";
            else
               f << std::setprecision(std::numeric_limits<float>::max_digits10) << v;
         } break;
         case ETensorType::INT8: f << (int)static_cast<const int8_t *>(kv.second.data.get())[i]; break;
         case ETensorType::UINT8: case ETensorType::BOOL: case ETensorType::FLOAT8E4M3FN:
            f << (unsigned)static_cast<const uint8_t *>(kv.second.data.get())[i];
            break;
         case ETensorType::INT32: f << static_cast<const int32_t *>(kv.second.data.get())[i]; break;
         case ETensorType::INT64: f << static_cast<const int64_t *>(kv.second.data.get())[i]; break;
         default: throw std::runtime_error("sofie tensor tensor_" + kv.first + " with type " + ConvertTypeToString(kv.second.type) + " cannot be written to a file");
         }
         f << (i + 1 < len ? " " : "\n");
      }
      if (len == 0)
         f << "\n";
      if (f.fail())
         throw std::runtime_error("sofie failed to write tensor data to file for  tensor_" + kv.first);
   }
}

void RModel::OutputGenerated(std::string filename)
{
   if (fGC.empty())
      throw std::runtime_error("SOFIE: OutputGenerated called before GenerateGPU_HIP");
   if (filename.empty())
      filename = fName + "_GPU_HIP.hxx";
   std::ofstream f(filename);
   if (!f.is_open())
      throw std::runtime_error("tmva-sofie failed to open file " + filename + " for the generated code");
   f << fGC;
   f.close();
   std::string dat = filename;
   auto dot = dat.find_last_of('.');
   if (dot != std::string::npos)
      dat = dat.substr(0, dot);
   if (fSafetensors)
      WriteSafetensorsFile(dat + ".safetensors");
   else
      WriteWeightFile(dat + ".dat");
}

void RModel::WriteSafetensorsFile(const std::string &filename) const
{
   const std::uint16_t one = 1;
   if (!*reinterpret_cast<const std::uint8_t *>(&one))
      throw std::runtime_error("sofie: safetensors weights can only be written on a little-endian host");
   auto escape = [](const std::string &in) {
      std::string out;
      for (char c : in) {
         if (c == '"' || c == '\\')
            out.push_back('\\');
         out.push_back(c);
      }
      return out;
   };
   std::string header = "{";
   std::uint64_t offset = 0;
   bool first = true;
   for (auto &kv : fInitializedTensors) { // std::map: sorted by name, as the reference's writer sorts them
      if (kv.second.constant)
         continue;
      const std::uint64_t nbytes = ConvertShapeToLength(kv.second.shape) * GetTypeSize(kv.second.type);
      header += std::string(first ? "" : ",") + "\"" + escape("tensor_" + kv.first) + "\":{\"dtype\":\"" + SafetensorsDType(kv.second.type) +
                "\",\"shape\":[";
      for (std::size_t i = 0; i < kv.second.shape.size(); ++i)
         header += (i ? "," : "") + std::to_string(kv.second.shape[i]);
      header += "],\"data_offsets\":[" + std::to_string(offset) + "," + std::to_string(offset + nbytes) + "]}";
      offset += nbytes;
      first = false;
   }
   header += "}";
   std::ofstream f(filename, std::ios::binary);
   if (!f.is_open())
      throw std::runtime_error("tmva-sofie failed to open file " + filename + " for tensor weight data");
   char size8[8];
   for (int i = 0; i < 8; ++i)
      size8[i] = static_cast<char>((static_cast<std::uint64_t>(header.size()) >> (8 * i)) & 0xff);
   f.write(size8, 8);
   f.write(header.data(), header.size());
   for (auto &kv : fInitializedTensors) {
      if (kv.second.constant)
         continue;
      f.write(static_cast<const char *>(kv.second.data.get()), ConvertShapeToLength(kv.second.shape) * GetTypeSize(kv.second.type));
   }
   if (f.fail())
      throw std::runtime_error("sofie failed to write safetensors payload");
}

} // namespace SOFIE_HIP
