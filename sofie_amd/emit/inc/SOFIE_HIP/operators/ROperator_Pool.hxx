// GlobalAveragePool (core/inc/SOFIE/operators/ROperator_Pool.hxx:225-237: AveragePool with kernel = image).
#ifndef SOFIE_HIP_ROPERATOR_POOL
#define SOFIE_HIP_ROPERATOR_POOL

#include "SOFIE_HIP/operators/ROperator_Gemm.hxx"

namespace SOFIE_HIP {

enum PoolOpMode { InvalidPoolOp, MaxPool, AveragePool, GlobalAveragePool };

template <typename T>
class ROperator_Pool final : public ROperator {
public:
   ROperator_Pool(PoolOpMode mode, std::string nameX, std::string nameY) : fMode(mode), fNX(UTILITY::Clean_name(nameX)), fNY(UTILITY::Clean_name(nameY))
   {
      if (mode != GlobalAveragePool)
         throw std::runtime_error("SOFIE Pool Op: this backend emits GlobalAveragePool only");
      fInputTensorNames = {fNX};
      fOutputTensorNames = {fNY};
      fKind = OperatorKind::POOL;
   }
   void Initialize(RModel &model) override
   {
      if (!model.CheckIfTensorAlreadyExist(fNX))
         throw std::runtime_error("SOFIE Pool op Input Tensor " + fNX + " is not found in model");
      fShapeX = model.GetTensorShape(fNX);
      if (fShapeX.size() < 3)
         throw std::runtime_error("SOFIE Pool Op input data tensor" + fNX + " has fewer than 3 dimensions");
      fType = model.GetTensorType(fNX);
      if (fType != ETensorType::FLOAT)
         throw std::runtime_error("SOFIE Pool Op: input tensor " + fNX + " is not float");
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
      out << "\n" << SP << "//----  operator GlobalAveragePool " << opName << "\n";
      out << SP << "detail::Check(sofie_hip_global_avg_pool_f32(fCtx, tensor_" << fNY << ", tensor_" << fNX << ", " << BatchScaledInt(fDynamic, fShapeX[0] * fShapeX[1])
          << ", " << hw << "), \"" << opName << " GlobalAveragePool\");\n";
      return out.str();
   }

private:
   PoolOpMode fMode;
   std::string fNX, fNY;
   std::vector<std::size_t> fShapeX;
   ETensorType fType = ETensorType::FLOAT;
   bool fDynamic = false;
};

} // namespace SOFIE_HIP
#endif
