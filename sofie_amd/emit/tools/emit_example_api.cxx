// Builds a model through the RModel API, without any ONNX file (the way the reference's
// tests/models/ExternalStreamModelGenerator.cxx does): Y = Relu(X[1,3] * W[3,1] + B), W = 1, B = 0.5,
// so that ones -> 3.5.  Usage: sofie_hip_emit_example <out_dir>
#include "SOFIE_HIP/operators/OperatorList.hxx"

#include <iostream>

int main(int argc, char **argv)
{
   if (argc < 2) {
      std::cerr << "usage: " << argv[0] << " <out_dir>\n";
      return 2;
   }
   using namespace SOFIE_HIP;
   try {
      RModel model("ApiGemmRelu");
      model.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<std::size_t>{1, 3});
      model.AddInputTensorName("X");
      const float w[3] = {1.f, 1.f, 1.f}, b[1] = {0.5f};
      model.AddInitializedTensor("W", ETensorType::FLOAT, {3, 1}, w);
      model.AddInitializedTensor("B", ETensorType::FLOAT, {1}, b);
      model.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.f, 1.f, 0, 0, "X", "W", "B", "G"));
      model.AddOperator(std::make_unique<ROperator_Relu<float>>("G", "Y"));
      model.AddOutputTensorNameList({"Y"});
      model.GenerateGPU_HIP(Options::kExternalStream);
      model.OutputGenerated(std::string(argv[1]) + "/ApiGemmRelu_GPU_HIP.hxx");
   } catch (const std::exception &e) {
      std::cerr << "error: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
