// Builds a model through the RModel API, without any ONNX file (the way the reference's
// tests/models/ExternalStreamModelGenerator.cxx does): Y = Relu(X[1,3] * W[3,1] + B), W = 1, B = 0.5,
// so that ones -> 3.5.  Usage: sofie_hip_emit_example <out_dir>
#include "SOFIE_HIP/operators/OperatorList.hxx"

#include <cstdint>
#include <iostream>
#include <vector>

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
      // the chain of the reference's tests/models/CustomMemoryModelGenerator.cxx, with caller-owned device memory:
      // X[3,5] -> Gemm(W = 0.5, B = 1) -> Relu -> Sigmoid -> Tanh; ones -> tanh(sigmoid(3.5))
      for (int withStream = 0; withStream < 2; ++withStream) {
         RModel cm(withStream ? "CustomMemoryStreamChain" : "CustomMemoryChain");
         cm.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<std::size_t>{3, 5});
         cm.AddInputTensorName("X");
         std::vector<float> W(5 * 4, 0.5f), B(4, 1.0f);
         cm.AddInitializedTensor("W", ETensorType::FLOAT, {5, 4}, W.data());
         cm.AddInitializedTensor("B", ETensorType::FLOAT, {4}, B.data());
         cm.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 1.0f, 0, 0, "X", "W", "B", "H1"));
         cm.AddOperator(std::make_unique<ROperator_Relu<float>>("H1", "H2"));
         cm.AddOperator(std::make_unique<ROperator_Sigmoid<float>>("H2", "H3"));
         cm.AddOperator(std::make_unique<ROperator_Tanh<float>>("H3", "Y"));
         cm.AddOutputTensorNameList({"Y"});
         if (withStream)
            cm.GenerateGPU_HIP(Options::kCustomMemory | Options::kExternalStream);
         else
            cm.GenerateGPU_HIP(Options::kCustomMemory);
         cm.OutputGenerated(std::string(argv[1]) + "/" + cm.GetName() + "_GPU_HIP.hxx");
      }
      // the same chain with every Session option at once: the batch a run-time parameter (default 2), caller-owned memory,
      // caller-owned stream, weights in a safetensors file
      {
         RModel all("CustomMemoryDynamicChain");
         all.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<Dim>{Dim(std::string("N"), 2), Dim(5)});
         all.AddInputTensorName("X");
         std::vector<float> W(5 * 4, 0.5f), B(4, 1.0f);
         all.AddInitializedTensor("W", ETensorType::FLOAT, {5, 4}, W.data());
         all.AddInitializedTensor("B", ETensorType::FLOAT, {4}, B.data());
         all.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 1.0f, 0, 0, "X", "W", "B", "H1"));
         all.AddOperator(std::make_unique<ROperator_Relu<float>>("H1", "H2"));
         all.AddOperator(std::make_unique<ROperator_Sigmoid<float>>("H2", "H3"));
         all.AddOperator(std::make_unique<ROperator_Tanh<float>>("H3", "Y"));
         all.AddOutputTensorNameList({"Y"});
         all.GenerateGPU_HIP((Options::kCustomMemory | Options::kExternalStream) | static_cast<std::underlying_type_t<Options>>(Options::kSafetensorsWeightFile));
         all.OutputGenerated(std::string(argv[1]) + "/" + all.GetName() + "_GPU_HIP.hxx");
      }
      // FP8 Gemm with bias and GELU: X[48,256] fp32, W e4m3 [96,256] (K contiguous), codes from a linear congruential
      // sequence so that a test can rebuild them, bias[n] = 0.25 (n mod 7 - 3)
      RModel f8("ApiFp8Gemm");
      f8.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<std::size_t>{48, 256});
      f8.AddInputTensorName("X");
      std::vector<uint8_t> w8(96 * 256);
      uint32_t s = 2024;
      for (auto &v : w8) {
         s = s * 1664525u + 1013904223u;
         v = (uint8_t)((s >> 24) & 0xbe); // exponent at most 7 (|w| < 32), never the NaN code
      }
      std::vector<float> bias(96);
      for (std::size_t n = 0; n < bias.size(); ++n)
         bias[n] = 0.25f * ((int)(n % 7) - 3);
      f8.AddInitializedTensor("W", ETensorType::FLOAT8E4M3FN, {96, 256}, w8.data());
      f8.AddInitializedTensor("B", ETensorType::FLOAT, {96}, bias.data());
      f8.AddOperator(std::make_unique<ROperator_Fp8Gemm>(0.03125f, 0.0078125f, 1, "X", "W", "B", EActivationType::GELU, ETensorType::FLOAT, "Y"));
      f8.AddOutputTensorNameList({"Y"});
      f8.GenerateGPU_HIP();
      f8.OutputGenerated(std::string(argv[1]) + "/ApiFp8Gemm_GPU_HIP.hxx");
      // the same product with the batch left to the Session (maximum given to the constructor, default 48)
      RModel f8d("ApiDynamicFp8Gemm");
      f8d.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<Dim>{Dim(std::string("batch"), 48), Dim(256)});
      f8d.AddInputTensorName("X");
      f8d.AddInitializedTensor("W", ETensorType::FLOAT8E4M3FN, {96, 256}, w8.data());
      f8d.AddInitializedTensor("B", ETensorType::FLOAT, {96}, bias.data());
      f8d.AddOperator(std::make_unique<ROperator_Fp8Gemm>(0.03125f, 0.0078125f, 1, "X", "W", "B", EActivationType::GELU, ETensorType::FLOAT, "Y"));
      f8d.AddOutputTensorNameList({"Y"});
      f8d.GenerateGPU_HIP();
      f8d.OutputGenerated(std::string(argv[1]) + "/ApiDynamicFp8Gemm_GPU_HIP.hxx");
      // Gemm operands that are graph inputs read through strides given to the Session (Options::kStridedInput): the four
      // models of the reference's tests/models/StridedInputModelGenerator.cxx:104-129, 738-745, with its weights
      // (tests/common/strided_input_test_utils.h:43-49: v[i] = scale * ((7 i) mod 11) - 0.5)
      auto gemmValues = [](std::size_t n, float scale) {
         std::vector<float> v(n);
         for (std::size_t i = 0; i < n; i++)
            v[i] = scale * float((i * 7) % 11) - 0.5f;
         return v;
      };
      {
         RModel m("StridedGemmBiasRelu"); // Y = Relu(X[3,5] * W[5,4] + B)
         m.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<std::size_t>{3, 5});
         m.AddInputTensorName("X");
         auto W = gemmValues(5 * 4, 0.1f), B = gemmValues(4, 0.3f);
         m.AddInitializedTensor("W", ETensorType::FLOAT, {5, 4}, W.data());
         m.AddInitializedTensor("B", ETensorType::FLOAT, {4}, B.data());
         m.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 1.0f, 0, 0, "X", "W", "B", "H"));
         m.AddOperator(std::make_unique<ROperator_Relu<float>>("H", "Y"));
         m.AddOutputTensorNameList({"Y"});
         m.GenerateGPU_HIP(Options::kStridedInput);
         m.OutputGenerated(std::string(argv[1]) + "/" + m.GetName() + "_GPU_HIP.hxx");
      }
      {
         RModel m("StridedGemmTransAB"); // Y = X^T * W^T, X stored [5,3], W stored [4,5]
         m.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<std::size_t>{5, 3});
         m.AddInputTensorName("X");
         auto W = gemmValues(4 * 5, 0.1f);
         m.AddInitializedTensor("W", ETensorType::FLOAT, {4, 5}, W.data());
         m.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 0.0f, 1, 1, "X", "W", "Y"));
         m.AddOutputTensorNameList({"Y"});
         m.GenerateGPU_HIP(Options::kStridedInput);
         m.OutputGenerated(std::string(argv[1]) + "/" + m.GetName() + "_GPU_HIP.hxx");
      }
      for (int t = 0; t < 2; ++t) {
         RModel m(t ? "StridedGemmABt" : "StridedGemmAB"); // both operands graph inputs; t: Y = A^T * B^T
         m.AddInputTensorInfo("A", ETensorType::FLOAT, t ? std::vector<std::size_t>{5, 3} : std::vector<std::size_t>{3, 5});
         m.AddInputTensorInfo("B", ETensorType::FLOAT, t ? std::vector<std::size_t>{4, 5} : std::vector<std::size_t>{5, 4});
         m.AddInputTensorName("A");
         m.AddInputTensorName("B");
         m.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 0.0f, t, t, "A", "B", "Y"));
         m.AddOutputTensorNameList({"Y"});
         m.GenerateGPU_HIP(Options::kStridedInput | Options::kNoWeightFile);
         m.OutputGenerated(std::string(argv[1]) + "/" + m.GetName() + "_GPU_HIP.hxx");
      }
      {
         // the batch a run-time parameter (maximum given to the constructor, default 8): rows of a larger matrix
         RModel m("StridedGemmDynamic"); // Y[N,4] = X[N,5] * W[5,4] + B
         m.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<Dim>{Dim(std::string("N"), 8), Dim(5)});
         m.AddInputTensorName("X");
         auto W = gemmValues(5 * 4, 0.1f), B = gemmValues(4, 0.3f);
         m.AddInitializedTensor("W", ETensorType::FLOAT, {5, 4}, W.data());
         m.AddInitializedTensor("B", ETensorType::FLOAT, {4}, B.data());
         m.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 1.0f, 0, 0, "X", "W", "B", "Y"));
         m.AddOutputTensorNameList({"Y"});
         m.GenerateGPU_HIP(Options::kStridedInput);
         m.OutputGenerated(std::string(argv[1]) + "/" + m.GetName() + "_GPU_HIP.hxx");
      }
      {
         // strided input together with every other Session option: run-time batch, caller-owned memory and stream,
         // weights in a safetensors file (the constructor that reads the file hands the strides on to the one that takes the payload)
         RModel m("StridedGemmAllOptions"); // Y[N,4] = X[N,5] * W[5,4] + B
         m.AddInputTensorInfo("X", ETensorType::FLOAT, std::vector<Dim>{Dim(std::string("N"), 8), Dim(5)});
         m.AddInputTensorName("X");
         auto W = gemmValues(5 * 4, 0.1f), B = gemmValues(4, 0.3f);
         m.AddInitializedTensor("W", ETensorType::FLOAT, {5, 4}, W.data());
         m.AddInitializedTensor("B", ETensorType::FLOAT, {4}, B.data());
         m.AddOperator(std::make_unique<ROperator_Gemm<float>>(1.0f, 1.0f, 0, 0, "X", "W", "B", "Y"));
         m.AddOutputTensorNameList({"Y"});
         m.GenerateGPU_HIP((Options::kCustomMemory | Options::kExternalStream) | static_cast<std::underlying_type_t<Options>>(Options::kSafetensorsWeightFile) |
                           static_cast<std::underlying_type_t<Options>>(Options::kStridedInput));
         m.OutputGenerated(std::string(argv[1]) + "/" + m.GetName() + "_GPU_HIP.hxx");
      }
   } catch (const std::exception &e) {
      std::cerr << "error: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
