// sofie_hip_emit <model.onnx> <out_dir> [--safetensors] [--strided-input] [--name N] [--batch B]: parses a model and writes <out_dir>/<Model>_GPU_HIP.hxx + .dat (or .safetensors)
// (the flow of the reference's emitter template, tests/templates/EmitFromONNX.cxx.in:21-31).
#include "SOFIE_HIP/RModelParser_ONNX.hxx"

#include <iostream>

int main(int argc, char **argv)
{
   if (argc < 3) {
      std::cerr << "usage: " << argv[0] << " <model.onnx> <out_dir> [--plan] [--safetensors] [--strided-input] [--name <ModelName>] [--batch <B>]\n";
      return 2;
   }
   try {
      SOFIE_HIP::RModelParser_ONNX parser;
      bool plan = false, safetensors = false, stridedInput = false;
      std::string name;
      int batch = -1; // a named leading input dimension stays a run-time parameter unless a value is given here
      for (int i = 3; i < argc; ++i) {
         const std::string a = argv[i];
         if (a == "--plan")
            plan = true;
         else if (a == "--safetensors")
            safetensors = true;
         else if (a == "--strided-input")
            stridedInput = true; // Options::kStridedInput: the Session's constructor takes the strides of the inputs
         else if (a == "--name" && i + 1 < argc)
            name = argv[++i];
         else if (a == "--batch" && i + 1 < argc)
            batch = std::stoi(argv[++i]);
         else
            throw std::runtime_error("unknown argument " + a);
      }
      auto model = parser.Parse(argv[1], false, name);
      auto options = static_cast<std::underlying_type_t<SOFIE_HIP::Options>>(safetensors ? SOFIE_HIP::Options::kSafetensorsWeightFile : SOFIE_HIP::Options::kDefault);
      if (stridedInput)
         options |= static_cast<std::underlying_type_t<SOFIE_HIP::Options>>(SOFIE_HIP::Options::kStridedInput);
      model->GenerateGPU_HIP(options, batch);
      model->OutputGenerated(std::string(argv[2]) + "/" + model->GetName() + "_GPU_HIP.hxx");
      if (plan) {
         std::cout << "arena " << model->GetArenaBytes() << " pool " << model->GetIntermediateMemoryPoolSize() << "\n";
         if (model->HasDynamicBatch())
            std::cout << "static " << model->GetStaticBytes() << " per_batch_entry " << model->GetBytesPerBatchEntry() << " parameter "
                      << model->GetBatchParamName() << "\n";
         for (auto &p : model->GetMemoryPlan())
            std::cout << p.name << " " << p.offset << " " << p.bytes << " " << p.begin << " " << p.end << " " << (p.view ? 2 : p.pooled ? 1 : 0)
                      << (model->HasDynamicBatch() ? (p.perBatch ? " per_batch_entry" : " static") : "") << "\n";
      }
   } catch (const std::exception &e) {
      std::cerr << "error: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
