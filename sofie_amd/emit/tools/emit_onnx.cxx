// sofie_hip_emit <model.onnx> <out_dir>: parses a model and writes <out_dir>/<Model>_GPU_HIP.hxx + .dat
// (the flow of the reference's emitter template, tests/templates/EmitFromONNX.cxx.in:21-31).
#include "SOFIE_HIP/RModelParser_ONNX.hxx"

#include <iostream>

int main(int argc, char **argv)
{
   if (argc < 3) {
      std::cerr << "usage: " << argv[0] << " <model.onnx> <out_dir> [--plan]\n";
      return 2;
   }
   try {
      SOFIE_HIP::RModelParser_ONNX parser;
      auto model = parser.Parse(argv[1]);
      model->GenerateGPU_HIP();
      model->OutputGenerated(std::string(argv[2]) + "/" + model->GetName() + "_GPU_HIP.hxx");
      if (argc > 3 && std::string(argv[3]) == "--plan") {
         std::cout << "arena " << model->GetArenaBytes() << " pool " << model->GetIntermediateMemoryPoolSize() << "\n";
         for (auto &p : model->GetMemoryPlan())
            std::cout << p.name << " " << p.offset << " " << p.bytes << " " << p.begin << " " << p.end << " " << (p.pooled ? 1 : 0) << "\n";
      }
   } catch (const std::exception &e) {
      std::cerr << "error: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
