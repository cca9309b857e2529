// A small ONNX front end for the operators of this backend's path.  The reference's parser
// (parsers/src/RModelParser_ONNX.cxx) stays the front end of a SOFIE build; this one exists so that the
// backend can be driven from .onnx files on its own (tests, tools).  It reads the protobuf wire format
// directly, like the reference's parsers/src/onnx.hxx, and applies the reference's parse-time rewrites that
// concern the path: MatMul followed by an Add of an initializer becomes a Gemm with bias
// (RModelParser_ONNX.cxx:1198-1202); activations are fused by the generator.
#ifndef SOFIE_HIP_RMODELPARSER_ONNX
#define SOFIE_HIP_RMODELPARSER_ONNX

#include "SOFIE_HIP/RModel.hxx"

namespace SOFIE_HIP {

class RModelParser_ONNX {
public:
   // throws std::runtime_error for an operator outside the path ("... is not yet supported")
   // modelName: name of the generated namespace and files (default: the file's stem)
   std::unique_ptr<RModel> Parse(std::string filename, bool verbose = false, std::string modelName = "");
};

} // namespace SOFIE_HIP
#endif
