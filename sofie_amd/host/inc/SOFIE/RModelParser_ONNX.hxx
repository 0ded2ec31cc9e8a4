// ONNX front end with the interface of the reference's RModelParser_ONNX
// (src/SOFIE_parsers/inc/SOFIE/RModelParser_ONNX.hxx:28-98): Parse(filename) returns an RModel filled with
// inputs, initializers, operators and outputs; CheckModel(filename) reports unsupported operators.
// The reference links protobuf and the generated onnx classes; this reader decodes the protobuf wire format
// of the few messages it needs itself (ModelProto.graph = 7; GraphProto node/initializer/input/output =
// 1/5/11/12; NodeProto input/output/name/op_type/attribute = 1..5; AttributeProto name/f/i/s/t/floats/ints =
// 1,2,3,4,5,7,8; TensorProto dims/data_type/float_data/int32_data/int64_data/name/raw_data = 1,2,4,5,7,8,9).
// Operators: Gemm, MatMul (+Add), Conv, Relu, MaxPool, Flatten, Reshape, QuantizeLinear, DequantizeLinear,
// QLinearMatMul, QLinearConv, with the reference's fusion rules Gemm->Relu and MatMul->Add
// (src/SOFIE_parsers/src/RModelParser_ONNX.cxx:279-341). Unlike the reference (:560-591) int8 / uint8 / int32
// initializers are accepted.
#ifndef SOFIE_RMODELPARSER_ONNX
#define SOFIE_RMODELPARSER_ONNX

#include <map>
#include <string>
#include <vector>

#include "SOFIE/RModel.hxx"

namespace SOFIE {

class RModelParser_ONNX {
public:
   RModelParser_ONNX() noexcept {}
   // Parse the file and return the model; the model name is the file name without directory and extension.
   RModel Parse(std::string filename, bool verbose = false);
   // true if every operator of the graph can be parsed; prints the missing ones otherwise
   bool CheckModel(std::string filename, bool verbose = false);
   bool IsRegisteredOperator(const std::string &name);
   std::vector<std::string> GetRegisteredOperators();
};

}   // namespace SOFIE
#endif
