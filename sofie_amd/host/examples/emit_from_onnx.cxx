// ONNX file -> generated Session header and weight file, the flow of the reference's own tests
// (src/SOFIE_core/test/EmitFromONNX.cxx.in: Parse, Generate, OutputGenerated).
//   emit_from_onnx <model.onnx> <output directory> [--check | --batch N [--runtime]] [--host]
// --batch N gives a parametric batch dimension of the inputs ("bs", "batch_size", a -1) the value N, the way the
// reference's users pass a batch size to RModel::Generate; with --runtime N is a capacity and the Session also
// takes infer(n, ...) for any n up to it (Options::kRuntimeBatch). --host (last argument) emits the Session for the
// host cores (Options::kHostCode: BLAS calls and loops, as the reference generates it).
#include <iostream>

#include "SOFIE/RModelParser_ONNX.hxx"

int main(int argc, char **argv)
{
   if (argc < 3) {
      std::cerr << "usage: emit_from_onnx <model.onnx> <output directory> [--check | --batch N [--runtime]] [--host]\n";
      return 2;
   }
   try {
      SOFIE::RModelParser_ONNX parser;
      if (argc > 3 && std::string(argv[3]) == "--check") return parser.CheckModel(argv[1], true) ? 0 : 1;
      SOFIE::RModel model = parser.Parse(argv[1]);
      int batch = -1;
      if (argc > 4 && std::string(argv[3]) == "--batch") batch = std::stoi(argv[4]);
      auto options = static_cast<std::underlying_type_t<SOFIE::Options>>(SOFIE::Options::kDefault);
      if (argc > 5 && std::string(argv[5]) == "--runtime") options = options | SOFIE::Options::kRuntimeBatch;
      if (std::string(argv[argc - 1]) == "--host") options = options | SOFIE::Options::kHostCode;
      model.Generate(options, batch);
      const std::string out = std::string(argv[2]) + "/" + model.GetName() + ".hxx";
      model.OutputGenerated(out);
      std::cout << "generated " << out << ", intermediate pool " << model.GetIntermediateMemorySize() << " bytes\n";
   } catch (const std::exception &e) {
      std::cerr << "emit_from_onnx: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
