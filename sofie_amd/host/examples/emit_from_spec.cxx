// Emit program: builds an RModel through the programmatic API from a small text description and writes
// <name>.hxx + <name>.dat. Plays the role of the reference's test/EmitFromONNX.cxx.in (parse -> Generate ->
// OutputGenerated) without the protobuf front end: the description is produced by a script from a decoded
// ONNX file or from a synthetic network.
//
//   emit_from_spec <spec file> <directory of raw tensor files> <output directory>
//
// Statements (one per line, '-' stands for "absent"):
//   model NAME
//   input NAME TYPE RANK d0 d1 ...                 a dimension that is not a number is a shape parameter (e.g. bs)
//   init NAME TYPE RANK d0 d1 ... FILE           raw little-endian values
//   output NAME                                    once per output tensor, in the order infer() returns them
//   op Gemm ALPHA BETA TRANSA TRANSB A B C Y RELU
//   op Conv AUTOPAD GROUP nk k.. np p.. ns s.. nd d.. X W B Y
//   op BatchNormalization EPSILON X SCALE B MEAN VAR Y
//   op ConvTranspose AUTOPAD GROUP nk k.. np p.. ns s.. nd d.. nop op.. nos os.. X W B Y
//   op Einsum EQUATION nx X.. Y                  (the equation without blanks)
//   op Relu X Y
//   op MaxPool|AveragePool|AveragePoolIncludePad nk k.. np p.. ns s.. X Y
//   op GlobalAveragePool X Y
//   op Flatten AXIS X Y
//   op QuantizeLinear X SCALE ZP Y | op DequantizeLinear X SCALE ZP Y
//   op QLinearMatMul A AS AZ B BS BZ YS YZ BIAS Y TRANSB
//   op QLinearConv AUTOPAD GROUP nk k.. np p.. ns s.. X XS XZ W WS WZ YS YZ BIAS Y
//   op GemmFP8 A AS B BS BIAS Y TRANSB
//   generate [noweightfile | binaryweightfile | nosession] [batch N] [param NAME VALUE]... [runtimebatch] [layerpercall] [hostcode]
//                                                  batch N resolves the shape parameters; runtimebatch makes N a capacity
#include <cctype>
#include <fstream>
#include <iostream>
#include <sstream>

#include "SOFIE/OperatorList.hxx"
#include "SOFIE/RModel.hxx"

using namespace SOFIE;

static ETensorType TypeOf(const std::string &s)
{
   if (s == "FLOAT") return ETensorType::FLOAT;
   if (s == "INT8") return ETensorType::INT8;
   if (s == "UINT8") return ETensorType::UINT8;
   if (s == "INT32") return ETensorType::INT32;
   if (s == "INT64") return ETensorType::INT64;
   if (s == "FLOAT8E4M3FN") return ETensorType::FLOAT8E4M3FN;
   throw std::runtime_error("unknown type " + s);
}
static std::string Opt(const std::string &s) { return s == "-" ? "" : s; }
static std::vector<size_t> List(std::istringstream &in)
{
   size_t n;
   in >> n;
   std::vector<size_t> v(n);
   for (auto &x : v) in >> x;
   return v;
}

int main(int argc, char **argv)
{
   if (argc < 4) {
      std::cerr << "usage: emit_from_spec <spec> <tensor dir> <out dir>\n";
      return 2;
   }
   try {
      std::ifstream spec(argv[1]);
      if (!spec) throw std::runtime_error(std::string("cannot open ") + argv[1]);
      const std::string tdir = argv[2], odir = argv[3];
      std::unique_ptr<RModel> model;
      std::string line, name;
      std::vector<std::string> outputs;
      int order = 0;
      while (std::getline(spec, line)) {
         std::istringstream in(line);
         std::string kw;
         if (!(in >> kw) || kw[0] == '#') continue;
         if (kw == "model") {
            in >> name;
            model.reset(new RModel(name + ".onnx", "generated from a model description \n"));
         } else if (kw == "input") {
            std::string n, t;
            size_t rank;
            in >> n >> t >> rank;
            std::vector<Dim> dims;
            bool parametric = false;
            for (size_t i = 0; i < rank; ++i) {
               std::string tok;
               in >> tok;
               if (!tok.empty() && std::isdigit(static_cast<unsigned char>(tok[0]))) dims.push_back(Dim{(size_t)std::stoull(tok)});
               else { dims.push_back(Dim{tok}); parametric = true; }
            }
            if (parametric) model->AddInputTensorInfo(n, TypeOf(t), dims);
            else model->AddInputTensorInfo(n, TypeOf(t), ConvertShapeToInt(dims));
            model->AddInputTensorName(n);
         } else if (kw == "init") {
            std::string n, t, file;
            in >> n >> t;
            std::vector<size_t> shape = List(in);
            in >> file;
            const ETensorType type = TypeOf(t);
            const size_t bytes = ConvertShapeToLength(shape) * GetTypeSize(type);
            std::shared_ptr<void> data(malloc(bytes + 1), free);
            std::ifstream f(tdir + "/" + file, std::ios::binary);
            if (!f.read(static_cast<char *>(data.get()), bytes) && bytes) throw std::runtime_error("cannot read " + file);
            model->AddInitializedTensor(n, type, shape, data);
         } else if (kw == "output") {
            std::string n;
            in >> n;
            outputs.push_back(n);
            model->AddOutputTensorNameList(outputs);   // every "output" statement extends the list
         } else if (kw == "op") {
            std::string op;
            in >> op;
            std::unique_ptr<ROperator> r;
            if (op == "Gemm") {
               float alpha, beta;
               int ta, tb, relu;
               std::string a, b, c, y;
               in >> alpha >> beta >> ta >> tb >> a >> b >> c >> y >> relu;
               auto act = relu ? EActivationType::RELU : EActivationType::UNDEFINED;
               if (c == "-") r.reset(new ROperator_Gemm<float>(alpha, beta, ta, tb, a, b, y, act));
               else r.reset(new ROperator_Gemm<float>(alpha, beta, ta, tb, a, b, c, y, act));
            } else if (op == "Conv") {
               std::string autopad, x, w, b, y;
               size_t group;
               in >> autopad >> group;
               auto k = List(in), p = List(in), s = List(in), d = List(in);
               in >> x >> w >> b >> y;
               if (b == "-") r.reset(new ROperator_Conv<float>(autopad, d, group, k, p, s, x, w, y));
               else r.reset(new ROperator_Conv<float>(autopad, d, group, k, p, s, x, w, b, y));
            } else if (op == "ConvTranspose") {
               std::string autopad, x, w, b, y;
               size_t group;
               in >> autopad >> group;
               auto k = List(in), p = List(in), s = List(in), d = List(in), op_ = List(in), os = List(in);
               in >> x >> w >> b >> y;
               r.reset(new ROperator_ConvTranspose<float>(autopad, d, group, k, op_, os, p, s, x, w, b == "-" ? std::string() : b, y));
            } else if (op == "BatchNormalization") {
               float eps;
               std::string x, sc, b, m, v, y;
               in >> eps >> x >> sc >> b >> m >> v >> y;
               r.reset(new ROperator_BatchNormalization<float>(eps, 0.9f, 0, x, sc, b, m, v, y));
            } else if (op == "Einsum") {
               std::string eq, y;
               size_t nx;
               in >> eq >> nx;
               std::vector<std::string> xs(nx);
               for (auto &x : xs) in >> x;
               in >> y;
               r.reset(new ROperator_Einsum<float>(eq, xs, y));
            } else if (op == "Relu") {
               std::string x, y;
               in >> x >> y;
               r.reset(new ROperator_Relu<float>(x, y));
            } else if (op == "MaxPool" || op == "AveragePool" || op == "AveragePoolIncludePad") {
               RAttributes_Pool attr;
               attr.kernel_shape = List(in);
               attr.pads = List(in);
               attr.strides = List(in);
               attr.count_include_pad = op == "AveragePoolIncludePad";
               std::string x, y;
               in >> x >> y;
               r.reset(new ROperator_Pool<float>(op == "MaxPool" ? MaxPool : AveragePool, attr, x, y));
            } else if (op == "GlobalAveragePool") {
               std::string x, y;
               in >> x >> y;
               r.reset(new ROperator_Pool<float>(GlobalAveragePool, RAttributes_Pool(), x, y));
            } else if (op == "Flatten") {
               int axis;
               std::string x, y;
               in >> axis >> x >> y;
               r.reset(new ROperator_Reshape(Flatten, axis, x, "", y));
            } else if (op == "QuantizeLinear" || op == "DequantizeLinear") {
               std::string x, s, z, y;
               in >> x >> s >> z >> y;
               if (op == "QuantizeLinear") r.reset(new ROperator_QuantizeLinear(x, s, Opt(z), y));
               else r.reset(new ROperator_DequantizeLinear(x, s, Opt(z), y));
            } else if (op == "QLinearMatMul") {
               std::string a, as, az, b, bs, bz, ys, yz, bias, y;
               int tb;
               in >> a >> as >> az >> b >> bs >> bz >> ys >> yz >> bias >> y >> tb;
               r.reset(new ROperator_QLinearMatMul(a, as, Opt(az), b, bs, Opt(bz), Opt(ys), Opt(yz), y, Opt(bias), tb));
            } else if (op == "QLinearConv") {
               std::string autopad;
               size_t group;
               in >> autopad >> group;
               auto k = List(in), p = List(in), s = List(in);
               std::string x, xs, xz, w, ws, wz, ys, yz, bias, y;
               in >> x >> xs >> xz >> w >> ws >> wz >> ys >> yz >> bias >> y;
               r.reset(new ROperator_QLinearConv(autopad, {}, group, k, p, s, x, xs, Opt(xz), w, ws, Opt(wz), ys, Opt(yz), Opt(bias), y));
            } else if (op == "GemmFP8") {
               std::string a, as, b, bs, bias, y;
               int tb;
               in >> a >> as >> b >> bs >> bias >> y >> tb;
               r.reset(new ROperator_GemmFP8(a, as, b, bs, Opt(bias), y, tb));
            } else {
               throw std::runtime_error("unknown operator " + op);
            }
            if (!in) throw std::runtime_error("malformed statement: " + line);
            model->AddOperator(std::move(r), order++);
         } else if (kw == "generate") {
            std::underlying_type_t<Options> options = static_cast<std::underlying_type_t<Options>>(Options::kDefault);
            int batch = -1;
            std::map<std::string, size_t> params;
            for (std::string flag; in >> flag;) {
               if (flag == "noweightfile") options = options | Options::kNoWeightFile;
               else if (flag == "binaryweightfile") options = options | Options::kBinaryWeightFile;
               else if (flag == "nosession") options = options | Options::kNoSession;
               else if (flag == "runtimebatch") options = options | Options::kRuntimeBatch;
               else if (flag == "layerpercall") options = options | Options::kLayerPerCall;
               else if (flag == "hostcode") options = options | Options::kHostCode;
               else if (flag == "batch") in >> batch;
               else if (flag == "param") {
                  std::string pname;
                  size_t value = 0;
                  in >> pname >> value;
                  params[pname] = value;
               }
               else throw std::runtime_error("unknown generate flag " + flag);
            }
            // several shape parameters: the values by name, as RModel::Initialize(const std::map<...> &) takes them
            // (the batch number still answers for "bs", "batch_size" and "input_size")
            if (!params.empty()) {
               if (batch > 0)
                  for (const char *n : {"input_size", "batch_size", "bs"})
                     if (!params.count(n)) params[n] = (size_t)batch;
               model->Initialize(params);
            }
            model->Generate(options, batch);
            model->OutputGenerated(odir + "/" + name + ".hxx");
            std::cout << "generated " << odir << "/" << name << ".hxx, intermediate pool " << model->GetIntermediateMemorySize()
                      << " bytes\n";
         } else {
            throw std::runtime_error("unknown statement: " + line);
         }
      }
   } catch (const std::exception &e) {
      std::cerr << "emit_from_spec: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
