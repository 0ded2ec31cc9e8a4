// ONNX wire-format reader and graph -> RModel translation (interface: RModelParser_ONNX.hxx).
#include "SOFIE/RModelParser_ONNX.hxx"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <fstream>
#include <iostream>
#include <map>
#include <set>
#include <sstream>
#include <stdexcept>

#include "SOFIE/OperatorList.hxx"

namespace SOFIE {
namespace {

// --------------------------------------------------------------------------- protobuf wire format
struct Span {
   const unsigned char *p = nullptr;
   size_t n = 0;
};

struct Field {
   int num = 0, wire = 0;
   uint64_t value = 0;   // wire types 0, 1, 5
   Span bytes;           // wire type 2
};

class Reader {
   const unsigned char *fP, *fEnd;
public:
   explicit Reader(Span s) : fP(s.p), fEnd(s.p + s.n) {}
   bool Done() const { return fP >= fEnd; }
   uint64_t Varint()
   {
      uint64_t r = 0;
      int shift = 0;
      while (true) {
         if (fP >= fEnd || shift > 63) throw std::runtime_error("TMVA::SOFIE - malformed ONNX file (varint)");
         const unsigned char b = *fP++;
         r |= (uint64_t)(b & 0x7f) << shift;
         if (!(b & 0x80)) return r;
         shift += 7;
      }
   }
   Field Next()
   {
      Field f;
      const uint64_t key = Varint();
      f.num = (int)(key >> 3);
      f.wire = (int)(key & 7);
      size_t len = 0;
      switch (f.wire) {
      case 0: f.value = Varint(); return f;
      case 1: len = 8; break;
      case 5: len = 4; break;
      case 2: len = (size_t)Varint(); break;
      default: throw std::runtime_error("TMVA::SOFIE - malformed ONNX file (wire type " + std::to_string(f.wire) + ")");
      }
      if ((size_t)(fEnd - fP) < len) throw std::runtime_error("TMVA::SOFIE - malformed ONNX file (truncated field)");
      if (f.wire == 2) {
         f.bytes = {fP, len};
      } else {
         uint64_t v = 0;
         std::memcpy(&v, fP, len);
         f.value = v;
      }
      fP += len;
      return f;
   }
};

std::string Str(Span s) { return std::string(reinterpret_cast<const char *>(s.p), s.n); }

// repeated integers, packed or not
void Ints(const Field &f, std::vector<int64_t> &out)
{
   if (f.wire == 0) {
      out.push_back((int64_t)f.value);
      return;
   }
   Reader r(f.bytes);
   while (!r.Done()) out.push_back((int64_t)r.Varint());
}

void Floats(const Field &f, std::vector<float> &out)
{
   if (f.wire == 5) {
      float v;
      const uint32_t bits = (uint32_t)f.value;
      std::memcpy(&v, &bits, 4);
      out.push_back(v);
      return;
   }
   for (size_t i = 0; i + 4 <= f.bytes.n; i += 4) {
      float v;
      std::memcpy(&v, f.bytes.p + i, 4);
      out.push_back(v);
   }
}

// --------------------------------------------------------------------------- ONNX messages
struct Tensor {
   std::string name;
   int dataType = 1;
   std::vector<int64_t> dims;
   std::vector<float> floats;
   std::vector<int64_t> i32, i64;
   Span raw;
   bool hasRaw = false;
};

Tensor ParseTensor(Span s)
{
   Tensor t;
   Reader r(s);
   while (!r.Done()) {
      const Field f = r.Next();
      switch (f.num) {
      case 1: Ints(f, t.dims); break;
      case 2: t.dataType = (int)f.value; break;
      case 4: Floats(f, t.floats); break;
      case 5: Ints(f, t.i32); break;
      case 7: Ints(f, t.i64); break;
      case 8: t.name = Str(f.bytes); break;
      case 9: t.raw = f.bytes; t.hasRaw = true; break;
      default: break;
      }
   }
   return t;
}

struct Attribute {
   std::string name, s;
   float f = 0;
   int64_t i = 0;
   std::vector<float> floats;
   std::vector<int64_t> ints;
   bool hasF = false, hasI = false, hasS = false;
};

struct Node {
   std::vector<std::string> inputs, outputs;
   std::string name, opType;
   std::map<std::string, Attribute> attrs;
   int64_t Int(const std::string &k, int64_t def) const
   {
      auto it = attrs.find(k);
      return (it != attrs.end() && it->second.hasI) ? it->second.i : def;
   }
   float Float(const std::string &k, float def) const
   {
      auto it = attrs.find(k);
      return (it != attrs.end() && it->second.hasF) ? it->second.f : def;
   }
   std::string String(const std::string &k, const std::string &def) const
   {
      auto it = attrs.find(k);
      return (it != attrs.end() && it->second.hasS) ? it->second.s : def;
   }
   std::vector<size_t> Sizes(const std::string &k) const
   {
      std::vector<size_t> out;
      auto it = attrs.find(k);
      if (it != attrs.end())
         for (auto v : it->second.ints) out.push_back((size_t)v);
      return out;
   }
};

Node ParseNode(Span s)
{
   Node n;
   Reader r(s);
   while (!r.Done()) {
      const Field f = r.Next();
      switch (f.num) {
      case 1: n.inputs.push_back(Str(f.bytes)); break;
      case 2: n.outputs.push_back(Str(f.bytes)); break;
      case 3: n.name = Str(f.bytes); break;
      case 4: n.opType = Str(f.bytes); break;
      case 5: {
         Attribute a;
         Reader ar(f.bytes);
         while (!ar.Done()) {
            const Field g = ar.Next();
            switch (g.num) {
            case 1: a.name = Str(g.bytes); break;
            case 2: {
               const uint32_t bits = (uint32_t)g.value;
               std::memcpy(&a.f, &bits, 4);
               a.hasF = true;
               break;
            }
            case 3: a.i = (int64_t)g.value; a.hasI = true; break;
            case 4: a.s = Str(g.bytes); a.hasS = true; break;
            case 7: Floats(g, a.floats); break;
            case 8: Ints(g, a.ints); break;
            default: break;
            }
         }
         n.attrs[a.name] = a;
         break;
      }
      default: break;
      }
   }
   return n;
}

struct ValueInfo {
   std::string name;
   int elemType = 0;
   std::vector<Dim> shape;
};

ValueInfo ParseValueInfo(Span s)
{
   ValueInfo v;
   Reader r(s);
   while (!r.Done()) {
      const Field f = r.Next();
      if (f.num == 1) v.name = Str(f.bytes);
      if (f.num != 2) continue;
      Reader type(f.bytes);                      // TypeProto
      while (!type.Done()) {
         const Field t = type.Next();
         if (t.num != 1) continue;               // tensor_type
         Reader tt(t.bytes);
         while (!tt.Done()) {
            const Field u = tt.Next();
            if (u.num == 1) v.elemType = (int)u.value;
            if (u.num != 2) continue;            // TensorShapeProto
            Reader shape(u.bytes);
            while (!shape.Done()) {
               const Field d = shape.Next();
               if (d.num != 1) continue;         // Dimension
               Dim dim;
               Reader dr(d.bytes);
               while (!dr.Done()) {
                  const Field e = dr.Next();
                  if (e.num == 1) dim.dim = (size_t)e.value;
                  if (e.num == 2) {
                     dim.isParam = true;
                     dim.param = Str(e.bytes);
                  }
               }
               v.shape.push_back(dim);
            }
         }
      }
   }
   return v;
}

struct Graph {
   std::vector<Node> nodes;
   std::vector<Tensor> initializers;
   std::vector<ValueInfo> inputs, outputs;
};

Graph LoadGraph(const std::string &filename, std::vector<unsigned char> &storage)
{
   std::ifstream f(filename, std::ios::binary | std::ios::ate);
   if (!f) throw std::runtime_error("TMVA::SOFIE - Failed to open onnx file " + filename);
   storage.resize((size_t)f.tellg());
   f.seekg(0);
   f.read(reinterpret_cast<char *>(storage.data()), (std::streamsize)storage.size());
   Span graph;
   Reader model({storage.data(), storage.size()});
   while (!model.Done()) {
      const Field fld = model.Next();
      if (fld.num == 7 && fld.wire == 2) graph = fld.bytes;
   }
   if (!graph.p) throw std::runtime_error("TMVA::SOFIE - Failed to read onnx file " + filename + ": no graph");
   Graph g;
   Reader r(graph);
   while (!r.Done()) {
      const Field fld = r.Next();
      switch (fld.num) {
      case 1: g.nodes.push_back(ParseNode(fld.bytes)); break;
      case 5: g.initializers.push_back(ParseTensor(fld.bytes)); break;
      case 11: g.inputs.push_back(ParseValueInfo(fld.bytes)); break;
      case 12: g.outputs.push_back(ParseValueInfo(fld.bytes)); break;
      default: break;
      }
   }
   return g;
}

ETensorType TypeOfOnnx(int t, const std::string &what)
{
   switch (t) {
   case 1: return ETensorType::FLOAT;
   case 2: return ETensorType::UINT8;
   case 3: return ETensorType::INT8;
   case 6: return ETensorType::INT32;
   case 7: return ETensorType::INT64;
   case 17: return ETensorType::FLOAT8E4M3FN;
   default:
      throw std::runtime_error("Data type in weight tensor " + what + " not supported!\n");
   }
}

// tensor payload -> contiguous host buffer of its element type
std::shared_ptr<void> TensorData(const Tensor &t, ETensorType type, size_t length)
{
   const size_t esz = GetTypeSize(type);
   std::shared_ptr<void> data(malloc(length * esz + 1), free);
   char *dst = static_cast<char *>(data.get());
   if (t.hasRaw) {
      if (t.raw.n != length * esz) throw std::runtime_error("TMVA::SOFIE - tensor " + t.name + " has raw data of the wrong size");
      std::memcpy(dst, t.raw.p, t.raw.n);
      return data;
   }
   auto need = [&](size_t have) {
      if (have != length) throw std::runtime_error("TMVA::SOFIE - tensor " + t.name + " has the wrong number of elements");
   };
   switch (type) {
   case ETensorType::FLOAT: need(t.floats.size()); std::memcpy(dst, t.floats.data(), length * 4); break;
   case ETensorType::INT64: need(t.i64.size()); std::memcpy(dst, t.i64.data(), length * 8); break;
   case ETensorType::INT32:
      need(t.i32.size());
      for (size_t i = 0; i < length; ++i) reinterpret_cast<int32_t *>(dst)[i] = (int32_t)t.i32[i];
      break;
   default:   // int8 / uint8 / fp8 travel in int32_data
      need(t.i32.size());
      for (size_t i = 0; i < length; ++i) dst[i] = (char)t.i32[i];
      break;
   }
   return data;
}

const std::set<std::string> &Supported()
{
   static const std::set<std::string> ops = {"Gemm", "MatMul", "Add", "BatchNormalization", "Conv", "ConvTranspose", "Einsum", "Relu", "MaxPool", "AveragePool", "GlobalAveragePool", "Flatten", "Reshape",
                                             "QuantizeLinear", "DequantizeLinear", "QLinearMatMul", "QLinearConv"};
   return ops;
}

std::string InputOr(const Node &n, size_t i) { return i < n.inputs.size() ? n.inputs[i] : std::string(); }


// ---- QDQ pattern: DequantizeLinear -> Conv / MatMul / Gemm -> [Add] -> [Relu] -> QuantizeLinear ------------
// A graph exported in the "QDQ" format keeps float operators between DequantizeLinear and QuantizeLinear nodes;
// the integer operator it stands for is QLinearConv / QLinearMatMul on the quantized tensors (the reference's
// parser rejects the int8 initializers such a graph holds, RModelParser_ONNX.cxx:560-591). The weight must be
// an int8 initializer behind its own DequantizeLinear; the bias is an int32 initializer behind a
// DequantizeLinear, or a float initializer that is quantized here with scale x_scale * w_scale[c].
struct QdqPlan {
   bool conv = false;
   std::string xq, xScale, xZp, wq, wScale, wZp, yScale, yZp, bias, yq;
   int64_t transB = 0;
   bool relu = false;
   std::vector<size_t> skip;       // nodes replaced by the fused operator (besides the anchor)
   size_t dqx = 0;                 // the activation's DequantizeLinear (dropped when nothing else reads it)
   std::vector<int32_t> quantizedBias;   // set when the bias was a float initializer
};

const Tensor *FindInit(const Graph &g, const std::string &name)
{
   for (auto &t : g.initializers)
      if (t.name == name) return &t;
   return nullptr;
}

std::vector<float> FloatsOf(const Tensor &t)
{
   size_t length = 1;
   for (auto d : t.dims) length *= (size_t)d;
   std::shared_ptr<void> data = TensorData(t, ETensorType::FLOAT, length);
   const float *p = static_cast<const float *>(data.get());
   return std::vector<float>(p, p + length);
}

bool PlanQdq(const Graph &g, size_t idx, const std::map<std::string, size_t> &producer, std::map<std::string, int> &uses,
             QdqPlan &plan)
{
   const Node &n = g.nodes[idx];
   const bool conv = n.opType == "Conv";
   if (!conv && n.opType != "MatMul" && n.opType != "Gemm") return false;
   if (n.inputs.size() < 2 || n.outputs.empty()) return false;
   if (n.opType == "Gemm" && (n.Float("alpha", 1.0f) != 1.0f || n.Float("beta", 1.0f) != 1.0f || n.Int("transA", 0) != 0))
      return false;
   auto dq_of = [&](const std::string &tensor) -> const Node * {
      auto it = producer.find(tensor);
      if (it == producer.end()) return nullptr;
      const Node &d = g.nodes[it->second];
      return (d.opType == "DequantizeLinear" && d.inputs.size() >= 2) ? &d : nullptr;
   };
   const Node *dx = dq_of(n.inputs[0]);
   const Node *dw = dq_of(n.inputs[1]);
   if (!dx || !dw) return false;
   const Tensor *w = FindInit(g, dw->inputs[0]);
   if (!w || w->dataType != 3 /* INT8 */ || uses[dw->outputs[0]] != 1) return false;
   if (FindInit(g, dx->inputs[0])) return false;               // a constant activation: nothing to gain
   if (!FindInit(g, dx->inputs[1]) || !FindInit(g, dw->inputs[1])) return false;
   {
      // per-channel weight scales must run along the output channels
      size_t nscale = 1;
      for (auto d : FindInit(g, dw->inputs[1])->dims) nscale *= (size_t)d;
      const int64_t want = conv ? 0 : ((n.opType == "Gemm" && n.Int("transB", 0)) ? 0 : 1);
      if (nscale > 1 && dw->Int("axis", 1) != want) return false;
   }
   plan = QdqPlan();
   plan.conv = conv;
   plan.xq = dx->inputs[0];
   plan.xScale = dx->inputs[1];
   plan.xZp = InputOr(*dx, 2);
   plan.wq = dw->inputs[0];
   plan.wScale = dw->inputs[1];
   plan.wZp = InputOr(*dw, 2);
   plan.transB = n.opType == "Gemm" ? n.Int("transB", 0) : 0;
   plan.dqx = producer.at(n.inputs[0]);
   plan.skip.push_back(producer.at(n.inputs[1]));

   // the tail: [Add bias] -> [Relu] -> QuantizeLinear, each the only reader of its input
   std::string biasName = InputOr(n, 2);
   std::string cur = n.outputs[0];
   auto only_reader = [&](const std::string &tensor) -> size_t {
      if (uses[tensor] != 1) return g.nodes.size();
      for (size_t j = idx + 1; j < g.nodes.size(); ++j)
         if (std::find(g.nodes[j].inputs.begin(), g.nodes[j].inputs.end(), tensor) != g.nodes[j].inputs.end()) return j;
      return g.nodes.size();
   };
   size_t j = only_reader(cur);
   if (n.opType == "MatMul" && j < g.nodes.size() && g.nodes[j].opType == "Add" && g.nodes[j].inputs.size() == 2) {
      const Node &add = g.nodes[j];
      biasName = add.inputs[0] == cur ? add.inputs[1] : add.inputs[0];
      plan.skip.push_back(j);
      cur = add.outputs[0];
      j = only_reader(cur);
   }
   if (j < g.nodes.size() && g.nodes[j].opType == "Relu") {
      plan.relu = true;
      plan.skip.push_back(j);
      cur = g.nodes[j].outputs[0];
      j = only_reader(cur);
   }
   if (j >= g.nodes.size() || g.nodes[j].opType != "QuantizeLinear" || g.nodes[j].inputs.size() < 2) return false;
   const Node &q = g.nodes[j];
   if (!FindInit(g, q.inputs[1])) return false;
   plan.skip.push_back(j);
   plan.yScale = q.inputs[1];
   plan.yZp = InputOr(q, 2);
   plan.yq = q.outputs[0];

   if (!biasName.empty()) {
      if (const Node *db = dq_of(biasName)) {
         const Tensor *b = FindInit(g, db->inputs[0]);
         if (!b || b->dataType != 6 /* INT32 */ || uses[db->outputs[0]] != 1) return false;
         plan.bias = db->inputs[0];
         plan.skip.push_back(producer.at(biasName));
      } else if (const Tensor *bf = FindInit(g, biasName)) {
         if (bf->dataType != 1 /* FLOAT */) return false;
         const std::vector<float> b = FloatsOf(*bf);
         const std::vector<float> sx = FloatsOf(*FindInit(g, plan.xScale));
         const std::vector<float> sw = FloatsOf(*FindInit(g, plan.wScale));
         if (sx.size() != 1 || (sw.size() != 1 && sw.size() != b.size())) return false;
         plan.quantizedBias.resize(b.size());
         for (size_t c = 0; c < b.size(); ++c) {
            const float sb = sx[0] * sw[sw.size() == 1 ? 0 : c];
            plan.quantizedBias[c] = (int32_t)std::nearbyint((double)b[c] / (double)sb);
         }
         plan.bias = biasName + "_quantized";
      } else {
         return false;
      }
   }
   return true;
}

}   // namespace

bool RModelParser_ONNX::IsRegisteredOperator(const std::string &name) { return Supported().count(name) != 0; }

std::vector<std::string> RModelParser_ONNX::GetRegisteredOperators()
{
   return std::vector<std::string>(Supported().begin(), Supported().end());
}

bool RModelParser_ONNX::CheckModel(std::string filename, bool verbose)
{
   std::vector<unsigned char> storage;
   const Graph g = LoadGraph(filename, storage);
   std::map<std::string, int> missing;
   for (auto &n : g.nodes)
      if (!IsRegisteredOperator(n.opType)) missing[n.opType]++;
   if (verbose || !missing.empty())
      for (auto &m : missing) std::cout << "Missing operator " << m.first << " (" << m.second << " nodes)\n";
   return missing.empty();
}

RModel RModelParser_ONNX::Parse(std::string filename, bool verbose)
{
   std::vector<unsigned char> storage;
   const Graph g = LoadGraph(filename, storage);

   // model name = file name without directory and extension, as in the reference (RModelParser_ONNX.cxx:395-412)
   std::string name = filename;
   const size_t slash = name.find_last_of("/\\");
   if (slash != std::string::npos) name = name.substr(slash + 1);
   std::time_t ttime = std::time(0);
   std::tm *gmt = std::gmtime(&ttime);
   std::string parsetime(std::asctime(gmt));
   RModel model(name, parsetime);

   std::set<std::string> initNames;
   for (auto &t : g.initializers) initNames.insert(t.name);
   for (auto &in : g.inputs) {
      if (initNames.count(in.name)) continue;
      if (in.shape.empty()) throw std::runtime_error("TMVA::SOFIE - input tensor " + in.name + " has no shape");
      // a dimension given by name (dim_param) or as -1 is a parameter; the -1 form gets the name "<input>_size"
      // (RModelParser_ONNX.cxx:492-513). RModel::Initialize replaces parameters by the batch size it is given.
      bool dynamic = false;
      std::vector<size_t> shape;
      std::vector<Dim> dims = in.shape;
      for (auto &d : dims) {
         if (!d.isParam && (int64_t)d.dim < 0) {
            d.isParam = true;
            d.param = UTILITY::Clean_name(in.name) + "_size";
         }
         if (d.isParam) dynamic = true;
         shape.push_back(d.dim);
      }
      const ETensorType type = TypeOfOnnx(in.elemType, in.name);
      if (dynamic) model.AddInputTensorInfo(in.name, type, dims);
      else model.AddInputTensorInfo(in.name, type, shape);
      model.AddInputTensorName(in.name);
      if (verbose) std::cout << "input tensor " << in.name << " " << ConvertShapeToString(shape) << "\n";
   }
   // consumers of every tensor, for the single-consumer condition of the fusions
   std::map<std::string, int> uses;
   for (auto &n : g.nodes)
      for (auto &i : n.inputs) uses[i]++;
   for (auto &o : g.outputs) uses[o.name]++;

   std::vector<bool> fused(g.nodes.size(), false);

   // QDQ groups: the anchor (Conv / MatMul / Gemm) becomes the integer operator, the nodes around it vanish
   std::map<std::string, size_t> producer;
   for (size_t i = 0; i < g.nodes.size(); ++i)
      for (auto &o : g.nodes[i].outputs) producer[o] = i;
   std::map<size_t, QdqPlan> plans;
   {
      std::map<size_t, int> dqxReaders;
      for (size_t i = 0; i < g.nodes.size(); ++i) {
         QdqPlan plan;
         if (!PlanQdq(g, i, producer, uses, plan)) continue;
         bool clash = false;
         for (size_t k : plan.skip) clash = clash || fused[k] || plans.count(k);
         if (clash) continue;
         for (size_t k : plan.skip) fused[k] = true;
         dqxReaders[plan.dqx]++;
         plans[i] = plan;
      }
      for (auto &d : dqxReaders)
         if (uses[g.nodes[d.first].outputs[0]] == d.second) fused[d.first] = true;
   }
   // initializers: those some remaining node or fused operator still names
   {
      std::set<std::string> named;
      for (size_t i = 0; i < g.nodes.size(); ++i) {
         if (fused[i]) continue;
         auto it = plans.find(i);
         if (it == plans.end()) {
            for (auto &in : g.nodes[i].inputs) named.insert(in);
         } else {
            const QdqPlan &q = it->second;
            for (auto &nm : {q.xScale, q.xZp, q.wq, q.wScale, q.wZp, q.yScale, q.yZp, q.bias}) named.insert(nm);
         }
      }
      for (auto &o : g.outputs) named.insert(o.name);
      for (auto &t : g.initializers) {
         if (!plans.empty() && !named.count(t.name)) continue;
         const ETensorType type = TypeOfOnnx(t.dataType, t.name);
         std::vector<size_t> shape;
         for (auto d : t.dims) shape.push_back((size_t)d);
         const size_t length = ConvertShapeToLength(shape);
         model.AddInitializedTensor(t.name, type, shape, TensorData(t, type, length));
      }
   }
   int order = 0;
   for (size_t idx = 0; idx < g.nodes.size(); ++idx) {
      if (fused[idx]) continue;
      const Node &n = g.nodes[idx];
      if (verbose) std::cout << "\t" << idx << " " << n.opType << "\n";
      if (n.outputs.empty()) throw std::runtime_error("TMVA::SOFIE - node " + n.name + " has no output");
      const Node *next = idx + 1 < g.nodes.size() ? &g.nodes[idx + 1] : nullptr;
      const bool nextReadsOnlyThis = next && !next->inputs.empty() && uses[n.outputs[0]] == 1 &&
                                     std::find(next->inputs.begin(), next->inputs.end(), n.outputs[0]) != next->inputs.end();
      std::unique_ptr<ROperator> op;
      const std::string &t = n.opType;
      auto planned = plans.find(idx);
      if (planned != plans.end()) {
         const QdqPlan &q = planned->second;
         if (!q.quantizedBias.empty()) {
            std::shared_ptr<void> data(malloc(q.quantizedBias.size() * sizeof(int32_t)), free);
            std::memcpy(data.get(), q.quantizedBias.data(), q.quantizedBias.size() * sizeof(int32_t));
            model.AddInitializedTensor(q.bias, ETensorType::INT32, {q.quantizedBias.size()}, data);
         }
         if (q.conv)
            op.reset(new ROperator_QLinearConv(n.String("auto_pad", "NOTSET"), n.Sizes("dilations"), (size_t)n.Int("group", 1),
                                               n.Sizes("kernel_shape"), n.Sizes("pads"), n.Sizes("strides"), q.xq, q.xScale,
                                               q.xZp, q.wq, q.wScale, q.wZp, q.yScale, q.yZp, q.bias, q.yq));
         else
            op.reset(new ROperator_QLinearMatMul(q.xq, q.xScale, q.xZp, q.wq, q.wScale, q.wZp, q.yScale, q.yZp, q.yq, q.bias,
                                                 q.transB));
         if (q.relu && !op->FuseActivation(EActivationType::RELU))
            throw std::runtime_error("TMVA::SOFIE - cannot fuse the Relu of the quantized group at node " + n.name);
         if (verbose) std::cout << "\t\tQDQ group -> " << (q.conv ? "QLinearConv " : "QLinearMatMul ") << q.yq << "\n";
      } else if (t == "Gemm") {
         // Gemm -> Relu with a single consumer: the activation becomes a constructor argument (ParseFuseGemmRelu.cxx)
         std::string out = n.outputs[0];
         EActivationType act = EActivationType::UNDEFINED;
         if (nextReadsOnlyThis && next->opType == "Relu") {
            act = EActivationType::RELU;
            out = next->outputs[0];
            fused[idx + 1] = true;
         }
         const float alpha = n.Float("alpha", 1.0f), beta = n.Float("beta", 1.0f);
         const int_t ta = n.Int("transA", 0), tb = n.Int("transB", 0);
         if (n.inputs.size() == 2) op.reset(new ROperator_Gemm<float>(alpha, beta, ta, tb, n.inputs[0], n.inputs[1], out, act));
         else if (n.inputs.size() == 3)
            op.reset(new ROperator_Gemm<float>(alpha, beta, ta, tb, n.inputs[0], n.inputs[1], n.inputs[2], out, act));
         else throw std::runtime_error("TMVA::SOFIE - Gemm node " + n.name + " needs 2 or 3 inputs");
      } else if (t == "MatMul") {
         // MatMul -> Add(bias) becomes one Gemm with alpha = beta = 1 (ParseFuseMatMulAdd.cxx); alone it is a
         // Gemm with beta = 0 (ParseMatMul.cxx)
         if (n.inputs.size() != 2) throw std::runtime_error("TMVA::SOFIE - MatMul node " + n.name + " needs 2 inputs");
         if (nextReadsOnlyThis && next->opType == "Add" && next->inputs.size() == 2) {
            const std::string bias = next->inputs[0] == n.outputs[0] ? next->inputs[1] : next->inputs[0];
            op.reset(new ROperator_Gemm<float>(1.0f, 1.0f, 0, 0, n.inputs[0], n.inputs[1], bias, next->outputs[0]));
            fused[idx + 1] = true;
         } else {
            op.reset(new ROperator_Gemm<float>(1.0f, 0.0f, 0, 0, n.inputs[0], n.inputs[1], n.outputs[0]));
         }
      } else if (t == "Conv") {
         // group defaults to 0 = inferred from the shapes (ParseConv.cxx:8-72)
         const std::string autopad = n.String("auto_pad", "NOTSET");
         const size_t group = (size_t)n.Int("group", 0);
         if (n.inputs.size() == 2)
            op.reset(new ROperator_Conv<float>(autopad, n.Sizes("dilations"), group, n.Sizes("kernel_shape"), n.Sizes("pads"),
                                               n.Sizes("strides"), n.inputs[0], n.inputs[1], n.outputs[0]));
         else if (n.inputs.size() == 3)
            op.reset(new ROperator_Conv<float>(autopad, n.Sizes("dilations"), group, n.Sizes("kernel_shape"), n.Sizes("pads"),
                                               n.Sizes("strides"), n.inputs[0], n.inputs[1], n.inputs[2], n.outputs[0]));
         else throw std::runtime_error("TMVA::SOFIE - Conv node " + n.name + " needs 2 or 3 inputs");
      } else if (t == "ConvTranspose") {
         // attributes as read by ParseConvTranspose.cxx: group defaults to 0 (= 1 in the operator)
         if (n.inputs.size() != 2 && n.inputs.size() != 3)
            throw std::runtime_error("TMVA::SOFIE - ConvTranspose node " + n.name + " needs 2 or 3 inputs");
         op.reset(new ROperator_ConvTranspose<float>(n.String("auto_pad", "NOTSET"), n.Sizes("dilations"), (size_t)n.Int("group", 0),
                                                     n.Sizes("kernel_shape"), n.Sizes("output_padding"), n.Sizes("output_shape"),
                                                     n.Sizes("pads"), n.Sizes("strides"), n.inputs[0], n.inputs[1], InputOr(n, 2),
                                                     n.outputs[0]));
      } else if (t == "BatchNormalization") {
         // The reference's parser passes epsilon = 1e-5 whatever the node says (ParseBatchNormalization.cxx:20-31);
         // the attribute is honoured here, so files written with the ONNX default give the same numbers.
         if (n.inputs.size() != 5)
            throw std::runtime_error("TMVA::SOFIE - BatchNormalization node " + n.name + " needs 5 inputs");
         op.reset(new ROperator_BatchNormalization<float>(n.Float("epsilon", 1e-05f), n.Float("momentum", 0.9f),
                                                          (size_t)n.Int("training_mode", 0), n.inputs[0], n.inputs[1], n.inputs[2],
                                                          n.inputs[3], n.inputs[4], n.outputs[0]));
      } else if (t == "Einsum") {
         // as the reference's ParseEinsum.cxx:8-46: every operand known, the equation attribute present
         const std::string equation = n.String("equation", "");
         if (equation.empty())
            throw std::runtime_error("TMVA::SOFIE ONNX Parser Einsum op has  no attribute defining the equation");
         op.reset(new ROperator_Einsum<float>(equation, n.inputs, n.outputs[0]));
      } else if (t == "Relu") {
         op.reset(new ROperator_Relu<float>(n.inputs.at(0), n.outputs[0]));
      } else if (t == "GlobalAveragePool") {
         op.reset(new ROperator_Pool<float>(GlobalAveragePool, RAttributes_Pool(), n.inputs.at(0), n.outputs[0]));
      } else if (t == "MaxPool" || t == "AveragePool") {
         RAttributes_Pool attr;
         attr.auto_pad = n.String("auto_pad", "NOTSET");
         attr.ceil_mode = (int)n.Int("ceil_mode", 0);
         attr.count_include_pad = (int)n.Int("count_include_pad", 0);
         attr.storage_order = (int)n.Int("storage_order", 0);
         attr.dilations = n.Sizes("dilations");
         attr.kernel_shape = n.Sizes("kernel_shape");
         attr.pads = n.Sizes("pads");
         attr.strides = n.Sizes("strides");
         op.reset(new ROperator_Pool<float>(t == "MaxPool" ? MaxPool : AveragePool, attr, n.inputs.at(0), n.outputs[0]));
      } else if (t == "Flatten") {
         op.reset(new ROperator_Reshape(Flatten, (int)n.Int("axis", 1), n.inputs.at(0), "", n.outputs[0]));
      } else if (t == "Reshape") {
         op.reset(new ROperator_Reshape(Reshape, (int)n.Int("allowzero", 0), n.inputs.at(0), InputOr(n, 1), n.outputs[0]));
      } else if (t == "QuantizeLinear") {
         op.reset(new ROperator_QuantizeLinear(n.inputs.at(0), n.inputs.at(1), InputOr(n, 2), n.outputs[0]));
      } else if (t == "DequantizeLinear") {
         op.reset(new ROperator_DequantizeLinear(n.inputs.at(0), n.inputs.at(1), InputOr(n, 2), n.outputs[0]));
      } else if (t == "QLinearMatMul") {
         if (n.inputs.size() < 8) throw std::runtime_error("TMVA::SOFIE - QLinearMatMul node " + n.name + " needs 8 inputs");
         op.reset(new ROperator_QLinearMatMul(n.inputs[0], n.inputs[1], n.inputs[2], n.inputs[3], n.inputs[4], n.inputs[5],
                                              n.inputs[6], n.inputs[7], n.outputs[0], InputOr(n, 8), 0));
      } else if (t == "QLinearConv") {
         if (n.inputs.size() < 8) throw std::runtime_error("TMVA::SOFIE - QLinearConv node " + n.name + " needs 8 or 9 inputs");
         op.reset(new ROperator_QLinearConv(n.String("auto_pad", "NOTSET"), n.Sizes("dilations"), (size_t)n.Int("group", 1),
                                            n.Sizes("kernel_shape"), n.Sizes("pads"), n.Sizes("strides"), n.inputs[0],
                                            n.inputs[1], n.inputs[2], n.inputs[3], n.inputs[4], n.inputs[5], n.inputs[6],
                                            n.inputs[7], InputOr(n, 8), n.outputs[0]));
      } else {
         throw std::runtime_error("TMVA::SOFIE Operator type " + t + " is not yet supported");
      }
      model.AddOperator(std::move(op), order++);
   }
   std::vector<std::string> outputs;
   for (auto &o : g.outputs) outputs.push_back(o.name);
   model.AddOutputTensorNameList(outputs);
   return model;
}

}   // namespace SOFIE
